/* Included twice by cpu_ref.c with SCALAR = float / double and FN(name) = name##_f32 / name##_f64.
 * TEST INFRASTRUCTURE ONLY (parity checker and timed CPU baseline), never linked into the product.
 *
 * Restates the reference's CPU path (paths relative to src/gmc/cpp/extensions/):
 *   per-pair forward   util/gaussian.h:82-95   (determinant and sqrt recomputed for every pair)
 *   per-pair backward  util/grad/gaussian.h:19-66, util/grad/glm.h:15-51 (second exp in grad::exp)
 *   loops              evaluate_inversed/parallel_implementation.cu:23-55 (forward), :133-173 (backward)
 *   schedule           parallel_start.h:92-111: one OpenMP thread per threadIdx of a 128-wide block, every
 *                      thread walks all blocks serially => thread t owns the points n = t (mod 128)
 *   atomics            cuda_operations.h:152-164: compare-and-swap loop
 * The stored row-major DxD matrix is read through a column-major type in the reference (util/glm.h:108-128);
 * `MAT(c, col, row)` keeps that reading so that non-symmetric inputs behave the same.
 */

#define MAT(c, col, row) ((c)[(col) * D + (row)])

static inline SCALAR FN(det)(const SCALAR* c, int D) {
    if (D == 2)
        return MAT(c, 0, 0) * MAT(c, 1, 1) - MAT(c, 1, 0) * MAT(c, 0, 1);
    return MAT(c, 0, 0) * (MAT(c, 1, 1) * MAT(c, 2, 2) - MAT(c, 2, 1) * MAT(c, 1, 2))
         - MAT(c, 1, 0) * (MAT(c, 0, 1) * MAT(c, 2, 2) - MAT(c, 2, 1) * MAT(c, 0, 2))
         + MAT(c, 2, 0) * (MAT(c, 0, 1) * MAT(c, 1, 2) - MAT(c, 1, 1) * MAT(c, 0, 2));
}

/* glm (mat * vec): result[row] = sum_col m[col][row] * v[col] */
static inline void FN(matvec)(const SCALAR* c, const SCALAR* v, SCALAR* r, int D) {
    for (int row = 0; row < D; ++row) {
        SCALAR s = 0;
        for (int col = 0; col < D; ++col) s += MAT(c, col, row) * v[col];
        r[row] = s;
    }
}

static inline void FN(atomic_add)(SCALAR* addr, SCALAR val) {
    /* cuda_operations.h:152-164 */
    SCALAR old_v, new_v;
    __atomic_load(addr, &old_v, __ATOMIC_RELAXED);
    do {
        new_v = old_v + val;
    } while (!__atomic_compare_exchange(addr, &old_v, &new_v, 1, __ATOMIC_RELAXED, __ATOMIC_RELAXED));
}

static inline SCALAR FN(eval_pair)(const SCALAR* g, const SCALAR* x, int D) {
    const SCALAR factor = (D == 2) ? (SCALAR)0.15915494309189535 : (SCALAR)0.06349363593424097;
    SCALAR t[3], u[3];
    for (int i = 0; i < D; ++i) t[i] = x[i] - g[1 + i];
    const SCALAR* c = g + 1 + D;
    FN(matvec)(c, t, u, D);
    SCALAR dot = 0;
    for (int i = 0; i < D; ++i) dot += t[i] * u[i];
    const SCALAR v = (SCALAR)(-0.5) * dot;
    const SCALAR norm = SQRT(FN(det)(c, D)) * factor;
    return g[0] * norm * EXP(v);
}

/* mask (may be NULL): boxes [B*L*M][2*D] = lower, upper; a pair contributes iff lower <= x <= upper. */
static inline int FN(inside)(const SCALAR* box, const SCALAR* x, int D) {
    for (int i = 0; i < D; ++i)
        if (x[i] < box[i] || x[i] > box[D + i]) return 0;
    return 1;
}

void FN(cpu_ref_forward)(const SCALAR* mixture, const SCALAR* xes, SCALAR* out, const SCALAR* boxes,
                         int B, int L, int M, int N, int D, int Bx, int Lx, int n_threads) {
    const int G = 1 + D + D * D;
    const int block = 128;
    const int n_blocks_x = (N + block - 1) / block;
    memset(out, 0, sizeof(SCALAR) * (size_t)B * L * N);
#pragma omp parallel for num_threads(n_threads) schedule(static, 1)
    for (int thread_x = 0; thread_x < block; ++thread_x) {
        for (int b = 0; b < B; ++b)
        for (int l = 0; l < L; ++l)
        for (int bx = 0; bx < n_blocks_x; ++bx) {
            const int n = bx * block + thread_x;
            if (n >= N) continue;
            const int xb = b < Bx - 1 ? b : Bx - 1;
            const int xl = l < Lx - 1 ? l : Lx - 1;
            const SCALAR* x = xes + (((size_t)xb * Lx + xl) * N + n) * D;
            SCALAR* o = out + ((size_t)b * L + l) * N + n;
            for (int m = 0; m < M; ++m) {
                const size_t gi = ((size_t)b * L + l) * M + m;
                if (boxes && !FN(inside)(boxes + gi * 2 * D, x, D)) continue;
                *o += FN(eval_pair)(mixture + gi * G, x, D);
            }
        }
    }
}

static inline void FN(grad_pair)(const SCALAR* g, const SCALAR* x, SCALAR incoming, SCALAR* gg, SCALAR* gx, int D) {
    const SCALAR factor = (D == 2) ? (SCALAR)0.15915494309189535 : (SCALAR)0.06349363593424097;
    SCALAR t[3], u[3];
    for (int i = 0; i < D; ++i) t[i] = x[i] - g[1 + i];
    const SCALAR* c = g + 1 + D;
    FN(matvec)(c, t, u, D);
    SCALAR dot = 0;
    for (int i = 0; i < D; ++i) dot += t[i] * u[i];
    const SCALAR v = (SCALAR)(-0.5) * dot;
    const SCALAR det = FN(det)(c, D);
    const SCALAR root = SQRT(det);
    const SCALAR norm = root * factor;
    const SCALAR ex = EXP(v);
    gg[0] = norm * ex * incoming;
    const SCALAR grad_norm = g[0] * ex * incoming;
    const SCALAR grad_exp = g[0] * norm * incoming;
    const SCALAR grad_root = grad_norm * factor;
    const SCALAR grad_det = grad_root / (2 * root);
    const SCALAR grad_v = EXP(v) * grad_exp;            /* util/grad/scalar.h:18-21 recomputes exp */
    const SCALAR gd = grad_v * (SCALAR)(-0.5);
    SCALAR grad_t[3], grad_u[3], ct[3];
    for (int i = 0; i < D; ++i) { grad_t[i] = u[i] * gd; grad_u[i] = t[i] * gd; }
    FN(matvec)(c, grad_u, ct, D);
    for (int i = 0; i < D; ++i) grad_t[i] += ct[i];
    SCALAR* gc = gg + 1 + D;
    /* outerProduct(grad_u, t): glm col j row i = grad_u[i] * t[j]  (util/glm.h:102-105) */
    for (int col = 0; col < D; ++col)
        for (int row = 0; row < D; ++row)
            MAT(gc, col, row) = grad_u[row] * t[col];
    if (D == 2) {
        MAT(gc, 0, 0) += MAT(c, 1, 1) * grad_det;
        MAT(gc, 0, 1) += -MAT(c, 1, 0) * grad_det;
        MAT(gc, 1, 0) += -MAT(c, 0, 1) * grad_det;
        MAT(gc, 1, 1) += MAT(c, 0, 0) * grad_det;
    } else {
        for (int i = 0; i < 3; ++i) {
            const int i1 = i < 1, i2 = 2 - (i >> 1);
            for (int j = 0; j < 3; ++j) {
                const int j1 = j < 1, j2 = 2 - (j >> 1);
                const SCALAR sign = ((i ^ j) % 2 == 0) ? (SCALAR)1 : (SCALAR)-1;
                MAT(gc, i, j) += sign * (MAT(c, i1, j1) * MAT(c, i2, j2) - MAT(c, i1, j2) * MAT(c, i2, j1)) * grad_det;
            }
        }
    }
    for (int i = 0; i < D; ++i) { gx[i] = grad_t[i]; gg[1 + i] = -grad_t[i]; }
}

void FN(cpu_ref_backward)(const SCALAR* grad_out, const SCALAR* mixture, const SCALAR* xes,
                          SCALAR* grad_mixture, SCALAR* grad_xes, const SCALAR* boxes,
                          int B, int L, int M, int N, int D, int Bx, int Lx,
                          int need_grad_mixture, int need_grad_xes, int n_threads) {
    const int G = 1 + D + D * D;
    const int block = 128;
    const int n_blocks_x = (N + block - 1) / block;
    memset(grad_mixture, 0, sizeof(SCALAR) * (size_t)B * L * M * G);
    memset(grad_xes, 0, sizeof(SCALAR) * (size_t)Bx * Lx * N * D);
#pragma omp parallel for num_threads(n_threads) schedule(static, 1)
    for (int thread_x = 0; thread_x < block; ++thread_x) {
        for (int b = 0; b < B; ++b)
        for (int l = 0; l < L; ++l)
        for (int bx = 0; bx < n_blocks_x; ++bx) {
            const int n = bx * block + thread_x;
            if (n >= N) continue;
            const int xb = b < Bx - 1 ? b : Bx - 1;
            const int xl = l < Lx - 1 ? l : Lx - 1;
            const size_t xi = ((size_t)xb * Lx + xl) * N + n;
            const SCALAR* x = xes + xi * D;
            const SCALAR incoming = grad_out[((size_t)b * L + l) * N + n];
            for (int m = 0; m < M; ++m) {
                const size_t gi = ((size_t)b * L + l) * M + m;
                if (boxes && !FN(inside)(boxes + gi * 2 * D, x, D)) continue;
                SCALAR gg[13], gx[3];
                FN(grad_pair)(mixture + gi * G, x, incoming, gg, gx, D);
                if (need_grad_xes)
                    for (int i = 0; i < D; ++i) FN(atomic_add)(grad_xes + xi * D + i, gx[i]);
                if (need_grad_mixture)
                    for (int i = 0; i < G; ++i) FN(atomic_add)(grad_mixture + gi * G + i, gg[i]);
            }
        }
    }
}

#undef MAT
