// LBVH-culled Gaussian-mixture evaluation for gfx950.
//
// Semantics (what the reference's parts define; the composed evaluator is not in the reference snapshot):
//   every Gaussian gets an axis-aligned box from the contribution cutoff (src/gmc/cpp/extensions/lbvh/bvh.cu:164-231);
//   a point receives the contributions of exactly those Gaussians whose own box contains it (closed interval,
//   lbvh/aabb.h:39-47; traversal lbvh/query.h:13-66).  Internal boxes are exact unions of their children
//   (lbvh/bvh.cu:460-510), so the result does not depend on tree shape, Morton resolution or sort order.
//
// Build, one tree per (b,l) mixture, all on device and without host synchronisation:
//   centre bounds -> 30-bit Morton codes of the centres (lbvh/morton_code.h:77-85,145-168) -> stable sort of the codes
//   (segmented LSD radix sort, 8 bits per pass; a single large tree: one launch whose 256 workgroups each gather and
//   sort their share of the keys in LDS) -> leaves in Morton order with their boxes and evaluation records, Karras
//   radix tree over the unique keys (morton << 32 | rank) as lbvh/building.h:11-103 -> boxes of the internal nodes as
//   unions of the leaf boxes of their ranges (order-preserving integers: exactly the unions a bottom-up merge gives,
//   lbvh/bvh.cu:460-510).
// Query points are Morton-sorted the same way (on their top 16 or 8 key bits) so that a wavefront owns 64
// neighbouring points; their two sort passes ride as extra workgroups in the two last launches of the tree
// construction, and one wavefront per tree leaves a cut through the tree a few levels below the root (tree_frontier).
//
// Small trees take short cuts: mixtures of at most 1024 components (query points in segments of at most 8192) are built
// by ONE launch, every tree inside the LDS of a wavefront or a workgroup (bvh_build_small_kernel: same trees bit for
// bit), and mixtures of at most 64 components are evaluated without the tree, all leaves against all points with the
// box test in front (bvh_all_pairs_kernel: same rule, same sums).
//
// Traversal: 64 sorted points form a group with ONE node stack (LDS); lanes work on tree nodes while the tree is
// descended and on points while the gathered leaves are evaluated; a workgroup serves up to four groups, whose
// descents overlap (see bvh_traverse_kernel).  A descent starts from the cut the build has left and tests node boxes
// against one or two boxes around the group's points (two where the group straddles a jump of the Morton curve,
// see group_boxes).  Backward collects the per-Gaussian sums of a batch of leaves in LDS
// and issues one global atomic per non-zero scalar, leaf and wavefront.  The candidate leaves of every group stay
// in the BVH object after the first traversal, so the backward pass after a forward pass does not descend, and
// long lists are cut into pieces that helper workgroups of the backward launch take over (see kPieceLeaves).
#include "gmc_common.h"

namespace gmc {

int check_shape(const gmc_shape* s);

constexpr double kSqFloor = 5.991464547107982;   // -2 ln 0.05 (lbvh/bvh.cu:194)

// ---------------------------------------------------------------------------------------------------------------
// layout of the opaque BVH object
// ---------------------------------------------------------------------------------------------------------------
struct BvhLayout {
    size_t node_box;            // T [BL][2M-1][2D]        lower, upper; internal nodes first, then leaves (Morton order)
    size_t child_box;           // T [BL][M-1][2][2D]      boxes of the left and right child, stored with the parent
    size_t leaf_rec;            // T [BL][M][RS]           evaluation records in leaf order
    size_t children;            // int2 [BL][M-1]          left, right: >= 0 internal node, < 0 leaf ~index
    size_t parent;              // int [BL][2M-1]
    size_t node_range;          // int2 [BL][M-1]          first and last leaf below every internal node
    size_t leaf_comp;           // int [BL][M]             component id of each leaf
    size_t run_box;             // intT [ceil(BL*M/kBoxBlock)*kBoxBlock][2][2D] leaves of all mixtures numbered through, in blocks of
                                //                          kBoxBlock: union of the leaf boxes from the start of the block up to the
                                //                          leaf, and from the leaf to the end of the block (order-preserving integers)
    size_t parts_g, parts_p;    // T [segments][blocks][2D] per-block partial bounds of the centres / the query points
    size_t keys_a, keys_b, vals_a, vals_b;       // uint32 [BL*M]   radix ping-pong of the leaves
    size_t pkeys_a, pkeys_b, pvals_a, pvals_b;   // uint32 [BxLx*N] radix ping-pong of the query points
    size_t hist_g, hist_p;      // uint32 [4 | 2][segments][blocks][256] block histograms of every radix pass (leaves: 4
                                // passes, points: 2), adjacent; all zero when the build starts to count
    size_t hist_words;          // uint32 words from hist_g to the end of hist_p
    size_t p_order;             // int [BxLx][N]           Morton order of the query points
    size_t g_keys;              // uint32 [BL][M]          sorted Morton codes of the leaves
    size_t frontier;            // int [BL][1 + kFrontier] count, then internal nodes that cut the tree a few levels below the root
    size_t cand_count;          // int [BL][ceil(N/64)]    candidate leaves of every point group, -1: not known
    size_t cand_list;           // int [BL][ceil(N/64)][kLeafCap], then a pool of pool_cap ints for the lists of
                                // later rounds (all empty when the lists would exceed kCandCacheBytes)
    size_t cand_stamp;          // uint64 [BL][ceil(N/64)] content stamp of the 64 points a group's list was gathered for
    size_t cand_pieces;         // int2 [BL][ceil(N/64)]   slots of the piece table that hold this group's pieces (first, count)
    size_t cand_ctl;            // int [4]                 pieces published, pool ints handed out, error flags (kErr*), -
    size_t sums;                // T [BL][M][1+D+D(D+1)/2]  per-Gaussian sums of the backward pass: all zero between calls (the
                                //                          build clears them, the backward epilogue clears what it has read)
    size_t pieces;              // int4 [pieces_max]       (point group, offset into cand_list, leaves, -)
    size_t piece_gx;            // T [pieces_max][D][64]   dL/dx of the pieces, added to grad_xes by the epilogue
    bool cand_cache;
    int pieces_max, pool_cap;
    size_t point_groups;
    size_t total;
};

constexpr int kLeafFlush = 512;         // traversal: candidate leaves are evaluated whenever this many have gathered
constexpr int kLeafCap = kLeafFlush + 128;
// The candidate list of a point group depends on the tree and the points only, so the first traversal after a
// build leaves it in the BVH object and later ones (the backward pass after the forward pass) skip the descent.
constexpr size_t kCandCacheBytes = size_t(64) << 20;    // no such lists for launches that would need more
// Point groups in dense regions have candidate lists ten times the average, and the workgroup that owns such a
// group would finish long after all others.  The first traversal therefore cuts a list of more than kPieceLeaves
// leaves into equal pieces of at most that size and publishes all but the first as (group, offset, leaves); in a
// backward pass on known lists the owner works on the first piece only and helper workgroups, one per published
// piece, on the others (their dL/dx goes through piece_gx and the epilogue).  Lists of later rounds of a long
// descent live in a pool behind the fixed slots and are handed out as pieces entirely.
constexpr int kPieceLeaves = 240;        // measured 160 ... 480: shorter pieces cost more in fixed work per workgroup
constexpr int kPiecesMax = 512;         // helper workgroups of a backward launch
constexpr int kPendMax = 16;            // pieces of one point group
constexpr int kCandSplit = 1 << 20;     // flag in cand_count: pieces of this group's list are published
constexpr int kCandRounds = 1 << 21;    // flag in cand_count: the fixed slot holds the first round's list only
constexpr int kCandMask = kCandSplit - 1;

__host__ __device__ inline int own_share(int n) {
    const int pieces = (n + kPieceLeaves - 1) / kPieceLeaves;
    return pieces > 1 ? (n + pieces - 1) / pieces : n;
}

// A list describes the 64 points it was gathered for.  A traversal may be given other points than the build (or the
// same tensor after an in-place change): every list therefore carries a 64-bit stamp of the coordinates of its 64
// points, and a traversal uses a list only when the points it has just loaded give the same stamp; otherwise it
// descends the tree (the build's point order is then only a poor grouping, the result is still right).
struct CandidateCache {
    int* count;                     // null: this object keeps no lists
    int* list;
    int* ctl;                       // always there (error flags)
    int4* pieces;
    unsigned long long* stamp;
    int2* piece_range;
    int pieces_max, pool_cap, pool_base;
};
constexpr int kBoxBlock = 128;          // leaves whose internal nodes get their boxes inside one workgroup (see bvh_leaves_kernel)
constexpr int kFrontier = 64;           // internal nodes a descent starts from (see tree_frontier)
constexpr int kErrStack = 1;            // a traversal's node stack was full and a push was dropped (results incomplete)
constexpr int kErrSort = 2;             // a radix pass computed an output slot outside its segment
constexpr int kSortItems = 2;                       // items per lane and radix block: small chunks, many workgroups
constexpr int kSortBlocksMax = 128;                 // radix blocks per segment (more items per lane beyond that: every block sums
                                                    // the counts of all blocks of its segment; 100000 keys in 98 instead of 196
                                                    // blocks: the build 81 -> 77.5 us)
constexpr int kCoarseOrderMax = 8192;               // point segments up to this size are ordered by 8 Morton bits only
constexpr int kBoundsChunk = kBlock * 2;            // points per workgroup of the partial bounds of the query points

// items per lane of a radix block for segments of `count` keys
static int sort_items(size_t count) {
    size_t items = kSortItems;
    while ((count + kBlock * items - 1) / (kBlock * items) > size_t(kSortBlocksMax)) items *= 2;
    return int(items);
}
static size_t sort_blocks(size_t count) {
    const size_t chunk = size_t(kBlock) * sort_items(count);
    return (count + chunk - 1) / chunk;
}

template <int D> struct LeafRec { static constexpr int kStride = (D == 2) ? 12 : 18; };
// own box (lower[D], upper[D]), then  D=3: b0 b1 b2 c00 c01 c02 c11 c12 c22 amp comp -   D=2: b0 b1 c00 c01 c11 amp comp -

static size_t align_up(size_t v) { return (v + 255) & ~size_t(255); }

static BvhLayout bvh_layout(const gmc_shape& s) {
    const size_t e = s.dtype == GMC_F32 ? 4 : 8;
    const size_t BL = size_t(s.B) * s.L, XL = size_t(s.Bx) * s.Lx;
    const size_t M = s.M, N = s.N, D = s.D;
    const size_t nodes = M > 0 ? 2 * M - 1 : 0;
    const size_t rs = s.D == 2 ? LeafRec<2>::kStride : LeafRec<3>::kStride;
    BvhLayout l;
    size_t o = 0;
    auto take = [&](size_t bytes) { const size_t at = o; o = align_up(o + bytes); return at; };
    l.node_box = take(BL * nodes * 2 * D * e);
    l.child_box = take(BL * (M > 0 ? M - 1 : 0) * 4 * D * e);
    l.leaf_rec = take(BL * M * rs * e);
    l.children = take(BL * (M > 0 ? M - 1 : 0) * 8);
    l.parent = take(BL * nodes * 4);
    l.node_range = take(BL * (M > 0 ? M - 1 : 0) * 8);
    l.leaf_comp = take(BL * M * 4);
    l.run_box = take((BL * M + kBoxBlock - 1) / kBoxBlock * kBoxBlock * 4 * D * e);
    l.parts_g = take(BL * ((M + kBlock - 1) / kBlock) * 2 * D * e);
    l.parts_p = take(XL * ((N + kBoundsChunk - 1) / kBoundsChunk) * 2 * D * e);
    l.keys_a = take(BL * M * 4);
    l.keys_b = take(BL * M * 4);
    l.vals_a = take(BL * M * 4);
    l.vals_b = take(BL * M * 4);
    l.pkeys_a = take(XL * N * 4);
    l.pkeys_b = take(XL * N * 4);
    l.pvals_a = take(XL * N * 4);
    l.pvals_b = take(XL * N * 4);
    l.hist_g = take(4 * BL * sort_blocks(M) * 256 * 4);
    l.hist_p = take(2 * XL * sort_blocks(N) * 256 * 4);
    l.hist_words = (o - l.hist_g) / 4;
    l.p_order = take(XL * N * 4);
    l.g_keys = take(BL * M * 4);
    l.frontier = take(BL * (1 + kFrontier) * 4);
    {
        const size_t point_groups = BL * ((N + kWave - 1) / kWave);
        l.point_groups = point_groups;
        l.cand_cache = M > 1 && point_groups > 0 && point_groups * kLeafCap * 4 <= kCandCacheBytes;
        l.pieces_max = l.cand_cache ? int(point_groups / 2 < size_t(kPiecesMax) ? point_groups / 2 : size_t(kPiecesMax)) : 0;
        l.pool_cap = l.cand_cache ? int(65536 + point_groups * 16) : 0;
        l.cand_count = take(l.cand_cache ? point_groups * 4 : 0);
        l.cand_list = take(l.cand_cache ? (point_groups * kLeafCap + l.pool_cap) * 4 : 0);
        l.cand_stamp = take(l.cand_cache ? point_groups * 8 : 0);
        l.cand_pieces = take(l.cand_cache ? point_groups * 8 : 0);
        l.cand_ctl = take(16);
        l.sums = take(BL * M * (D == 2 ? 6 : 10) * e);
        l.pieces = take(size_t(l.pieces_max) * 16);
        l.piece_gx = take(size_t(l.pieces_max) * D * kWave * e);
    }
    l.total = o;
    return l;
}

static CandidateCache candidate_cache(char* bvh, const BvhLayout& lay) {
    CandidateCache c{};
    c.ctl = (int*)(bvh + lay.cand_ctl);
    if (!lay.cand_cache) return c;
    c.count = (int*)(bvh + lay.cand_count);
    c.list = (int*)(bvh + lay.cand_list);
    c.pieces = (int4*)(bvh + lay.pieces);
    c.stamp = (unsigned long long*)(bvh + lay.cand_stamp);
    c.piece_range = (int2*)(bvh + lay.cand_pieces);
    c.pieces_max = lay.pieces_max;
    c.pool_cap = lay.pool_cap;
    c.pool_base = int(lay.point_groups * kLeafCap);
    return c;
}

// ---------------------------------------------------------------------------------------------------------------
// per-Gaussian boxes
// ---------------------------------------------------------------------------------------------------------------

// Symmetric eigen-decomposition as the reference's device functions define it (math/symeig_detail.h:17-72 for
// 2x2, :75-138 for 3x3), restated here because the "reference" box rule is a function of ITS outputs, quirks
// included (absolute 1e-7 test for "diagonal", identity vectors when the off-diagonal is exactly zero).
// lam[j]: values in the reference's output order; v[i][j]: j-th component of the i-th vector.
__device__ inline void ref_symeig2(const double a[2][2], double lam[2], double v[2][2]) {
    const double tr = a[0][0] + a[1][1];
    const double det = a[0][0] * a[1][1] - a[0][1] * a[1][0];
    const double aa = a[0][0], bb = a[0][1], dd = a[1][1];
    const double f1 = tr / 2.0, f2 = sqrt(fabs(tr * tr / 4.0 - det));
    lam[0] = f1 - f2;
    lam[1] = f1 + f2;
    if (bb == 0.0) {
        v[0][0] = 1.0; v[0][1] = 0.0; v[1][0] = 0.0; v[1][1] = 1.0;
        return;
    }
    double e0[2], e1[2];
    if (aa < dd) { e0[0] = bb; e0[1] = lam[0] - aa; e1[0] = bb; e1[1] = lam[1] - aa; }
    else         { e0[0] = lam[0] - dd; e0[1] = bb; e1[0] = lam[1] - dd; e1[1] = bb; }
    const double n0 = sqrt(e0[0] * e0[0] + e0[1] * e0[1]), n1 = sqrt(e1[0] * e1[0] + e1[1] * e1[1]);
    v[0][0] = e0[0] / n0; v[0][1] = e0[1] / n0;
    v[1][0] = e1[0] / n1; v[1][1] = e1[1] / n1;
}

// longest column of the symmetric matrix p, normalised; false if every column vanishes
__device__ inline bool longest_column(const double p[3][3], double out[3]) {
    double best = 0.0;
    int idx = -1;
    for (int j = 0; j < 3; ++j) {
        const double len = p[0][j] * p[0][j] + p[1][j] * p[1][j] + p[2][j] * p[2][j];
        if (len > best) { best = len; idx = j; }
    }
    if (idx < 0) return false;
    const double inv = 1.0 / sqrt(best);
    for (int i = 0; i < 3; ++i) out[i] = p[i][idx] * inv;
    return true;
}

__device__ inline void shifted_product(const double a[3][3], double s1, double s2, double p[3][3]) {
    double x[3][3], y[3][3];
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) {
            x[i][j] = a[i][j] - (i == j ? s1 : 0.0);
            y[i][j] = a[i][j] - (i == j ? s2 : 0.0);
        }
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) p[i][j] = x[i][0] * y[0][j] + x[i][1] * y[1][j] + x[i][2] * y[2][j];
}

__device__ inline bool ref_symeig3(const double a[3][3], double lam[3], double v[3][3]) {
    const double kPi = 3.14159265358979323846;
    double eig0, eig1, eig2;
    const double p1 = a[0][1] * a[0][1] + a[0][2] * a[0][2] + a[1][2] * a[1][2];
    if (p1 <= 0.0000001) {
        eig0 = a[0][0]; eig1 = a[1][1]; eig2 = a[2][2];
    } else {
        const double q = (a[0][0] + a[1][1] + a[2][2]) / 3.0;
        const double p2 = (a[0][0] - q) * (a[0][0] - q) + (a[1][1] - q) * (a[1][1] - q) + (a[2][2] - q) * (a[2][2] - q) + 2.0 * p1;
        const double p = sqrt(p2 / 6.0);
        double b[3][3];
        for (int i = 0; i < 3; ++i)
            for (int j = 0; j < 3; ++j) b[i][j] = (a[i][j] - (i == j ? q : 0.0)) / p;
        const double detb = b[0][0] * (b[1][1] * b[2][2] - b[1][2] * b[2][1]) - b[0][1] * (b[1][0] * b[2][2] - b[1][2] * b[2][0]) +
                            b[0][2] * (b[1][0] * b[2][1] - b[1][1] * b[2][0]);
        const double r = detb / 2.0;
        double phi;
        if (r <= -1.0) phi = kPi / 3.0;
        else if (r >= 1.0) phi = 0.0;
        else phi = acos(r) / 3.0;
        eig0 = q + 2.0 * p * cos(phi);
        eig2 = q + 2.0 * p * cos(phi + 2.0 * kPi / 3.0);
        eig1 = 3.0 * q - eig0 - eig2;
    }
    double pm[3][3], v0[3], v1[3];
    shifted_product(a, eig1, eig2, pm);
    if (!longest_column(pm, v0)) return false;
    shifted_product(a, eig0, eig2, pm);
    if (!longest_column(pm, v1)) return false;
    lam[0] = eig2; lam[1] = eig1; lam[2] = eig0;
    v[0][0] = v0[1] * v1[2] - v0[2] * v1[1];
    v[0][1] = v0[2] * v1[0] - v0[0] * v1[2];
    v[0][2] = v0[0] * v1[1] - v0[1] * v1[0];
    for (int j = 0; j < 3; ++j) { v[1][j] = v1[j]; v[2][j] = v0[j]; }
    return true;
}

// half extents of the cutoff box of one Gaussian (record g: weight, position, inverse covariance)
template <typename T, int D>
__device__ inline void box_half_extent(const T* __restrict__ g, double threshold, int mode, bool covariance_form,
                                       double* delta) {
    const double w = fabs(double(g[0]));
    double s2 = -2.0 * log(threshold / w);
    s2 = fmax(s2, kSqFloor);
    const double s = sqrt(s2);
    const T* c = g + 1 + D;
    double sigma[D][D];
    // the reference inverts the stored matrix read column-major, i.e. C^T (util/glm.h:108-128); a record in
    // covariance form holds S with C = (S^-1)^T (src/gmc/mixture.py:149), so that inverse is S itself
    if (covariance_form) {
        for (int i = 0; i < D; ++i)
            for (int j = 0; j < D; ++j) sigma[i][j] = double(c[i * D + j]);
    } else if constexpr (D == 2) {
        const double m00 = c[0], m01 = c[2], m10 = c[1], m11 = c[3];
        const double inv = 1.0 / (m00 * m11 - m01 * m10);        // one division; the entries are products with it
        sigma[0][0] = m11 * inv; sigma[0][1] = -m01 * inv; sigma[1][0] = -m10 * inv; sigma[1][1] = m00 * inv;
    } else {
        double m[3][3];
        for (int i = 0; i < 3; ++i)
            for (int j = 0; j < 3; ++j) m[i][j] = double(c[j * 3 + i]);
        const double c00 = m[1][1] * m[2][2] - m[1][2] * m[2][1];
        const double c01 = m[1][2] * m[2][0] - m[1][0] * m[2][2];
        const double c02 = m[1][0] * m[2][1] - m[1][1] * m[2][0];
        const double inv = 1.0 / (m[0][0] * c00 + m[0][1] * c01 + m[0][2] * c02);
        sigma[0][0] = c00 * inv;
        sigma[1][1] = (m[0][0] * m[2][2] - m[0][2] * m[2][0]) * inv;
        sigma[2][2] = (m[0][0] * m[1][1] - m[0][1] * m[1][0]) * inv;
        if (mode == GMC_AABB_REFERENCE) {                        // the tight box needs the diagonal only
            sigma[1][0] = c01 * inv;
            sigma[2][0] = c02 * inv;
            sigma[0][1] = (m[0][2] * m[2][1] - m[0][1] * m[2][2]) * inv;
            sigma[2][1] = (m[0][1] * m[2][0] - m[0][0] * m[2][1]) * inv;
            sigma[0][2] = (m[0][1] * m[1][2] - m[0][2] * m[1][1]) * inv;
            sigma[1][2] = (m[0][2] * m[1][0] - m[0][0] * m[1][2]) * inv;
        } else {
            sigma[1][0] = sigma[2][0] = sigma[0][1] = sigma[2][1] = sigma[0][2] = sigma[1][2] = 0.0;
        }
    }
    double tight[D];
    for (int k = 0; k < D; ++k) tight[k] = sqrt(fmax(sigma[k][k], 0.0));
    bool literal = (mode == GMC_AABB_REFERENCE);
    double lit[D];
    if (literal) {
        double lam[D], v[D][D];
        if constexpr (D == 2) ref_symeig2(sigma, lam, v);
        else literal = ref_symeig3(sigma, lam, v);
        if (literal) {
            for (int k = 0; k < D; ++k) {
                double acc = 0.0;
                for (int j = 0; j < D; ++j) acc += lam[j] * v[k][j] * v[k][j];
                lit[k] = sqrt(acc);
                if (!(lit[k] == lit[k]) || isinf(lit[k])) literal = false;   // undefined rule -> tight box
            }
        }
    }
    for (int k = 0; k < D; ++k) delta[k] = s * (literal ? lit[k] : tight[k]);
}

// One launch for two independent jobs.
// Workgroups [0, box_blocks): workgroup (blk, seg) leaves the bounds of its 256 centres in parts_g[seg][blk].  (The
// cutoff boxes of the Gaussians, a long chain of double arithmetic, are not needed before the leaves are written:
// bvh_leaves_kernel computes them, next to the tree build, off the critical path of the sort.)
// Workgroups behind them: partial bounds of the query points; workgroup (blk, seg) reduces kBoundsChunk points to
// parts_p[seg][blk] = (min_0..min_D-1, max_0..max_D-1).  The Morton kernel combines the partial records.
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void bvh_bounds_kernel(const T* __restrict__ mixture, int M, int blocks_per_mixture,
                                                           T* __restrict__ parts_g, unsigned box_blocks, const T* __restrict__ xes, int N,
                                                           int blocks_per_xseg, T* __restrict__ parts_p, int* __restrict__ ctl,
                                                           uint32_t* __restrict__ hist, size_t hist_words) {
    constexpr int G = 1 + D + D * D;
    __shared__ T red[2 * D][kBlock];
    // first launch of a build: a new tree has no published pieces, an empty pool and no error
    if (blockIdx.x == 0 && threadIdx.x < 4) ctl[threadIdx.x] = 0;
    // the block histograms of all radix passes are counted with atomics by the kernels that follow
    for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < hist_words; i += size_t(gridDim.x) * kBlock) hist[i] = 0u;
    T lo[D], hi[D];
    for (int d = 0; d < D; ++d) { lo[d] = T(INFINITY); hi[d] = T(-INFINITY); }
    if (blockIdx.x < box_blocks) {
        const int seg = blockIdx.x / blocks_per_mixture, blk = blockIdx.x - seg * blocks_per_mixture;
        const int m = blk * kBlock + threadIdx.x;
        if (m < M) {
            const size_t i = size_t(seg) * M + m;
            const T* g = mixture + i * G;
            for (int k = 0; k < D; ++k) {
                lo[k] = g[1 + k] < lo[k] ? g[1 + k] : lo[k];       // a NaN coordinate is skipped
                hi[k] = g[1 + k] > hi[k] ? g[1 + k] : hi[k];
            }
        }
        const T v = block_bounds<T, D>(lo, hi, red);
        if (threadIdx.x < 2 * D) parts_g[size_t(blockIdx.x) * 2 * D + threadIdx.x] = v;
    } else {
        const unsigned id = blockIdx.x - box_blocks;
        const int seg = id / blocks_per_xseg, blk = id - seg * blocks_per_xseg;
        const T* p = xes + size_t(seg) * N * D;
        const int begin = blk * kBoundsChunk;
        const int end = begin + kBoundsChunk < N ? begin + kBoundsChunk : N;
        for (int i = begin + threadIdx.x; i < end; i += kBlock)
            for (int d = 0; d < D; ++d) {
                const T a = p[size_t(i) * D + d];
                lo[d] = a < lo[d] ? a : lo[d];
                hi[d] = a > hi[d] ? a : hi[d];
            }
        const T v = block_bounds<T, D>(lo, hi, red);
        if (threadIdx.x < 2 * D) parts_p[size_t(id) * 2 * D + threadIdx.x] = v;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Morton keys
// ---------------------------------------------------------------------------------------------------------------

__device__ __forceinline__ uint32_t expand_bits3(uint32_t v) {
    v = (v * 0x00010001u) & 0xFF0000FFu;
    v = (v * 0x00000101u) & 0x0F00F00Fu;
    v = (v * 0x00000011u) & 0xC30C30C3u;
    v = (v * 0x00000005u) & 0x49249249u;
    return v;
}

// 10 bits per axis of the position normalised by `bounds`, in the arithmetic of the tensors' own precision as the
// reference does it (lbvh/bvh.cu:281-287: p -= lower; p /= upper - lower; lbvh/morton_code.h:145-168: cell =
// uint32(p * 1024) clamped to 1023); an axis of zero extent (0/0 in the reference) maps to cell 0
template <typename T, int D>
__device__ __forceinline__ uint32_t morton30(const T* __restrict__ p, const T* __restrict__ bounds) {
    uint32_t code = 0;
#pragma unroll
    for (int d = 0; d < D; ++d) {
        const T lo = bounds[d], ext = bounds[D + d] - lo;
        T q = ext > T(0) ? (p[d] - lo) / ext * T(1024)   /* hipcc divides with correct rounding by default */ : T(0);
        q = q < T(0) ? T(0) : (q > T(1023) ? T(1023) : q);
        q = (q == q) ? q : T(0);
        code |= expand_bits3(uint32_t(q)) << (2 - d);
    }
    return code;
}

// a set of points to be Morton-coded: the centres of the mixtures or the query points
template <typename T> struct MortonJob {
    const T* pts; int stride, offset, count;
    int items, blocks_per_seg;                                     // workgroup (blk, seg) codes kBlock * items points
    const T* parts; int n_parts;                                   // partial bounds of every segment
    uint32_t* keys; uint32_t* vals;
    unsigned blocks;                                               // workgroups of this job in the launch
    uint32_t* hist; int shift;       // block histograms of the first radix pass, one per workgroup (null: none wanted)
};

// Morton keys and index payload for two jobs in one launch (job b behind job a); every workgroup first combines
// its segment's partial bounds.  A workgroup codes the keys of exactly one block of the first radix pass, so that the
// block's digit histogram is counted in LDS and stored (global atomics would leave the launch waiting for their round
// trip to the memory side).
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void morton_kernel(MortonJob<T> a, MortonJob<T> b) {
    __shared__ T red[2 * D][kBlock];
    __shared__ T bounds[2 * D];
    __shared__ uint32_t digits[256];
    const bool first = blockIdx.x < a.blocks;
    const MortonJob<T>& j = first ? a : b;
    const unsigned id = first ? blockIdx.x : blockIdx.x - a.blocks;
    const int seg = id / j.blocks_per_seg, blk = id - seg * j.blocks_per_seg;
    // eight points per lane at a time, all loads in flight; the first ones are fetched while the bounds are combined
    constexpr int kBatch = 8;
    T p[kBatch][D];
    auto fetch = [&](int r0) {
#pragma unroll
        for (int r = 0; r < kBatch; ++r) {
            const int i = (blk * j.items + r0 + r) * kBlock + threadIdx.x;
            if (r0 + r < j.items && i < j.count) {
                const T* src = j.pts + (size_t(seg) * j.count + i) * j.stride + j.offset;
                for (int d = 0; d < D; ++d) p[r][d] = src[d];
            }
        }
    };
    fetch(0);
    T lo[D], hi[D];
    for (int d = 0; d < D; ++d) { lo[d] = T(INFINITY); hi[d] = T(-INFINITY); }
    for (int i = threadIdx.x; i < j.n_parts; i += kBlock) {
        const T* q = j.parts + (size_t(seg) * j.n_parts + i) * 2 * D;
        for (int d = 0; d < D; ++d) {
            lo[d] = q[d] < lo[d] ? q[d] : lo[d];
            hi[d] = q[D + d] > hi[d] ? q[D + d] : hi[d];
        }
    }
    const T v = block_bounds<T, D>(lo, hi, red);
    if (threadIdx.x < 2 * D) bounds[threadIdx.x] = v;
    digits[threadIdx.x] = 0u;
    __syncthreads();
    for (int r0 = 0; r0 < j.items; r0 += kBatch) {
        if (r0 > 0) fetch(r0);
#pragma unroll
        for (int r = 0; r < kBatch; ++r) {
            const int i = (blk * j.items + r0 + r) * kBlock + threadIdx.x;
            if (r0 + r < j.items && i < j.count) {
                const size_t at = size_t(seg) * j.count + i;
                const uint32_t key = morton30<T, D>(p[r], bounds);
                j.keys[at] = key;
                j.vals[at] = uint32_t(i);
                if (j.hist) atomicAdd(&digits[(key >> j.shift) & 255u], 1u);
            }
        }
    }
    if (!j.hist) return;
    __syncthreads();
    j.hist[(size_t(seg) * j.blocks_per_seg + blk) * 256 + threadIdx.x] = digits[threadIdx.x];
}

// ---------------------------------------------------------------------------------------------------------------
// segmented LSD radix sort, 8 bits per pass, stable; segments of equal length `count`
// ---------------------------------------------------------------------------------------------------------------
// one pass over one set of segments
struct SortJob {
    const uint32_t* keys_in; const uint32_t* vals_in; uint32_t* keys_out; uint32_t* vals_out;
    const uint32_t* hist;                // [segments][blocks_per_seg][256] of this pass
    uint32_t* hist_next;                 // the same for the next pass, counted here; null in the last pass
    int count, items, blocks_per_seg, shift, chunk_shift;
    unsigned blocks;                     // workgroups of this job in the launch
    int* err;                            // error flags of the BVH object
};

// One pass of the sort by workgroup `id` of job j (all kBlock lanes of the workgroup call it).  The block histograms of
// a pass are counted by the kernel that writes the pass's input (the Morton kernel, or the pass before) with one
// atomic per key, which saves a histogram launch per pass: the passes are short kernels, bound by launch latency.
__device__ __forceinline__ void radix_scatter_pass(const SortJob& j, unsigned id) {
    __shared__ uint32_t running[256];        // next output slot of every digit for this block
    __shared__ uint32_t wave_count[4][256];
    __shared__ uint32_t wave_total[4];
    const int blocks_per_seg = j.blocks_per_seg, count = j.count, shift = j.shift;
    const int seg = id / blocks_per_seg, blk = id - seg * blocks_per_seg;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // thread d: keys of digit d in the whole segment and in the blocks before this one (at most kSortBlocksMax
    // counts per digit, so no separate scan pass is needed)
    const size_t seg_off = size_t(seg) * count;
    const int begin = blk * j.items * kBlock;
    // the keys of the first round are fetched while the histogram columns are summed
    uint32_t next_key = 0, next_val = 0;
    if (begin + int(threadIdx.x) < count) {
        next_key = j.keys_in[seg_off + begin + threadIdx.x];
        next_val = j.vals_in[seg_off + begin + threadIdx.x];
    }
    uint32_t mine = 0, earlier = 0;
    {
        const uint32_t* col = j.hist + size_t(seg) * blocks_per_seg * 256 + threadIdx.x;
        // the loop is latency-bound: groups of 32, then of 8 independent loads in flight
        int q0 = 0;
        for (; q0 + 32 <= blocks_per_seg; q0 += 32) {
            uint32_t c[32];
#pragma unroll
            for (int q = 0; q < 32; ++q) c[q] = col[size_t(q0 + q) * 256];
#pragma unroll
            for (int q = 0; q < 32; ++q) { mine += c[q]; earlier += q0 + q < blk ? c[q] : 0u; }
        }
        for (; q0 + 8 <= blocks_per_seg; q0 += 8) {
            uint32_t c[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) c[q] = col[size_t(q0 + q) * 256];
#pragma unroll
            for (int q = 0; q < 8; ++q) { mine += c[q]; earlier += q0 + q < blk ? c[q] : 0u; }
        }
        for (; q0 < blocks_per_seg; ++q0) {
            const uint32_t c = col[size_t(q0) * 256];
            mine += c;
            earlier += q0 < blk ? c : 0u;
        }
    }
    // exclusive scan of the segment's digit totals = first slot of every digit: inclusive scan inside each
    // wavefront, then the totals of the wavefronts before
    uint32_t scan = mine;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const uint32_t up = __shfl_up(scan, off, kWave);
        scan += lane >= off ? up : 0u;
    }
    if (lane == kWave - 1) wave_total[wave] = scan;
#pragma unroll
    for (int w = 0; w < 4; ++w) wave_count[w][threadIdx.x] = 0;
    __syncthreads();
    for (int w = 0; w < wave; ++w) scan += wave_total[w];
    running[threadIdx.x] = scan - mine + earlier;
    __syncthreads();
    for (int round = 0; round < j.items; ++round) {
        const int i = begin + round * kBlock + threadIdx.x;
        const bool valid = i < count;
        const uint32_t key = next_key, val = next_val;
        const uint32_t digit = valid ? (key >> shift) & 255u : 0u;
        if (round + 1 < j.items && i + kBlock < count) {
            next_key = j.keys_in[seg_off + i + kBlock];
            next_val = j.vals_in[seg_off + i + kBlock];
        }
        // lanes of this wavefront holding the same digit
        unsigned long long same = __ballot(valid);
#pragma unroll
        for (int bit = 0; bit < 8; ++bit) {
            const unsigned long long m = __ballot((digit >> bit) & 1u);
            same &= ((digit >> bit) & 1u) ? m : ~m;
        }
        const int rank = __popcll(same & ((1ull << lane) - 1ull));
        if (valid && rank == 0) wave_count[wave][digit] = uint32_t(__popcll(same));
        __syncthreads();
        if (valid) {
            uint32_t slot = running[digit] + rank;
            for (int w = 0; w < wave; ++w) slot += wave_count[w][digit];
            if (slot < uint32_t(count)) {          // always true for a consistent histogram; keeps a bug from writing out of bounds
                j.keys_out[seg_off + slot] = key;
                j.vals_out[seg_off + slot] = val;
                if (j.hist_next)
                    atomicAdd(&j.hist_next[(size_t(seg) * blocks_per_seg + (slot >> j.chunk_shift)) * 256 + ((key >> (shift + 8)) & 255u)], 1u);
            } else {
                atomicOr(j.err, kErrSort);
            }
        }
        __syncthreads();
        {
            uint32_t add = 0;
#pragma unroll
            for (int w = 0; w < 4; ++w) { add += wave_count[w][threadIdx.x]; wave_count[w][threadIdx.x] = 0; }
            running[threadIdx.x] += add;
        }
        __syncthreads();
    }
}

// A pass for two jobs in one launch (job b behind job a).
__global__ __launch_bounds__(kBlock) void radix_scatter_kernel(SortJob a, SortJob b) {
    if (blockIdx.x < a.blocks) radix_scatter_pass(a, blockIdx.x);
    else radix_scatter_pass(b, blockIdx.x - a.blocks);
}

// orders the LDS traffic of one wavefront: stores of some lanes before loads of other lanes
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The leaves' sort for one large tree (kSmallTreeMax < M <= kBucketSortMax; two trees of up to half that size, whose
// workgroups fit a compute unit in pairs: more would queue up) in ONE launch instead of four radix
// passes at their latency floor: 256 workgroups per tree, one per value of the top 8 key bits.  Workgroup d reads all
// keys of the tree (in component order, as the Morton kernel wrote them; 64 KB at most, from L2), keeps those whose top
// bits are d as unique keys (Morton code << 32 | component) in LDS, counts those with smaller top bits -- the first
// slot of its own --, sorts its keys (by counting ranks; more than kBucketRankMax: a bitonic network) and writes them out: ascending
// unique keys are the stable order of the codes.  No histograms, no passes that wait for each other.  A digit that
// holds most keys (all centres in one cell) is one long sort by a single workgroup: slower than the four passes, same
// result.
constexpr int kBucketSortLanes = 1024;
constexpr int kBucketSortMax = 16384;
constexpr int kBucketRankMax = 256;        // keys of one digit up to which counting ranks beats the sorting network
constexpr int kBucketCrowded = 1024;       // expected keys of one value of the top bits from which splitters are taken instead

template <int CAP>
__global__ __launch_bounds__(kBucketSortLanes) void bucket_sort_kernel(const uint32_t* __restrict__ keys_in, uint32_t* __restrict__ keys_out,
                                                                      uint32_t* __restrict__ vals_out, int count, int* __restrict__ err) {
    constexpr int kPerLane = CAP / kBucketSortLanes;         // keys of the tree per lane, at most
    __shared__ unsigned long long k[CAP];
    __shared__ int n_mine, n_before;
    const int seg = blockIdx.x >> 8, lane = threadIdx.x & 63;
    const uint32_t digit = blockIdx.x & 255;
    const uint32_t* in = keys_in + size_t(seg) * count;
    if (threadIdx.x == 0) { n_mine = 0; n_before = 0; }
    static_assert(kPerLane % 4 == 0 || kPerLane == 2, "keys are fetched four (two) at a time");
    constexpr int kVec = kPerLane == 2 ? 2 : 4, kLoads = kPerLane / kVec;
    uint32_t key[kPerLane];
    // (a second segment may start off a multiple of the vector width: key by key then)
    const bool wide = (size_t(seg) * count) % kVec == 0;
#pragma unroll
    for (int r = 0; r < kLoads; ++r) {                       // all loads in flight together
        const int i = (r * kBucketSortLanes + threadIdx.x) * kVec;
        if (wide && i + kVec <= count) {
            if constexpr (kVec == 4) {
                const uint4 v = *reinterpret_cast<const uint4*>(in + i);
                key[4 * r] = v.x; key[4 * r + 1] = v.y; key[4 * r + 2] = v.z; key[4 * r + 3] = v.w;
            } else {
                const uint2 v = *reinterpret_cast<const uint2*>(in + i);
                key[2 * r] = v.x; key[2 * r + 1] = v.y;
            }
        } else {
#pragma unroll
            for (int c = 0; c < kVec; ++c) key[kVec * r + c] = i + c < count ? in[i + c] : 0xffffffffu;   // (real keys have 30 bits)
        }
    }
    // the component of key r of this lane
    auto component = [&](int r) { return ((r / kVec) * kBucketSortLanes + int(threadIdx.x)) * kVec + r % kVec; };
    // Which workgroup takes a key: the one numbered by its top 8 bits -- unless the centres crowd into a few Morton
    // cells (a stray Gaussian far from the others is enough to stretch the bounds), when one workgroup would sort most
    // of the tree alone.  Every workgroup tests the same sample for that (every lane one of its keys: 1024 of the tree's),
    // and all take splitters instead when a value of the top bits is expected to hold more than kBucketCrowded keys:
    // 256 sampled unique keys, sorted by counting; workgroup d takes the keys from splitter d up to splitter d + 1, found
    // by bisection.  Same result either way; the choice is a function of the keys alone.
    __shared__ uint32_t sample_bins[256];
    __shared__ unsigned long long sample[256], splitter[256];
    if (threadIdx.x < 256) sample_bins[threadIdx.x] = 0u;
    __syncthreads();
    {
        // (which of its keys a lane samples, and which lane of four gives a splitter candidate, change with the higher bits
        // of the lane number: components that follow a pattern of period 2, 4, 8 ... are all represented)
        uint32_t mine = key[0];
        int r_mine = 0;
#pragma unroll
        for (int r = 1; r < kPerLane; ++r)
            if (int(threadIdx.x >> 3) % kPerLane == r) { mine = key[r]; r_mine = r; }
        const int i = component(r_mine);
        if (i < count) atomicAdd(&sample_bins[(mine >> 22) & 255u], 1u);
        if ((threadIdx.x & 3) == ((threadIdx.x >> 5) & 3))
            sample[threadIdx.x >> 2] = i < count ? ((unsigned long long)mine << 32) | uint32_t(i) : ~0ull;
    }
    __syncthreads();                                         // the sample is counted
    const bool crowded = __syncthreads_or(threadIdx.x < 256 && sample_bins[threadIdx.x & 255] * kPerLane > uint32_t(kBucketCrowded));
    if (crowded) {
        if (threadIdx.x < 256) {
            const unsigned long long mine = sample[threadIdx.x];
            int rank = 0;
#pragma unroll 8
            for (int j = 0; j < 256; ++j) rank += (sample[j] < mine || (sample[j] == mine && j < int(threadIdx.x))) ? 1 : 0;
            splitter[rank] = mine;                           // (absent samples, all ones, share the end)
        }
        __syncthreads();
    }
    // number of the workgroup that takes unique key x: the last splitter not above it (workgroup 0 also takes what lies below splitter 0)
    auto taker = [&](unsigned long long x) {
        int lo = 0;                                          // splitter[lo] <= x or lo == 0
#pragma unroll
        for (int step = 128; step > 0; step >>= 1)
            lo = splitter[lo + step] <= x ? lo + step : lo;
        return uint32_t(lo);
    };
    uint32_t top[kPerLane];
#pragma unroll
    for (int r = 0; r < kPerLane; ++r) top[r] = key[r] >> 22;
    if (crowded) {                                           // (the searches of a lane's keys side by side)
#pragma unroll
        for (int r = 0; r < kPerLane; ++r) {
            const int i = component(r);
            top[r] = i < count ? taker(((unsigned long long)key[r] << 32) | uint32_t(i)) : 1024u;
        }
    }
    int before = 0;
#pragma unroll
    for (int r = 0; r < kPerLane; ++r) {
        const int i = component(r);
        const unsigned long long unique = ((unsigned long long)key[r] << 32) | uint32_t(i);
        before += top[r] < digit ? 1 : 0;
        const bool mine = top[r] == digit;
        const unsigned long long m = __ballot(mine);
        if (m != 0ull) {                                     // (the order inside the digit does not matter: the keys are unique)
            int base = 0;
            if (lane == __ffsll((long long)m) - 1) base = atomicAdd(&n_mine, __popcll(m));
            base = __shfl(base, __ffsll((long long)m) - 1, kWave);
            if (mine) k[base + __popcll(m & ((1ull << lane) - 1ull))] = unique;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off, kWave);
    if (lane == 0 && before != 0) atomicAdd(&n_before, before);
    __syncthreads();
    const int n = n_mine, begin = n_before;
    if (n == 0) return;                                      // (the same for every lane of the workgroup)
    if (begin + n > count) {                                 // never
        if (threadIdx.x == 0) atomicOr(err, kErrSort);
        return;
    }
    const size_t at = size_t(seg) * count + begin;
    if (n <= kBucketRankMax) {
        // a few keys (the usual case: M / 256 on average): lane i counts the keys below key i and puts it there -- every
        // read is a broadcast, no step waits for another
        if (int(threadIdx.x) < n) {
            const unsigned long long mine = k[threadIdx.x];
            int rank = 0;
#pragma unroll 8
            for (int j = 0; j < n; ++j) rank += k[j] < mine ? 1 : 0;
            keys_out[at + rank] = uint32_t(mine >> 32);
            vals_out[at + rank] = uint32_t(mine);
        }
        return;
    }
    int np = 2;
    while (np < n) np <<= 1;
    // (wavefronts without a pair of keys leave before the barriers)
    const int lanes = np / 2 < kBucketSortLanes ? np / 2 : kBucketSortLanes;
    if (int(threadIdx.x) >= lanes) return;
    for (int i = n + threadIdx.x; i < np; i += lanes) k[i] = ~0ull;
    __syncthreads();
    for (int size = 2; size <= np; size <<= 1)
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int q = threadIdx.x; q < np / 2; q += lanes) {
                const int i0 = ((q & ~(stride - 1)) << 1) | (q & (stride - 1)), i1 = i0 | stride;
                const unsigned long long k0 = k[i0], k1 = k[i1];
                if ((k0 > k1) == ((i0 & size) == 0)) { k[i0] = k1; k[i1] = k0; }
            }
            __syncthreads();
        }
    for (int i = threadIdx.x; i < n; i += lanes) {
        keys_out[at + i] = uint32_t(k[i] >> 32);
        vals_out[at + i] = uint32_t(k[i]);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// leaves, radix tree, boxes
// ---------------------------------------------------------------------------------------------------------------
// Order-preserving map from a floating-point value to a signed 64-bit integer (a < b <=> ordered(a) < ordered(b)),
// so that box unions can be formed with integer atomic min/max.
__device__ __forceinline__ long long ordered_bits(double v) {
    const long long b = __builtin_bit_cast(long long, v);
    return b ^ ((b >> 63) & 0x7fffffffffffffffll);
}
__device__ __forceinline__ double from_ordered_bits(long long k) {
    return __builtin_bit_cast(double, k ^ ((k >> 63) & 0x7fffffffffffffffll));
}
__device__ __forceinline__ int ordered_bits(float v) {
    const int b = __builtin_bit_cast(int, v);
    return b ^ ((b >> 31) & 0x7fffffff);
}
__device__ __forceinline__ float from_ordered_bits(int k) { return __builtin_bit_cast(float, k ^ ((k >> 31) & 0x7fffffff)); }
// the integer type of T's width, and the empty box in it: lower = +inf, upper = -inf
template <typename T> struct OrderedInt;
template <> struct OrderedInt<float> { using type = int; static constexpr int kEmptyLo = 0x7fffffff, kEmptyHi = -0x7fffffff - 1; };
template <> struct OrderedInt<double> {
    using type = long long;
    static constexpr long long kEmptyLo = 0x7fffffffffffffffll, kEmptyHi = -0x7fffffffffffffffll - 1;
};

// Internal node i of the radix tree over the M sorted keys (Karras 2012; lbvh/building.h:11-103); key_at(j) returns the
// j-th sorted Morton code, the unique keys are (code << 32 | j).  first / last: the range of leaves below the node;
// left / right: its children, >= 0 an internal node, < 0 leaf ~index.
template <typename KeyAt>
__device__ __forceinline__ void radix_tree_node(KeyAt key_at, int M, int i, int& first, int& last, int& left, int& right) {
    // number of leading bits shared by the unique keys a and b; -1 outside
    auto common_prefix = [&](int a, int b) -> int {
        if (b < 0 || b >= M) return -1;
        const uint32_t ka = key_at(a), kb = key_at(b);
        if (ka != kb) return __clz(ka ^ kb);
        return 32 + __clz(uint32_t(a) ^ uint32_t(b));
    };
    // range of keys covered by internal node i
    if (i == 0) { first = 0; last = M - 1; }
    else {
        const int dl = common_prefix(i, i - 1), dr = common_prefix(i, i + 1);
        const int dir = dr > dl ? 1 : -1;
        const int dmin = dr > dl ? dl : dr;
        int lmax = 2;
        while (common_prefix(i, i + lmax * dir) > dmin) lmax <<= 1;
        int len = 0;
        for (int step = lmax >> 1; step > 0; step >>= 1)
            if (common_prefix(i, i + (len + step) * dir) > dmin) len += step;
        const int j = i + len * dir;
        first = i < j ? i : j;
        last = i < j ? j : i;
    }
    // split: the highest key that shares more than the node's prefix with the first key
    const int dnode = common_prefix(first, last);
    int split = first, stride = last - first;
    do {
        stride = (stride + 1) >> 1;
        const int mid = split + stride;
        if (mid < last && common_prefix(first, mid) > dnode) split = mid;
    } while (stride > 1);
    left = (split == first) ? ~split : split;               // leaf `split` or internal node `split`
    right = (split + 1 == last) ? ~(split + 1) : split + 1;
}

// internal node i of the radix tree of mixture bl (key_at(j): the j-th sorted key of the mixture); returns its range
template <typename KeyAt>
__device__ __forceinline__ int2 build_internal_node(KeyAt key_at, int2* __restrict__ children,
                                                    int* __restrict__ parent, int2* __restrict__ node_range, int M,
                                                    size_t bl, int i) {
    const size_t t = bl * (M - 1) + i;
    int first, last, left, right;
    radix_tree_node(key_at, M, i, first, last, left, right);
    children[t] = make_int2(left, right);
    node_range[t] = make_int2(first, last);
    int* par = parent + bl * (2 * size_t(M) - 1);
    par[left >= 0 ? left : (M - 1) + ~left] = i;
    par[right >= 0 ? right : (M - 1) + ~right] = i;
    if (i == 0) par[0] = -1;
    return make_int2(first, last);
}

// Leaf `leaf` (Morton order) of mixture bl, which holds component `comp` with the record g: the cutoff box of the Gaussian
// (lbvh/bvh.cu:164-231; stored as the leaf's node box), its evaluation record behind its own box, zeroed sums of the
// backward pass.  blo / bhi receive the box.
template <typename T, int D>
__device__ __forceinline__ void write_leaf(const T* __restrict__ g, double threshold, int mode, bool covariance_form, T* __restrict__ node_box,
                                           T* __restrict__ leaf_rec, int* __restrict__ parent, T* __restrict__ sums, int M,
                                           size_t bl, int leaf, int comp, T (&blo)[D], T (&bhi)[D]) {
    constexpr int RS = LeafRec<D>::kStride;
    constexpr int NS = 1 + D + D * (D + 1) / 2;
    const size_t i = bl * M + leaf;
    // the per-Gaussian sums of the backward pass start from zero (and return to zero after every backward pass)
    for (int k = 0; k < NS; ++k) sums[i * NS + k] = T(0);
    const size_t node = bl * (2 * size_t(M) - 1) + (M - 1) + leaf;
    {
        double delta[D];
        box_half_extent<T, D>(g, threshold, mode, covariance_form, delta);
        for (int d = 0; d < D; ++d) {
            blo[d] = T(double(g[1 + d]) - delta[d]);
            bhi[d] = T(double(g[1 + d]) + delta[d]);
        }
    }
    for (int d = 0; d < D; ++d) {
        node_box[node * 2 * D + d] = blo[d];
        node_box[node * 2 * D + D + d] = bhi[d];
    }
    if (M == 1) parent[node] = -1;                  // a single leaf is its own root
    T* r = leaf_rec + i * RS;
    for (int d = 0; d < D; ++d) { r[d] = blo[d]; r[D + d] = bhi[d]; }
    r += 2 * D;
    double cm[D][D];                                  // inverse covariance as evaluate_inversed takes it
    load_inverse_covariance<T, D>(g + 1 + D, covariance_form, cm);
    for (int d = 0; d < D; ++d) r[d] = g[1 + d];
    if constexpr (D == 2) {
        const double det = determinant<T, 2>(cm);
        r[2] = T(cm[0][0]); r[3] = T(0.5 * (cm[0][1] + cm[1][0])); r[4] = T(cm[1][1]);
        r[5] = T(double(g[0]) * Kappa<2>::v * sqrt(det));
        reinterpret_cast<int*>(r + 6)[0] = comp;
    } else {
        const double c00 = cm[0][0], c01 = cm[0][1], c02 = cm[0][2], c10 = cm[1][0], c11 = cm[1][1], c12 = cm[1][2],
                     c20 = cm[2][0], c21 = cm[2][1], c22 = cm[2][2];
        const double det = determinant<T, 3>(cm);
        r[3] = T(c00); r[4] = T(0.5 * (c01 + c10)); r[5] = T(0.5 * (c02 + c20));
        r[6] = T(c11); r[7] = T(0.5 * (c12 + c21)); r[8] = T(c22);
        r[9] = T(double(g[0]) * Kappa<3>::v * sqrt(det));
        reinterpret_cast<int*>(r + 10)[0] = comp;
    }
}

// Boxes of the internal nodes without a walk through the tree.  Internal node i covers the leaves first ... last of the
// Morton order (its range), so its box is a range union over the leaf boxes, and min / max are idempotent: the union
// over any range is the union of two overlapping runs of 2^k leaves (a sparse table).  The leaves of all mixtures are
// numbered through and cut into blocks of kBoxBlock; the workgroup of a block
//   * writes the records and boxes of its leaves (lanes 0 ... kBoxBlock-1) while the other half of its lanes builds
//     the internal nodes with the same numbers (node i lies inside its own range; both are short chains of dependent
//     memory reads that do not depend on each other),
//   * builds the table of its leaf boxes in LDS (order-preserving integers: the same unions, bit for bit, as integer
//     atomic min / max would give) and looks up the box of every node whose range lies inside the block,
//   * leaves, for every leaf, the unions from the start of the block up to the leaf and from the leaf up to the end of
//     the block in run_box (the latter of the first leaf is the union of the whole block).
// The few nodes whose range crosses a block border get their box in the next launch (bvh_child_boxes_kernel): the run
// from the first leaf of the range to the end of its block, the whole blocks in between, the run from the start of the
// last block to the last leaf.  No step waits for another node: the bottom-up walk this replaces was a chain of one
// atomic round trip per tree level.
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void bvh_leaves_kernel(const T* __restrict__ mixture, double threshold, int mode,
                                                           const uint32_t* __restrict__ order,
                                                           const uint32_t* __restrict__ keys, T* __restrict__ node_box,
                                                           T* __restrict__ leaf_rec,
                                                           typename OrderedInt<T>::type* __restrict__ run_box,
                                                           int2* __restrict__ children, int* __restrict__ parent,
                                                           int2* __restrict__ node_range, int M, size_t total,
                                                           bool covariance_form, T* __restrict__ sums,
                                                           unsigned own_blocks, SortJob rider) {
    using Enc = typename OrderedInt<T>::type;
    constexpr int kLevels = 8;                              // runs of 1, 2, ... 128 leaves
    static_assert(kBoxBlock == 128 && kBlock == 2 * kBoxBlock, "one half of the lanes per leaf, the other per node");
    __shared__ Enc table[kLevels][2 * D][kBoxBlock];
    // The sort of the query points does not depend on the trees: a pass of it rides behind this kernel's own
    // workgroups, on compute units that would idle otherwise, instead of lengthening a pass of the leaves' sort.
    if (blockIdx.x >= own_blocks) { radix_scatter_pass(rider, blockIdx.x - own_blocks); return; }
    const size_t first_leaf = size_t(blockIdx.x) * kBoxBlock;
    const int idx = threadIdx.x & (kBoxBlock - 1);
    const bool node_lane = threadIdx.x >= kBoxBlock;
    const size_t t = first_leaf + idx;
    const size_t bl = t < total ? t / M : 0;
    const int leaf = int(t - bl * M);
    // The searches of a node (its range, its split) read keys at distances 1, 2, 4 ... from the node, each read after
    // the one before: the keys around the block wait in LDS, only the long steps of the nodes with long ranges go to
    // memory.  (Measured with all 16384 keys of a tree in LDS: the fetch costs more than the remaining memory reads.)
    constexpr int kBefore = 192, kWindow = 2 * kBlock;
    __shared__ uint32_t window[kWindow];
    const long long window_first = (long long)first_leaf - kBefore;
    for (int k = threadIdx.x; k < kWindow; k += kBlock) {
        const long long g = window_first + k;
        window[k] = g >= 0 && g < (long long)total ? keys[g] : 0u;
    }
    const int comp = !node_lane && t < total ? int(order[t]) : 0;
    __syncthreads();
    bool inside = false;                                    // node lanes: the node's range lies inside this block
    int range_lo = 0, range_hi = 0;                         // ... as slots of the block
    if (!node_lane) {
        Enc lo[D], hi[D];
        for (int d = 0; d < D; ++d) { lo[d] = OrderedInt<T>::kEmptyLo; hi[d] = OrderedInt<T>::kEmptyHi; }
        if (t < total) {
            T blo[D], bhi[D];
            const int c = (comp >= 0 && comp < M) ? comp : 0;      // a permutation by construction; never index out of bounds
            write_leaf<T, D>(mixture + (bl * M + c) * (1 + D + D * D), threshold, mode, covariance_form, node_box, leaf_rec, parent,
                             sums, M, bl, leaf, c, blo, bhi);
            for (int d = 0; d < D; ++d) { lo[d] = ordered_bits(blo[d]); hi[d] = ordered_bits(bhi[d]); }
        }
        for (int d = 0; d < D; ++d) { table[0][d][idx] = lo[d]; table[0][D + d][idx] = hi[d]; }
    } else if (t < total && leaf < M - 1) {
        // lane <-> internal node `leaf` of its mixture (there are M-1 of them)
        const long long shift = (long long)(bl * M) - window_first;       // key j of the mixture waits in slot j + shift
        const uint32_t* k = keys + bl * M;
        const int2 r = build_internal_node([&](int j) {
            const long long slot = j + shift;
            return slot >= 0 && slot < kWindow ? window[slot] : k[j];
        }, children, parent, node_range, M, bl, leaf);
        const size_t lo = bl * M + r.x, hi = bl * M + r.y;
        inside = lo >= first_leaf && hi < first_leaf + kBoxBlock;
        range_lo = int(lo - first_leaf);
        range_hi = int(hi - first_leaf);
    }
    __syncthreads();
    {
        // lane (i, h): entry i of every level, the lower bounds (h = 0: minima) or the upper bounds (h = 1: maxima); the
        // entry of the level before stays in registers
        const int h = threadIdx.x >> 7;
        Enc run[D];
        for (int d = 0; d < D; ++d) run[d] = table[0][h * D + d][idx];
        for (int k = 1; k < kLevels; ++k) {
            const int other = idx + (1 << (k - 1));
            if (other < kBoxBlock)                           // (runs that leave the block are never read)
                for (int d = 0; d < D; ++d) {
                    const Enc b = table[k - 1][h * D + d][other];
                    run[d] = h == 0 ? (b < run[d] ? b : run[d]) : (b > run[d] ? b : run[d]);
                }
            for (int d = 0; d < D; ++d) table[k][h * D + d][idx] = run[d];
            __syncthreads();
        }
    }
    // union of the leaf boxes in slots a ... b of the block
    auto range_union = [&](int a, int b, Enc (&out)[2 * D]) {
        const int k = 31 - __clz(b - a + 1);
        const int second = b + 1 - (1 << k);
        for (int c = 0; c < 2 * D; ++c) {
            const Enc u = table[k][c][a], v = table[k][c][second];
            out[c] = c < D ? (v < u ? v : u) : (v > u ? v : u);
        }
    };
    if (inside) {
        Enc u[2 * D];
        range_union(range_lo, range_hi, u);
        T* dst = node_box + (bl * (2 * size_t(M) - 1) + leaf) * 2 * D;
        for (int c = 0; c < 2 * D; ++c) dst[c] = from_ordered_bits(u[c]);
    }
    if (!node_lane) {
        // for the ranges that cross a block border: the unions from the first leaf of the block up to this one and from this
        // one up to the last leaf of the block
        Enc u[2 * D];
        range_union(0, idx, u);
        Enc* dst = run_box + t * 4 * D;
        for (int c = 0; c < 2 * D; ++c) dst[c] = u[c];
        range_union(idx, kBoxBlock - 1, u);
        for (int c = 0; c < 2 * D; ++c) dst[2 * D + c] = u[c];
    }
}

template <typename T>
__device__ __forceinline__ T wave_min(T v) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) { const T o = __shfl_xor(v, off, 64); v = o < v ? o : v; }
    return v;
}
template <typename T>
__device__ __forceinline__ T wave_max(T v) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) { const T o = __shfl_xor(v, off, 64); v = o > v ? o : v; }
    return v;
}

// Where a descent starts.  The first levels below the root hold one, two, four ... nodes, and a descent spends a memory
// round trip on each of them with most lanes idle; every descent of the tree goes through them.  One wavefront walks
// the tree breadth-first as long as a level consists of internal nodes only and the next has at most kFrontier entries,
// and leaves that level's nodes in the object: the descents push all of them at once (their children are tested in
// the first step; a subtree that is entered without need costs one step of one lane).  out[0] = count, then the nodes.
__device__ __forceinline__ void tree_frontier(const int2* __restrict__ kids, int M, int* __restrict__ out, int lane) {
    __shared__ int level[4][kFrontier];                     // one wavefront of the workgroup per mixture
    int* cur = level[threadIdx.x >> 6];
    int n = 1;
    if (lane == 0) cur[0] = 0;
    for (int depth = 0; depth < 16; ++depth) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (2 * n > kFrontier) break;
        const int node = lane < n ? cur[lane] : 0;
        const int2 ch = lane < n ? kids[node] : make_int2(0, 0);
        const bool leaf_below = lane < n && (ch.x < 0 || ch.y < 0);
        if (__ballot(leaf_below) != 0ull) break;            // the next level would not be internal nodes only
        __builtin_amdgcn_wave_barrier();                    // every lane has read its node before the level is overwritten
        if (lane < n) { cur[2 * lane] = ch.x; cur[2 * lane + 1] = ch.y; }
        n *= 2;
    }
    if (lane == 0) out[0] = n;
    if (lane < n) out[1 + lane] = cur[lane];
}

// Second half of the boxes, lane <-> node (internal nodes and leaves): the node takes its own box -- a leaf's and that
// of an internal node whose range lies inside one block of kBoxBlock leaves from bvh_leaves_kernel, otherwise the union
// of the runs at both ends of the range and of the whole blocks in between (run_box; up to kNearBlocks whole blocks by
// the lane itself in one batch of loads, more -- a handful of nodes next to the root -- by the whole wavefront) -- and
// stores it with its parent (child_box; traversals test both children of a node with one fetch) and, where it was not
// known before, as its node box.  Which child it is, an internal node reads off its own range (the left child of a
// node that splits behind leaf s is internal node s, the last leaf of its own range; the right child is s + 1, the
// first of its own range); a leaf looks at its parent's children.  No lane waits for another node.
// Behind these workgroups: a pass of the points' sort (see bvh_leaves_kernel), then one wavefront per tree that finds
// where descents start.
constexpr int kNearBlocks = 8;

template <typename T, int D>
__global__ __launch_bounds__(kBlock) void bvh_child_boxes_kernel(const int2* __restrict__ children, const int* __restrict__ parent,
                                                                const int2* __restrict__ node_range,
                                                                const typename OrderedInt<T>::type* __restrict__ run_box,
                                                                T* node_box, T* __restrict__ child_box, int M, size_t total,
                                                                CandidateCache cache, size_t point_groups,
                                                                unsigned own_blocks, SortJob rider, int* __restrict__ frontier,
                                                                size_t mixtures) {
    using Enc = typename OrderedInt<T>::type;
    if (blockIdx.x >= own_blocks + rider.blocks) {
        const size_t bl = size_t(blockIdx.x - own_blocks - rider.blocks) * (kBlock / kWave) + (threadIdx.x >> 6);
        if (bl < mixtures) tree_frontier(children + bl * (M - 1), M, frontier + bl * (1 + kFrontier), threadIdx.x & 63);
        return;
    }
    if (blockIdx.x >= own_blocks) { radix_scatter_pass(rider, blockIdx.x - own_blocks); return; }
    const size_t t = size_t(blockIdx.x) * kBlock + threadIdx.x;          // nodes of all trees, numbered through
    const int lane = threadIdx.x & 63;
    if (cache.count) {                               // a new tree: no candidate list is known yet
        for (size_t j = t; j < point_groups; j += size_t(own_blocks) * kBlock) cache.count[j] = -1;
    }
    const size_t n_nodes = 2 * size_t(M) - 1;
    const bool active = t < total;
    const size_t bl = active ? t / n_nodes : 0;
    const int node = active ? int(t - bl * n_nodes) : 0;
    const bool internal = active && node < M - 1;
    // union of the whole block b
    auto block_union = [&](size_t b) { return run_box + b * kBoxBlock * 4 * D + 2 * D; };
    const int up = active ? parent[bl * n_nodes + node] : -1;
    const int2 range = internal ? node_range[bl * (M - 1) + node] : make_int2(0, 0);
    const size_t lo = bl * M + range.x, hi = bl * M + range.y;
    const size_t b_lo = lo / kBoxBlock, b_hi = hi / kBoxBlock;
    const bool far = b_lo != b_hi;
    Enc box[2 * D];
    {
        const T* src = node_box + (bl * n_nodes + node) * 2 * D;      // written by the launch before, unless `far`
        for (int d = 0; d < 2 * D; ++d) box[d] = ordered_bits(src[d]);
    }
    // a leaf: which child of its parent?
    int side = node == range.y ? 0 : 1;
    if (active && !internal && up >= 0 && up < M - 1) side = children[bl * (M - 1) + up].x == ~(node - (M - 1)) ? 0 : 1;
    bool wide = false;
    if (far) {
        const Enc* head = run_box + lo * 4 * D + 2 * D;     // from the first leaf of the range to the end of its block
        const Enc* tail = run_box + hi * 4 * D;             // from the start of the last block to the last leaf of the range
        const size_t whole = b_hi - b_lo - 1;
        Enc v[2 + kNearBlocks][2 * D];
        for (int d = 0; d < 2 * D; ++d) { v[0][d] = head[d]; v[1][d] = tail[d]; }
        const bool near = whole <= size_t(kNearBlocks);
#pragma unroll
        for (int q = 0; q < kNearBlocks; ++q) {              // all loads in flight together
            const Enc* src = block_union(near && size_t(q) < whole ? b_lo + 1 + q : b_lo);
            for (int d = 0; d < 2 * D; ++d) v[2 + q][d] = src[d];
        }
        for (int d = 0; d < 2 * D; ++d) box[d] = v[0][d];
#pragma unroll
        for (int q = 1; q < 2 + kNearBlocks; ++q) {
            const bool use = q < 2 || (near && size_t(q - 2) < whole);
            for (int d = 0; d < D; ++d) {
                box[d] = use && v[q][d] < box[d] ? v[q][d] : box[d];
                box[D + d] = use && v[q][D + d] > box[D + d] ? v[q][D + d] : box[D + d];
            }
        }
        wide = !near;
    }
    unsigned long long todo = __ballot(wide);
    while (todo) {
        const int src = __ffsll((long long)todo) - 1;
        todo &= todo - 1;
        const size_t first = __shfl(b_lo, src, kWave) + 1, last = __shfl(b_hi, src, kWave) - 1;
        Enc acc[2 * D];
        for (int d = 0; d < D; ++d) { acc[d] = OrderedInt<T>::kEmptyLo; acc[D + d] = OrderedInt<T>::kEmptyHi; }
        for (size_t b0 = first; b0 <= last; b0 += 4 * kWave) {
            Enc v[4][2 * D];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const size_t b = b0 + q * kWave + lane;
                const Enc* from = block_union(b <= last ? b : first);
                for (int d = 0; d < 2 * D; ++d) v[q][d] = from[d];
            }
#pragma unroll
            for (int q = 0; q < 4; ++q)
                for (int d = 0; d < D; ++d) {
                    acc[d] = v[q][d] < acc[d] ? v[q][d] : acc[d];
                    acc[D + d] = v[q][D + d] > acc[D + d] ? v[q][D + d] : acc[D + d];
                }
        }
        for (int d = 0; d < D; ++d) { acc[d] = wave_min(acc[d]); acc[D + d] = wave_max(acc[D + d]); }
        if (lane == src)
            for (int d = 0; d < D; ++d) {
                box[d] = acc[d] < box[d] ? acc[d] : box[d];
                box[D + d] = acc[D + d] > box[D + d] ? acc[D + d] : box[D + d];
            }
    }
    if (!active) return;
    T out[2 * D];
    for (int d = 0; d < 2 * D; ++d) out[d] = from_ordered_bits(box[d]);
    if (far) {
        T* own = node_box + (bl * n_nodes + node) * 2 * D;
        for (int d = 0; d < 2 * D; ++d) own[d] = out[d];
    }
    if (up >= 0 && up < M - 1) {
        T* dst = child_box + ((bl * (M - 1) + up) * 2 + side) * 2 * D;
        for (int d = 0; d < 2 * D; ++d) dst[d] = out[d];
    }
}

// ---------------------------------------------------------------------------------------------------------------
// small trees: the whole build in one launch
// ---------------------------------------------------------------------------------------------------------------
// The chain of launches above costs about ten launch latencies whatever the size of the trees.  Mixtures of at most
// kSmallTreeMax components with at most kCoarseOrderMax query points per segment (the shapes of network layers:
// hundreds of mixtures of 64 ... 128 components) are built by ONE launch instead: a workgroup (a single wavefront for
// trees of at most 64 leaves) builds its tree entirely in LDS -- bounds of the centres, Morton codes, a bitonic sort of the unique keys (code << 32 | component: any
// sorting network gives the stable order), leaf boxes and records, the radix tree, the bottom-up box unions with LDS
// atomics, the decoded boxes (every node stores its own box with its parent), the cut below the root -- and the
// workgroups behind the trees' Morton-order one segment of query points each (bounds, one stable counting pass over
// the top 8 key bits).  Same trees and boxes as the chain of launches, bit for bit; the order of the points may differ
// where a point lies on the border of a Morton cell (any order of the points gives the same sums).
constexpr int kSmallTreeMax = 1024;
static int g_build_path = 0;            // test knob (gmc_bvh_set_build_path): 1 = always the chain of launches, 2 = and the
                                        // leaves' sort always as four radix passes

template <typename T> struct SmallBuild {
    T* node_box; T* child_box; T* leaf_rec; T* sums;
    int2* children; int* parent; int2* node_range; int* leaf_comp; uint32_t* g_keys; int* frontier;
    int* p_order; int* cand_count; int* ctl;
    double threshold;
    int mode, covariance_form, M, N, per_mixture /* 64-point groups per mixture */, sort_points;
    unsigned tree_blocks;
};

// Morton order of one segment of at most kCoarseOrderMax query points by the top 8 bits of their keys, stable.  Wavefront
// w owns a contiguous quarter of the points: per-wavefront digit counts, one scan, then every wavefront places its
// points round by round on its own (ranks inside a round from ballots), without workgroup barriers.
struct SmallPointsLds {
    uint32_t whist[4][256];
    uint32_t wtotal[4];
};

// (PP: points per lane, at least N / 256; the points stay in registers between the two passes and all their loads are in
// flight at once -- a loop that waits for every point's load would cost a memory round trip per 256 points)
template <typename T, int D, int PP>
__device__ __forceinline__ void order_points_small(const T* __restrict__ p, int N, int* __restrict__ order, T (*red)[kBlock],
                                                   SmallPointsLds& s) {
    uint32_t (*whist)[256] = s.whist;
    uint32_t* wtotal = s.wtotal;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int share = (N + kBlock - 1) / kBlock * kWave;
    const int begin = wave * share, end = begin + share < N ? begin + share : N;
    T x[PP][D];
#pragma unroll
    for (int r = 0; r < PP; ++r) {
        const int i = begin + r * kWave + lane;
#pragma unroll
        for (int d = 0; d < D; ++d) x[r][d] = i < end ? p[size_t(i) * D + d] : T(0);
    }
    T lo[D], hi[D];
    for (int d = 0; d < D; ++d) { lo[d] = T(INFINITY); hi[d] = T(-INFINITY); }
#pragma unroll
    for (int r = 0; r < PP; ++r)
        if (begin + r * kWave + lane < end)
            for (int d = 0; d < D; ++d) {
                lo[d] = x[r][d] < lo[d] ? x[r][d] : lo[d];
                hi[d] = x[r][d] > hi[d] ? x[r][d] : hi[d];
            }
    for (int w = 0; w < 4; ++w) whist[w][threadIdx.x] = 0u;
    block_bounds<T, D>(lo, hi, red);
    // The top 8 bits of the 30-bit key, i.e. bits 9, 8 (and 7 of the first two axes) of the 10-bit cell coordinates.  The
    // order of the points only groups neighbours: the cell is formed with one reciprocal per axis instead of a division
    // per coordinate (a point on a cell border may land in the neighbouring cell, which is as good a group).
    T base[D], scale[D];
    for (int d = 0; d < D; ++d) {
        const T ext = red[D + d][0] - red[d][0];
        base[d] = red[d][0];
        scale[d] = ext > T(0) ? T(1024) / ext : T(0);
    }
    uint32_t digit[PP];
#pragma unroll
    for (int r = 0; r < PP; ++r) {
        uint32_t cell[3] = {0u, 0u, 0u};
#pragma unroll
        for (int d = 0; d < D; ++d) {
            T q = (x[r][d] - base[d]) * scale[d];
            q = q < T(0) ? T(0) : (q > T(1023) ? T(1023) : q);
            q = (q == q) ? q : T(0);
            cell[d] = uint32_t(q);
        }
        digit[r] = ((cell[0] >> 9) & 1u) << 7 | ((cell[1] >> 9) & 1u) << 6 | ((cell[2] >> 9) & 1u) << 5 |
                   ((cell[0] >> 8) & 1u) << 4 | ((cell[1] >> 8) & 1u) << 3 | ((cell[2] >> 8) & 1u) << 2 |
                   ((cell[0] >> 7) & 1u) << 1 | ((cell[1] >> 7) & 1u);
        if (begin + r * kWave + lane < end) atomicAdd(&whist[wave][digit[r]], 1u);
    }
    __syncthreads();
    {   // thread d: first slot of digit d for every wavefront
        uint32_t c[4], mine = 0;
        for (int w = 0; w < 4; ++w) { c[w] = whist[w][threadIdx.x]; mine += c[w]; }
        uint32_t scan = mine;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const uint32_t up = __shfl_up(scan, off, kWave);
            scan += lane >= off ? up : 0u;
        }
        if (lane == kWave - 1) wtotal[wave] = scan;
        __syncthreads();
        for (int w = 0; w < wave; ++w) scan += wtotal[w];
        uint32_t at = scan - mine;
        for (int w = 0; w < 4; ++w) { whist[w][threadIdx.x] = at; at += c[w]; }
    }
    __syncthreads();
    const unsigned long long below = (1ull << lane) - 1ull;
#pragma unroll
    for (int r = 0; r < PP; ++r) {
        if (begin + r * kWave >= end) break;                // (wave-uniform)
        const int i = begin + r * kWave + lane;
        const bool valid = i < end;
        const uint32_t dg = valid ? digit[r] : 0u;
        unsigned long long same = __ballot(valid);
#pragma unroll
        for (int bit = 0; bit < 8; ++bit) {
            const unsigned long long m = __ballot((dg >> bit) & 1u);
            same &= ((dg >> bit) & 1u) ? m : ~m;
        }
        const int rank = __popcll(same & below);
        uint32_t slot = 0;
        if (valid) slot = whist[wave][dg] + rank;
        wave_lds_fence();
        if (valid) {
            if (slot < uint32_t(N)) order[slot] = i;        // always true for consistent counts
            if (rank == 0) whist[wave][dg] = slot + uint32_t(__popcll(same));
        }
        wave_lds_fence();
    }
}

// LDS of one tree that THREADS lanes build, K leaves per lane
template <typename T, int D, int THREADS, int K> struct SmallTreeLds {
    static constexpr int kCap = THREADS * K;
    using Enc = typename OrderedInt<T>::type;
    unsigned long long keys[kCap];              // code << 32 | component, sorted in place
    int parent[2 * kCap];                       // [0, M-1): internal nodes, [M-1, 2M-1): leaves
    int2 kids[kCap];
    Enc box[kCap][2 * D];                       // boxes of the internal nodes, order-preserving integers
};

// The lanes that build one tree wait for each other: a wavefront (its LDS traffic ordered) or the workgroup.  (Trees of
// 128 lanes share a workgroup in pairs and go through the same barriers side by side: every tree of a launch has the
// same number of leaves, and the loops whose length depends on the data hold no barrier.)
template <int THREADS> __device__ __forceinline__ void tree_sync() {
    if constexpr (THREADS == kWave) wave_lds_fence(); else __syncthreads();
}

// Tree bl by THREADS lanes (tid = 0 ... THREADS-1): one wavefront (trees of at most 64 leaves: four trees per
// workgroup, no workgroup barriers) or the whole workgroup.
template <typename T, int D, int THREADS, int K>
__device__ __forceinline__ void build_small_tree(const T* __restrict__ mixture, const SmallBuild<T>& a, size_t bl, int tid,
                                                 SmallTreeLds<T, D, THREADS, K>& s, T (*red)[kBlock]) {
    constexpr int G = 1 + D + D * D;
    using Enc = typename OrderedInt<T>::type;
    const int M = a.M;
    // a new tree: no candidate list is known yet
    if (a.cand_count)
        for (int g = tid; g < a.per_mixture; g += THREADS) a.cand_count[bl * a.per_mixture + g] = -1;
    // bounds of the centres and keys
    T c[K][D], bounds[2 * D];
    // one leaf per lane: the lane keeps ITS component (the whole record is fetched with the centre, one round trip) and
    // learns the leaf it becomes from the sort
    T rec[K == 1 ? G : 1];
    {
        T lo[D], hi[D];
        for (int d = 0; d < D; ++d) { lo[d] = T(INFINITY); hi[d] = T(-INFINITY); }
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int i = tid + k * THREADS;
            if constexpr (K == 1) {
#pragma unroll
                for (int q = 0; q < G; ++q) rec[q] = i < M ? mixture[(bl * M + i) * G + q] : T(0);
            }
            for (int d = 0; d < D; ++d) {
                if constexpr (K == 1) c[k][d] = rec[1 + d];
                else c[k][d] = i < M ? mixture[(bl * M + i) * G + 1 + d] : T(0);
                if (i < M) {
                    lo[d] = c[k][d] < lo[d] ? c[k][d] : lo[d];       // a NaN coordinate is skipped
                    hi[d] = c[k][d] > hi[d] ? c[k][d] : hi[d];
                }
            }
        }
        for (int d = 0; d < D; ++d) { bounds[d] = wave_min(lo[d]); bounds[D + d] = wave_max(hi[d]); }
        if constexpr (THREADS > kWave) {                    // combine the wavefronts of this tree
            const int wave = threadIdx.x >> 6, first = (threadIdx.x / THREADS) * (THREADS / kWave);
            T mine = bounds[0];
            for (int k = 1; k < 2 * D; ++k) mine = int(threadIdx.x & 63) == k ? bounds[k] : mine;
            if ((threadIdx.x & 63) < 2 * D) red[threadIdx.x & 63][wave] = mine;
            __syncthreads();
            for (int k = 0; k < 2 * D; ++k) bounds[k] = red[k][first];
            for (int w = 1; w < THREADS / kWave; ++w)
                for (int d = 0; d < D; ++d) {
                    const T a = red[d][first + w], b = red[D + d][first + w];
                    bounds[d] = a < bounds[d] ? a : bounds[d];
                    bounds[D + d] = b > bounds[D + d] ? b : bounds[D + d];
                }
        }
    }
    int leaf_of[K];                                         // the leaf (Morton order) whose box and record lane slot k writes
    T blo[K][D], bhi[K][D];
    if constexpr (K == 1) {
        // Sort by counting: the leaf of component i is the number of unique keys below its own (every read a broadcast,
        // no step waits for another); the keys then move to their places for the tree build.
        const unsigned long long mine = tid < M ? ((unsigned long long)morton30<T, D>(c[0], bounds) << 32) | (unsigned)tid : ~0ull;
        if (tid < M) s.keys[tid] = mine;
        tree_sync<THREADS>();
        int rank = 0;
#pragma unroll 8
        for (int j = 0; j < M; ++j) rank += s.keys[j] < mine ? 1 : 0;
        tree_sync<THREADS>();                               // every lane has counted before the keys move
        if (tid < M) s.keys[rank] = mine;
        leaf_of[0] = rank;
        if (tid < M) {
            a.g_keys[bl * M + rank] = uint32_t(mine >> 32);
            a.leaf_comp[bl * M + rank] = tid;
            write_leaf<T, D>(rec, a.threshold, a.mode, a.covariance_form != 0, a.node_box, a.leaf_rec, a.parent, a.sums, M, bl,
                             rank, tid, blo[0], bhi[0]);
        }
        tree_sync<THREADS>();                               // the sorted keys are in place
    } else {
        int Mp = 1;
        while (Mp < M) Mp <<= 1;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int i = tid + k * THREADS;
            if (i < Mp) s.keys[i] = i < M ? ((unsigned long long)morton30<T, D>(c[k], bounds) << 32) | (unsigned)i : ~0ull;
        }
        tree_sync<THREADS>();
        // bitonic sort of the unique keys
        for (int size = 2; size <= Mp; size <<= 1)
            for (int stride = size >> 1; stride > 0; stride >>= 1) {
                for (int q = tid; q < Mp / 2; q += THREADS) {
                    const int i0 = ((q & ~(stride - 1)) << 1) | (q & (stride - 1)), i1 = i0 | stride;
                    const unsigned long long k0 = s.keys[i0], k1 = s.keys[i1];
                    if ((k0 > k1) == ((i0 & size) == 0)) { s.keys[i0] = k1; s.keys[i1] = k0; }
                }
                tree_sync<THREADS>();
            }
        // leaves: lane <-> leaf i (Morton order)
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int i = tid + k * THREADS;
            leaf_of[k] = i;
            if (i < M) {
                const unsigned long long key = s.keys[i];
                int comp = int(unsigned(key));
                comp = (comp >= 0 && comp < M) ? comp : 0;  // a permutation by construction; never index out of bounds
                a.g_keys[bl * M + i] = uint32_t(key >> 32);
                a.leaf_comp[bl * M + i] = comp;
                write_leaf<T, D>(mixture + (bl * M + comp) * G, a.threshold, a.mode, a.covariance_form != 0, a.node_box, a.leaf_rec,
                                 a.parent, a.sums, M, bl, i, comp, blo[k], bhi[k]);
            }
        }
    }
    // below: lane <-> internal node i
    if (M < 2) return;
    int* par = a.parent + bl * (2 * size_t(M) - 1);
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int i = tid + k * THREADS;
        if (i < M - 1) {
            int first, last, left, right;
            radix_tree_node([&](int j) { return uint32_t(s.keys[j] >> 32); }, M, i, first, last, left, right);
            a.children[bl * (M - 1) + i] = make_int2(left, right);
            a.node_range[bl * (M - 1) + i] = make_int2(first, last);
            s.kids[i] = make_int2(left, right);
            const int li = left >= 0 ? left : (M - 1) + ~left, ri = right >= 0 ? right : (M - 1) + ~right;
            par[li] = i; par[ri] = i;
            s.parent[li] = i; s.parent[ri] = i;
            if (i == 0) { par[0] = -1; s.parent[0] = -1; }
            for (int d = 0; d < D; ++d) { s.box[i][d] = OrderedInt<T>::kEmptyLo; s.box[i][D + d] = OrderedInt<T>::kEmptyHi; }
        }
    }
    tree_sync<THREADS>();
    // Bottom-up unions without inter-lane ordering: every leaf walks towards the root and merges ITS OWN box into every
    // ancestor with atomic min/max, as long as it still enlarges the ancestor; it stops at the first ancestor that
    // already contains it.  Every extreme of that ancestor was set by some walker that enlarged it and therefore walks
    // on itself, so all higher ancestors end up containing the stopped box as well: the final boxes are the exact
    // unions of the leaves below each node.  Nothing is read back before the barrier except the atomics' own results.
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int i = tid + k * THREADS;
        if (i < M) {
            Enc lo[D], hi[D];
            for (int d = 0; d < D; ++d) { lo[d] = ordered_bits(blo[k][d]); hi[d] = ordered_bits(bhi[k][d]); }
            int node = s.parent[(M - 1) + leaf_of[k]];
            for (int level = 0; node >= 0 && node < M - 1 && level < 128; ++level) {
                bool grew = false;
                for (int d = 0; d < D; ++d) {
                    grew |= lo[d] < atomicMin(&s.box[node][d], lo[d]);
                    grew |= hi[d] > atomicMax(&s.box[node][D + d], hi[d]);
                }
                if (!grew) break;
                node = s.parent[node];
            }
        }
    }
    tree_sync<THREADS>();
    // every node stores its box with its parent (child_box) and, internal nodes, as its own node box
    const size_t nbase = bl * (2 * size_t(M) - 1);
    T* cb = a.child_box + bl * (M - 1) * 4 * D;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int i = tid + k * THREADS;
        if (i < M - 1) {
            T v[2 * D];
            for (int d = 0; d < 2 * D; ++d) v[d] = from_ordered_bits(s.box[i][d]);
            for (int d = 0; d < 2 * D; ++d) a.node_box[(nbase + i) * 2 * D + d] = v[d];
            const int up = s.parent[i];
            if (up >= 0 && up < M - 1) {
                const int side = s.kids[up].x == i ? 0 : 1;
                for (int d = 0; d < 2 * D; ++d) cb[(size_t(up) * 2 + side) * 2 * D + d] = v[d];
            }
        }
        if (i < M) {
            const int up = s.parent[(M - 1) + leaf_of[k]];
            if (up >= 0 && up < M - 1) {
                const int side = s.kids[up].x == ~leaf_of[k] ? 0 : 1;
                for (int d = 0; d < D; ++d) {
                    cb[(size_t(up) * 2 + side) * 2 * D + d] = blo[k][d];
                    cb[(size_t(up) * 2 + side) * 2 * D + D + d] = bhi[k][d];
                }
            }
        }
    }
    if (tid < kWave) tree_frontier(s.kids, M, a.frontier + bl * (1 + kFrontier), tid);
}

template <typename T, int D, int THREADS, int K, int PP>
__global__ __launch_bounds__(kBlock) void bvh_build_small_kernel(const T* __restrict__ mixture, const T* __restrict__ xes,
                                                                SmallBuild<T> a, size_t mixtures) {
    using Trees = SmallTreeLds<T, D, THREADS, K>[kBlock / THREADS];
    __shared__ T red[2 * D][kBlock];
    // a workgroup builds trees or orders points: one piece of LDS for either
    __shared__ __attribute__((aligned(16))) unsigned char lds[sizeof(Trees) > sizeof(SmallPointsLds) ? sizeof(Trees) : sizeof(SmallPointsLds)];
    Trees& trees = *reinterpret_cast<Trees*>(lds);
    if (blockIdx.x == 0 && threadIdx.x < 4) a.ctl[threadIdx.x] = 0;     // a new tree: no published pieces, no error
    if (blockIdx.x >= a.tree_blocks) {
        const size_t seg = blockIdx.x - a.tree_blocks;
        const int N = a.N;
        int* order = a.p_order + seg * N;
        if (!a.sort_points) { for (int i = threadIdx.x; i < N; i += kBlock) order[i] = i; return; }
        order_points_small<T, D, PP>(xes + seg * N * D, N, order, red, *reinterpret_cast<SmallPointsLds*>(lds));
        return;
    }
    const int sub = threadIdx.x / THREADS;                  // trees of THREADS lanes: kBlock / THREADS of them per workgroup
    size_t bl = size_t(blockIdx.x) * (kBlock / THREADS) + sub;
    if constexpr (THREADS == kWave) {
        if (bl >= mixtures) return;                         // (a wavefront on its own: no barriers ahead)
    } else {
        bl = bl < mixtures ? bl : mixtures - 1;             // a spare half builds the last tree once more: same values, same barriers
    }
    build_small_tree<T, D, THREADS, K>(mixture, a, bl, threadIdx.x % THREADS, trees[sub], red);
}

// ---------------------------------------------------------------------------------------------------------------
// traversal
// ---------------------------------------------------------------------------------------------------------------
// closed-interval test of a point against a box given as (lower[D], upper[D]); every comparison is evaluated
// (no short-circuit), so the box scalars can be fetched with one wide load before the test
template <typename T, int D>
__device__ __forceinline__ bool inside_box(const T (&x)[D], const T* box) {
    bool in = true;
#pragma unroll
    for (int d = 0; d < D; ++d) in = in & (x[d] >= box[d]) & (x[d] <= box[D + d]);
    return in;
}

// exp(-q / 2); `tab` is the workgroup's exp2 table (float: none)
template <typename T>
__device__ __forceinline__ T exp_neg_half(T q, const T* __restrict__ tab) {
    return pair_exp2(q * T(-0.72134752044448170368), tab);
}

// e = exp(-1/2 t^T C t), u = C t for the leaf record r
template <typename T, int D>
__device__ __forceinline__ T leaf_terms(const T* __restrict__ r, const T* __restrict__ tab, const T (&x)[D], T (&t)[D],
                                        T (&u)[D]) {
    if constexpr (D == 2) {
        t[0] = x[0] - r[0]; t[1] = x[1] - r[1];
        u[0] = fma_(r[2], t[0], r[3] * t[1]);
        u[1] = fma_(r[3], t[0], r[4] * t[1]);
        return exp_neg_half(fma_(t[0], u[0], t[1] * u[1]), tab);
    } else {
        t[0] = x[0] - r[0]; t[1] = x[1] - r[1]; t[2] = x[2] - r[2];
        u[0] = fma_(r[3], t[0], fma_(r[4], t[1], r[5] * t[2]));
        u[1] = fma_(r[4], t[0], fma_(r[6], t[1], r[7] * t[2]));
        u[2] = fma_(r[5], t[0], fma_(r[7], t[1], r[8] * t[2]));
        return exp_neg_half(fma_(t[0], u[0], fma_(t[1], u[1], t[2] * u[2])), tab);
    }
}

template <int D> struct BvhSums { static constexpr int k = 1 + D + D * (D + 1) / 2; };

constexpr int kStackCap = 512;          // soft capacity of a node stack (the array has 128 more)
constexpr int kTravWaves = 8;           // wavefronts per workgroup of the traversal
constexpr int kTravBlock = kTravWaves * kWave;
constexpr int kTwoBoxLeaves = 256;      // trees with fewer leaves get one box per point group (see group_boxes)
constexpr int kGroupsMax = 4;           // 64-point groups per workgroup (each descends the tree with its own wavefront)
constexpr int kStageBatch = 20;         // candidate leaves a wavefront stages in LDS at a time
constexpr int kTravSlots = 2 * 256;     // workgroups resident at once: two per compute unit

// 64-bit stamp of the coordinates of a group's 64 points (lanes beyond the last point count as absent): what a
// candidate list is valid for.  Wave-uniform.
template <typename T, int D>
__device__ __forceinline__ unsigned long long points_stamp(const T (&x)[D], bool valid, int lane) {
    unsigned long long h = 0x9E3779B97F4A7C15ull * (unsigned long long)(lane + 1);
#pragma unroll
    for (int d = 0; d < D; ++d) {
        unsigned long long bits;
        if constexpr (sizeof(T) == 4) bits = __builtin_bit_cast(unsigned int, x[d]);
        else bits = __builtin_bit_cast(unsigned long long, x[d]);
        h = (h ^ bits) * 0xff51afd7ed558ccdull;
        h ^= h >> 29;
    }
    h = valid ? h : 0ull;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) h += __shfl_xor(h, off, 64);
    // the same value in every lane: kept in scalar registers (it stays alive until the list is published)
    const unsigned lo = __builtin_amdgcn_readfirstlane(unsigned(h)), hi = __builtin_amdgcn_readfirstlane(unsigned(h >> 32));
    return ((unsigned long long)hi << 32) | lo;
}

// Largest float not above / smallest float not below a coordinate: boxes rounded outwards stay conservative.
__device__ __forceinline__ float float_below(float x) { return x; }
__device__ __forceinline__ float float_above(float x) { return x; }
__device__ __forceinline__ float float_below(double x) {
    const float f = float(x);
    const int b = __builtin_bit_cast(int, f);               // the next float towards -inf: one step in the bit pattern
    const float down = __builtin_bit_cast(float, f > 0.0f ? b - 1 : (f < 0.0f ? b + 1 : int(0x80000001u)));
    return double(f) > x ? down : f;
}
__device__ __forceinline__ float float_above(double x) {
    const float f = float(x);
    const int b = __builtin_bit_cast(int, f);
    const float up = __builtin_bit_cast(float, f > 0.0f ? b + 1 : (f < 0.0f ? b - 1 : 1));
    return double(f) < x ? up : f;
}

// Boxes of a group's 64 points for the descent (lanes = points in Morton order; every lane gets all values, lane 0
// stores them: out = lower[D], upper[D] of the first box, then of the second).  Neighbours on the Morton curve are
// neighbours in space except where the curve jumps, and a group that straddles a jump has a bounding box that spans a
// large part of the scene: ten times the candidates of its neighbours for the same number of hits, and the launch
// ends with such groups.  The points are therefore cut where two consecutive ones lie farthest apart (L1), and the two
// runs get a box each when that at least halves the volume (extents padded by 1/32 of the whole extent, so flat
// boxes compare sensibly); otherwise both boxes are the bounding box of all points.  `may_cut` is false for small trees:
// a list cannot be longer than the tree has leaves, and the cut costs a workgroup of a launch with thousands of small
// trees more than the shorter lists save (measured with 64 and 128 leaves per tree: 8-10 % of the forward pass).
template <typename T, int D>
__device__ __forceinline__ void group_boxes(const T (&x)[D], bool valid, int lane, bool may_cut, float* __restrict__ out) {
    float lo[D], hi[D], gap = 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
        lo[d] = valid ? float_below(x[d]) : INFINITY;
        hi[d] = valid ? float_above(x[d]) : -INFINITY;
    }
    if (!may_cut) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const float wlo = wave_min(lo[d]), whi = wave_max(hi[d]);
            if (lane == 0) { out[d] = wlo; out[D + d] = whi; out[2 * D + d] = wlo; out[3 * D + d] = whi; }
        }
        return;
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
        const float mid = float(x[d]);
        gap += fabsf(__shfl_down(mid, 1, 64) - mid);
    }
    const bool next_valid = __shfl_down(valid ? 1 : 0, 1, 64) != 0 && lane < 63;
    // the jump after lane i competes with its lane index in the low bits (gap >= 0: its bit pattern is ordered)
    unsigned key = (valid && next_valid && gap == gap) ? ((__builtin_bit_cast(unsigned, gap) & ~63u) | unsigned(lane)) : 0u;
    key = wave_max(key);
    const int cut = int(key & 63u);                         // the first run ends with this lane
    const bool first = lane <= cut;
    float alo[D], ahi[D], blo[D], bhi[D];
    float part_a = 1.0f, part_b = 1.0f;                     // volumes of the two boxes as fractions of the whole (any scale)
#pragma unroll
    for (int d = 0; d < D; ++d) {
        alo[d] = wave_min(first ? lo[d] : INFINITY);  ahi[d] = wave_max(first ? hi[d] : -INFINITY);
        blo[d] = wave_min(first ? INFINITY : lo[d]);  bhi[d] = wave_max(first ? -INFINITY : hi[d]);
        const float whole = fmaxf(ahi[d], bhi[d]) - fminf(alo[d], blo[d]);
        const float pad = fmaxf(whole * (1.0f / 32.0f), 1e-30f);
        const float inv = 1.0f / (whole + pad);
        part_a *= (fmaxf(ahi[d] - alo[d], 0.0f) + pad) * inv;
        part_b *= (fmaxf(bhi[d] - blo[d], 0.0f) + pad) * inv;
    }
    // (an empty second run leaves the first one as large as the whole: no cut; NaN or infinite coordinates: no cut)
    const bool split = part_a + part_b < 0.5f;
    if (lane == 0) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const float wlo = fminf(alo[d], blo[d]), whi = fmaxf(ahi[d], bhi[d]);
            out[d] = split ? alo[d] : wlo;              out[D + d] = split ? ahi[d] : whi;
            out[2 * D + d] = split ? blo[d] : wlo;      out[3 * D + d] = split ? bhi[d] : whi;
        }
    }
}

// Traversal of one tree by a workgroup of 8 wavefronts for up to kGroupsMax groups of 64 Morton-neighbouring
// points, in two alternating phases.
//   Phase 1 (wavefront i descends for group i, lanes = tree nodes): one stack of internal nodes per group in LDS;
//   up to 64 of them are popped at a time, each lane fetches the two child boxes of its node and tests them against
//   the one or two boxes around the group's points (group_boxes; a node that contains any of the points overlaps one).
//   Overlapping internal children go back on the stack, overlapping leaves into the group's candidate list (ballot
//   + prefix-popcount compaction).  The descents of the groups are independent chains of memory round trips (about
//   one per tree level) and run side by side.
//   Phase 2 (all wavefronts, group after group, lanes = points): the candidates of a group are dealt to the
//   wavefronts; each stages kStageBatch of its candidates (own box + evaluation record, one contiguous leaf
//   record) in LDS, the records of the next batch being fetched while the current one is worked on, tests every
//   lane's point against all staged boxes (closed interval, lbvh/aabb.h:39-47; the lane keeps a bit mask of the
//   leaves that contain its point) and then evaluates, lane by lane, only the leaves of its own mask: the loop
//   runs as often as the busiest lane has hits, not once per leaf.  The per-point partial results of the
//   wavefronts are added in wavefront order (deterministic).
// Phase 1 only filters, phase 2 applies the per-point rule of lbvh/query.h:13-66, so the result is the sum over the
// Gaussians whose own box contains the point.
// MODE 0: forward.  MODE 1: backward (grad_out given): dL/dx stays in the lanes' registers.  The per-Gaussian sums
// of a batch are collected in a per-wavefront LDS copy and flushed with one global atomic per non-zero scalar:
// a leaf that contains many of the points is evaluated by all lanes at once and its sums are reduced over the
// wavefront (DPP); the remaining hits go through the lane-by-lane loop and are added with LDS atomics (a few
// cycles per instruction when the lanes of an instruction address different leaves, hence the lanes start at
// different leaves of the batch).
template <typename T, int D, int MODE, bool NEED_GM, bool NEED_GX>
__global__ __launch_bounds__(kTravBlock) __attribute__((amdgpu_waves_per_eu(4))) void bvh_traverse_kernel(
        const T* __restrict__ xes, const int* __restrict__ p_order, const T* __restrict__ child_box,
        const int2* __restrict__ children, const T* __restrict__ leaf_rec, T* __restrict__ out,
        const T* __restrict__ grad_out, T* __restrict__ sums, T* __restrict__ grad_xes, CandidateCache cache,
        T* __restrict__ piece_gx, int helpers, int L, int M, int N, int Bx, int Lx, int chunks, int groups_per_workgroup,
        int xes_shared, const int* __restrict__ frontier) {
    constexpr int LS = LeafRec<D>::kStride;
    constexpr int NR = BvhSums<D>::k;
    constexpr int kVals = MODE == 0 ? 1 : D;
    constexpr int kAmp = 2 * D + D + D * (D + 1) / 2;       // position of the amplitude inside a leaf record
    __shared__ int stack[kGroupsMax][kStackCap + 128];
    __shared__ int leaves[kGroupsMax][kLeafCap];
    __shared__ int state[kGroupsMax][2];                    // [0] candidates gathered, [1] nodes left on the stack
    __shared__ int pids[kGroupsMax][kWave];                 // index of every point, -1 beyond the end
    __shared__ T pts[kGroupsMax][D + 1][kWave];             // coordinates and upstream gradient of every point
    __shared__ float gbox[kGroupsMax][4 * D];               // two boxes (lower, upper; rounded outwards) around every group's points
    // results per point, in double: the forward sums are added wavefront by wavefront (deterministic), dL/dx with
    // LDS atomics (cheap for doubles on distinct words, unlike floats)
    __shared__ double result[kGroupsMax][kVals][kWave];
    // per wavefront: the staged leaf records of a batch
    __shared__ __attribute__((aligned(16))) T staged_mem[kTravWaves][kStageBatch * LS];
    // forward pass: what every wavefront has summed for every group in this round; added up in wavefront order when all
    // groups of the round are through (one barrier per round; with a barrier pair per group the workgroup waited for
    // its slowest wavefront once per group)
    __shared__ T partial[MODE == 0 ? kGroupsMax : 1][MODE == 0 ? kTravWaves : 1][kWave];
    // double in both precisions: LDS atomic adds of doubles on distinct addresses cost a few cycles per
    // instruction, those of floats are serialised lane by lane
    __shared__ double rsum_mem[kTravWaves][NEED_GM ? kStageBatch * NR : 1];
    __shared__ int2 pend[kGroupsMax][kPendMax];             // pieces of a group's list that wait to be published
    __shared__ int piece_valid;                             // helper workgroups: the piece still describes the group's points
    const T* exp2_tab = exp2_table<T>();                    // (published by the barrier in front of the first evaluation)
    const int per_mixture = (N + kWave - 1) / kWave;        // point groups of one mixture
    // The last `helpers` workgroups of a backward launch each take one published piece of a long candidate list
    // (no descent: one group, its points, a slice of its list); all others own `groups_per_workgroup` groups.
    // (Last, because most of them find no piece: at the end of the grid they start when compute units run idle.)
    const int owners = int(gridDim.x) - (MODE == 1 ? helpers : 0);
    const int piece = int(blockIdx.x) >= owners ? int(blockIdx.x) - owners : -1;
    int4 piece_desc = make_int4(0, 0, 0, 0);
    if (piece >= 0) {
        if (!cache.count) return;
        const int published = cache.ctl[0] < cache.pieces_max ? cache.ctl[0] : cache.pieces_max;
        if (piece >= published) return;
        piece_desc = cache.pieces[piece];
        if (piece_desc.z <= 0) return;                      // a slot whose group could not publish all its pieces
    }
    const int groups = piece >= 0 ? 1 : groups_per_workgroup;
    const int wg = piece >= 0 ? 0 : int(blockIdx.x);
    const int bl = piece >= 0 ? piece_desc.x / per_mixture : wg / chunks;
    const int chunk = wg - bl * chunks;
    const int b = bl / L, l = bl - b * L;
    const int xb = b < Bx ? b : Bx - 1, xl = l < Lx ? l : Lx - 1;
    const size_t xseg = size_t(xb) * Lx + xl;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    T* staged = staged_mem[wave];
    double* rsum = rsum_mem[wave];
    const unsigned long long below = (1ull << lane) - 1ull;

    // wavefront i loads the points of group i and their bounding box
    int sp = 0;                                             // nodes on this wavefront's stack (wave-uniform)
    int cache_slot = -1;                                    // the group whose candidate list this wavefront's descent leaves
    bool cache_ok = true;                                   // ... as long as every part of it found room
    int first_round_leaves = 0, n_pend = 0;
    bool publish = false;                                   // the group's descent has ended with all parts in place
    int piece_slot = 0, publish_slot = 0, publish_flags = 0;
    unsigned long long my_stamp = 0ull;                     // of the points this wavefront has loaded
    if (wave < groups) {
        // The groups of a workgroup lie far apart in Morton order, one in every quarter of the range and at
        // different places within the quarters: point groups with long candidate lists come in clusters (dense
        // regions), often at matching places of a symmetric point set.
        const int group = piece >= 0 ? piece_desc.x - bl * per_mixture
                                     : wave * chunks + (chunk + wave * (chunks / (groups + 1))) % chunks;
        const int j = group * kWave + lane;
        const bool valid = j < N;
        // What an earlier traversal has left for this group is fetched together with the points, not after them: each
        // of these reads is a round trip through memory, and in a chain they add up to more than the evaluation of
        // a short list.  (The group's fixed slot of the list exists whatever its state; a backward owner works on at
        // most kPieceLeaves entries of it, a piece has at most as many.)
        constexpr int kAhead = (kPieceLeaves + kWave - 1) / kWave;
        int known_ahead = -1, list_ahead[kAhead];
        unsigned long long stamp_ahead = 0ull;
        int2 range_ahead = make_int2(0, 0);
#pragma unroll
        for (int k = 0; k < kAhead; ++k) list_ahead[k] = 0;
        const bool look = cache.count && group * kWave < N && (piece >= 0 || M > 1);
        if (look) {
            const size_t slot = piece >= 0 ? size_t(piece_desc.x) : size_t(bl) * per_mixture + group;
            known_ahead = cache.count[slot];
            stamp_ahead = cache.stamp[slot];
            if (piece >= 0) range_ahead = cache.piece_range[slot];
            const int* src = piece >= 0 ? cache.list + piece_desc.y : cache.list + slot * kLeafCap;
            const int n_ahead = piece >= 0 ? piece_desc.z : kLeafCap;
#pragma unroll
            for (int k = 0; k < kAhead; ++k)
                if (lane + k * kWave < n_ahead) list_ahead[k] = src[lane + k * kWave];
        }
        // the nodes the descent starts from (tree_frontier), fetched with everything else
        int start_count = 0, start_node = 0;
        if (piece < 0 && M > 1) {
            start_count = frontier[size_t(bl) * (1 + kFrontier)];
            start_node = frontier[size_t(bl) * (1 + kFrontier) + 1 + lane];
        }
        int pid = valid ? p_order[xseg * N + j] : 0;
        pid = unsigned(pid) < unsigned(N) ? pid : 0;        // a permutation by construction; never index out of bounds
        T x[D];
#pragma unroll
        for (int d = 0; d < D; ++d) x[d] = xes[(xseg * N + pid) * D + d];
        T g = T(0);
        if (MODE == 1) g = valid ? grad_out[size_t(bl) * N + pid] : T(0);
#pragma unroll
        for (int d = 0; d < D; ++d) pts[wave][d][lane] = x[d];
        pts[wave][D][lane] = g;
        pids[wave][lane] = valid ? pid : -1;
        if (cache.count) my_stamp = points_stamp<T, D>(x, valid, lane);
        const bool any = group * kWave < N;
        start_count = __builtin_amdgcn_readfirstlane(start_count);
        start_count = start_count < 1 ? 1 : (start_count > kFrontier ? kFrontier : start_count);
        // (a count or a node outside the tree cannot come from the build; the clamps keep a bug from indexing out of bounds)
        stack[wave][lane] = (lane < start_count && unsigned(start_node) < unsigned(M - 1)) ? start_node : 0;
        if (lane == 0) {
            // a single Gaussian is a tree without internal nodes: its leaf is the only candidate
            leaves[wave][0] = 0;
            state[wave][0] = (any && M == 1) ? 1 : 0;
            state[wave][1] = 0;
        }
        sp = (any && M > 1) ? start_count : 0;
        if (piece >= 0) {
            // A piece is worked on only while it is one of the pieces its group has published last, for points with
            // the stamp of the ones loaded here; the owner of the group applies the same test to the list and
            // otherwise evaluates all of it itself.
            const int known = look ? known_ahead : -1;
            const int2 range = range_ahead;
            const bool ok = known >= 0 && (known & kCandSplit) != 0 && piece >= range.x && piece < range.x + range.y &&
                            stamp_ahead == my_stamp;
            if (lane == 0) piece_valid = ok ? 1 : 0;
#pragma unroll
            for (int k = 0; k < kAhead; ++k)
                if (lane + k * kWave < piece_desc.z) leaves[0][lane + k * kWave] = list_ahead[k];
            for (int i = lane + kAhead * kWave; i < piece_desc.z; i += kWave) leaves[0][i] = cache.list[piece_desc.y + i];
            if (lane == 0) state[0][0] = piece_desc.z;
            sp = 0;
        } else if (cache.count && sp > 0) {
            // candidate list left by an earlier traversal of this tree: no descent.  The backward pass leaves the
            // published pieces of a long list to the helper workgroups; the forward pass has no helpers, so it
            // takes a whole single-round list and descends again for a list of several rounds.
            cache_slot = bl * per_mixture + group;
            const int known = __builtin_amdgcn_readfirstlane(known_ahead);
            if (known >= 0 && stamp_ahead != my_stamp) {
                // a list for other points (another tensor, or this one changed in place): descend.  The forward pass
                // then replaces the list; a backward launch leaves the group's entries alone, because helper
                // workgroups of the same launch may be reading them.
                if (MODE == 1) cache_slot = -1;
                // the descent writes the new list over the old one before it is known whether all its parts find
                // room: the group counts as unknown from here on
                else if (lane == 0) cache.count[cache_slot] = -1;
            } else if (known >= 0) {
                const int all = known & kCandMask;
                const int n = (MODE == 1 && (known & kCandSplit)) ? own_share(all) : all;
                if (MODE == 1 || !(known & kCandRounds)) {
#pragma unroll
                    for (int k = 0; k < kAhead; ++k)
                        if (lane + k * kWave < n) leaves[wave][lane + k * kWave] = list_ahead[k];
                    for (int i = lane + kAhead * kWave; i < n; i += kWave) leaves[wave][i] = cache.list[size_t(cache_slot) * kLeafCap + i];
                    if (lane == 0) state[wave][0] = n;
                    sp = 0;
                }
                cache_slot = -1;
            }
        }
        // only a wavefront that descends needs the boxes around its points (a known list or a piece does without)
        if (sp > 0) group_boxes<T, D>(x, valid, lane, M >= kTwoBoxLeaves, gbox[wave]);
    }
    for (int i = threadIdx.x; i < kGroupsMax * kVals * kWave; i += kTravBlock) (&result[0][0][0])[i] = 0.0;

    const T* cboxes = child_box + size_t(bl) * (M - 1) * 4 * D;
    const int2* kids = children + size_t(bl) * (M - 1);
    const T* recs = leaf_rec + size_t(bl) * M * LS;

    // Phase 2 walks this wavefront's batches of the round, group after group, with a wave-uniform cursor; the
    // leaf records of the NEXT batch (possibly of the next group) are fetched into registers before the current
    // batch is tested and evaluated, so their memory round trip overlaps that work and the group's barriers.
    constexpr int kPre = (kStageBatch * LS + kWave - 1) / kWave;
    constexpr int kDenseHits = sizeof(T) == 8 ? 16 : 6;    // lanes per leaf from which the reduction is cheaper
    int cur_group = -1, cur_base = 0, cur_end = 0;
    T pre[kPre];
    auto next_batch = [&]() {
        cur_base += kStageBatch;
        while (cur_base >= cur_end && cur_group < groups) {
            ++cur_group;
            if (cur_group >= groups) break;
            const int n = __builtin_amdgcn_readfirstlane(state[cur_group][0]);
            const int per = (n + kTravWaves - 1) / kTravWaves;
            cur_base = wave * per;
            cur_end = cur_base + per < n ? cur_base + per : n;
        }
    };
    auto prefetch = [&]() {
        if (cur_group >= groups) return;
        const int cnt = cur_end - cur_base < kStageBatch ? cur_end - cur_base : kStageBatch;
#pragma unroll
        for (int r = 0; r < kPre; ++r) {
            const int s = lane + r * kWave;
            if (s < cnt * LS) {
                const int c = s / LS, k = s - c * LS;
                pre[r] = recs[size_t(leaves[cur_group][cur_base + c]) * LS + k];
            }
        }
    };
    // all batches of group gi that belong to this wavefront; the cursor stands on the first of them (or beyond)
    auto evaluate_share = [&](int gi) {
        T x[D];
#pragma unroll
        for (int d = 0; d < D; ++d) x[d] = pts[gi][d][lane];
        const T g = pts[gi][D][lane];
        const bool valid = pids[gi][lane] >= 0;
        T acc = T(0);
        T gx[D];
#pragma unroll
        for (int d = 0; d < D; ++d) gx[d] = T(0);
        // lanes start at different leaves of a batch, so that LDS atomics of one instruction spread over the leaves
        const int rot = NEED_GM ? lane % kStageBatch : 0;
        while (cur_group == gi) {
            const int cnt = cur_end - cur_base < kStageBatch ? cur_end - cur_base : kStageBatch;
#pragma unroll
            for (int r = 0; r < kPre; ++r) {
                const int s = lane + r * kWave;
                if (s < cnt * LS) staged[s] = pre[r];
            }
            if (NEED_GM)
                for (int s = lane; s < cnt * NR; s += kWave) rsum[s] = 0.0;
            wave_lds_fence();
            next_batch();
            prefetch();
            unsigned mask = 0u;
#pragma unroll 1
            for (int i0 = 0; i0 < cnt; i0 += 2) {
                T box[2][2 * D];
#pragma unroll
                for (int q = 0; q < 2; ++q)
#pragma unroll
                    for (int k = 0; k < 2 * D; ++k) box[q][k] = staged[(i0 + q) * LS + k];
#pragma unroll
                for (int q = 0; q < 2; ++q) mask |= (valid & inside_box<T, D>(x, box[q])) ? (1u << (i0 + q)) : 0u;
            }
            mask &= (1u << cnt) - 1u;                   // slots beyond the batch hold stale records
            if (NEED_GM) {
                // Leaves that contain many of the points: every lane evaluates the same leaf, the sums are
                // reduced over the wavefront and lane 63 alone adds them to the LDS copy.  (LDS atomics serialise
                // the lanes that add to the same address; a reduction costs the same however many lanes hit.)
                for (int i = 0; i < cnt; ++i) {
                    const bool has = (mask >> i) & 1u;
                    if (__popcll(__ballot(has)) < kDenseHits) continue;
                    mask &= ~(1u << i);
                    const T* lf = staged + i * LS + 2 * D;
                    T r[kAmp - 2 * D + 1];
#pragma unroll
                    for (int k = 0; k < kAmp - 2 * D + 1; ++k) r[k] = lf[k];
                    T t[D], u[D];
                    const T e = leaf_terms<T, D>(r, exp2_tab, x, t, u);
                    if (NEED_GX) {
                        const T s = has ? r[kAmp - 2 * D] * e : T(0);
#pragma unroll
                        for (int d = 0; d < D; ++d) gx[d] = fma_(s, u[d], gx[d]);
                    }
                    T rs[NR];
                    rs[0] = has ? e * g : T(0);
#pragma unroll
                    for (int d = 0; d < D; ++d) rs[1 + d] = rs[0] * t[d];
                    int k = 1 + D;
#pragma unroll
                    for (int a = 0; a < D; ++a)
#pragma unroll
                        for (int c = a; c < D; ++c) rs[k++] = rs[1 + a] * t[c];
                    // four sums at a time; the lane at the end of row r receives sum {0, 2, 1, 3}[r] of the four
                    const int row = lane >> 4, mine = ((row & 1) << 1) | (row >> 1);
#pragma unroll
                    for (int q0 = 0; q0 < NR; q0 += 4) {
                        const T total = wave_sum4_to_row_ends(rs[q0], q0 + 1 < NR ? rs[q0 + 1] : T(0),
                                                              q0 + 2 < NR ? rs[q0 + 2] : T(0),
                                                              q0 + 3 < NR ? rs[q0 + 3] : T(0), lane);
                        if ((lane & 15) == 15 && q0 + mine < NR) rsum[i * NR + q0 + mine] += double(total);
                    }
                }
                mask = ((mask >> rot) | (mask << (kStageBatch - rot))) & ((1u << kStageBatch) - 1u);
            }
            while (__ballot(mask != 0u) != 0ull) {
                const bool has = mask != 0u;
                int i = has ? __builtin_ctz(mask) + rot : 0;
                i = i >= kStageBatch ? i - kStageBatch : i;
                mask &= mask - 1u;
                const T* lf = staged + i * LS + 2 * D;
                T r[kAmp - 2 * D + 1];
#pragma unroll
                for (int k = 0; k < kAmp - 2 * D + 1; ++k) r[k] = lf[k];
                T t[D], u[D];
                const T e = leaf_terms<T, D>(r, exp2_tab, x, t, u);
                const T amp = r[kAmp - 2 * D];
                if (MODE == 0) {
                    acc += has ? amp * e : T(0);
                } else {
                    if (NEED_GX) {
                        const T s = has ? amp * e : T(0);
#pragma unroll
                        for (int d = 0; d < D; ++d) gx[d] = fma_(s, u[d], gx[d]);
                    }
                    if (NEED_GM && has) {
                        double* rs = rsum + i * NR;
                        const T eg = e * g;
                        atomic_add(&rs[0], double(eg));
                        T rt[D];
#pragma unroll
                        for (int d = 0; d < D; ++d) { rt[d] = eg * t[d]; atomic_add(&rs[1 + d], double(rt[d])); }
                        int k = 1 + D;
#pragma unroll
                        for (int a = 0; a < D; ++a)
#pragma unroll
                            for (int c = a; c < D; ++c) atomic_add(&rs[k++], double(rt[a] * t[c]));
                    }
                }
            }
            if (NEED_GM) {
                wave_lds_fence();
                for (int s = lane; s < cnt * NR; s += kWave) {
                    const int c = s / NR, k = s - c * NR;
                    const T v = T(rsum[s]);
                    if (v != T(0)) {
                        const int comp = reinterpret_cast<const int*>(staged + c * LS + kAmp + 1)[0];
                        atomic_add(&sums[(size_t(bl) * M + comp) * NR + k], v);
                    }
                }
            }
            wave_lds_fence();
        }
        if (MODE == 0) {
            partial[gi][wave][lane] = acc;
        } else if (NEED_GX) {
#pragma unroll
            for (int d = 0; d < D; ++d) atomic_add(&result[gi][d][lane], double(gx[d]));
        }
    };

    __syncthreads();
    if (piece >= 0 && !piece_valid) {
        // the epilogue adds the dL/dx of every published piece: a piece that is not worked on contributes zeros
        if (NEED_GX && threadIdx.x < D * kWave) piece_gx[size_t(piece) * D * kWave + threadIdx.x] = T(0);
        return;
    }
    // every descent step retires at least one of the M-1 internal nodes, each of which is pushed at most once
    for (int round = 0; round < M; ++round) {
        if (sp > 0) {
            int n_leaf = 0;
            int* stk = stack[wave];
            int* cand = leaves[wave];
            T glo[2][D], ghi[2][D];
#pragma unroll
            for (int k = 0; k < 2; ++k)
#pragma unroll
                for (int d = 0; d < D; ++d) { glo[k][d] = T(gbox[wave][k * 2 * D + d]); ghi[k][d] = T(gbox[wave][k * 2 * D + D + d]); }
            // room in the pool for the list of a later round is asked for before the descent, so that the atomic's
            // round trip is over when the list is there (a whole list's worth; what is not used stays unused)
            int pool_at = 0;
            if (cache_slot >= 0 && cache_ok && round > 0 && lane == 0) pool_at = atomicAdd(&cache.ctl[1], kLeafCap);
            for (int iter = 0; sp > 0 && n_leaf < kLeafFlush && iter < M; ++iter) {
                wave_lds_fence();
                // wide pops only while the stack has room for 128 more entries; a narrow pop is a depth-first
                // step, which adds at most one entry per tree level
                const int k = sp <= kStackCap - 128 ? (sp < 64 ? sp : 64) : 1;
                const bool active = lane < k;
                const int node = active ? stk[sp - 1 - lane] : 0;
                sp -= k;
                const int2 ch = kids[node];
                T cb[4 * D];
#pragma unroll
                for (int i = 0; i < 4 * D; ++i) cb[i] = cboxes[size_t(node) * 4 * D + i];
                bool push[2], hit[2];
#pragma unroll
                for (int side = 0; side < 2; ++side) {
                    const int c = side == 0 ? ch.x : ch.y;
                    bool meets[2] = {true, M >= kTwoBoxLeaves};         // the child's box overlaps the group's first / second box
#pragma unroll
                    for (int d = 0; d < D; ++d)
                        meets[0] = meets[0] & (cb[side * 2 * D + d] <= ghi[0][d]) & (cb[side * 2 * D + D + d] >= glo[0][d]);
                    if (M >= kTwoBoxLeaves) {                           // (small trees have one box: the same for all wavefronts)
#pragma unroll
                        for (int d = 0; d < D; ++d)
                            meets[1] = meets[1] & (cb[side * 2 * D + d] <= ghi[1][d]) & (cb[side * 2 * D + D + d] >= glo[1][d]);
                    }
                    const bool ov = active & (c < M - 1) & (~c < M) & (meets[0] | meets[1]);    // ... and is a node of this tree
                    push[side] = ov & (c >= 0);
                    hit[side] = ov & (c < 0);
                }
                wave_lds_fence();
#pragma unroll
                for (int side = 0; side < 2; ++side) {
                    const int c = side == 0 ? ch.x : ch.y;
                    const unsigned long long mp = __ballot(push[side]), mh = __ballot(hit[side]);
                    const int at = sp + __popcll(mp & below);
                    if (push[side]) {
                        if (at < kStackCap + 128) stk[at] = c;                 // always in range, see the pop rule
                        else atomicOr(&cache.ctl[2], kErrStack);               // a dropped push is reported, never silent
                    }
                    sp += __popcll(mp);
                    sp = sp < kStackCap + 128 ? sp : kStackCap + 128;
                    if (hit[side]) cand[n_leaf + __popcll(mh & below)] = ~c;
                    n_leaf += __popcll(mh);
                }
            }
            if (lane == 0) { state[wave][0] = n_leaf; state[wave][1] = sp; }
            // Keep the group's list for later traversals: the first round's in the group's fixed slot, those of
            // later rounds in the pool; what exceeds the owner's share becomes pieces for helper workgroups,
            // published when the descent has ended and every part has found room.  Only the forward pass publishes
            // pieces (a backward launch has helpers running that read the piece table).
            if (cache_slot >= 0) {
                if (cache_ok && n_leaf > 0) {
                    int base = cache_slot * kLeafCap, own = 0, share = n_leaf;
                    if (n_leaf > kPieceLeaves) share = own_share(n_leaf);
                    if (round == 0) {
                        first_round_leaves = n_leaf;
                        own = share;
                    } else {
                        const int at = __builtin_amdgcn_readfirstlane(pool_at);
                        cache_ok = at + kLeafCap <= cache.pool_cap;
                        base = cache.pool_base + at;
                    }
                    const int wanted = (n_leaf - own + share - 1) / share;
                    if (wanted > 0 && (MODE != 0 || n_pend + wanted > kPendMax)) cache_ok = false;
                    if (cache_ok) {
                        wave_lds_fence();
                        for (int i = lane; i < n_leaf; i += kWave) cache.list[size_t(base) + i] = cand[i];
                        if (lane < wanted) {
                            const int from = own + lane * share;
                            pend[wave][n_pend + lane] = make_int2(base + from, n_leaf - from < share ? n_leaf - from : share);
                        }
                        n_pend += wanted;
                    }
                }
                if (sp == 0) {
                    // the descent has ended: ask for the slots of the pieces now, fill them after this round's
                    // evaluation (the atomic's round trip then overlaps the first record fetches)
                    publish = cache_ok;
                    if (cache_ok && n_pend > 0 && lane == 0) piece_slot = atomicAdd(&cache.ctl[0], n_pend);
                    publish_flags = first_round_leaves | (n_pend > 0 ? kCandSplit : 0) | (round > 0 ? kCandRounds : 0);
                    publish_slot = cache_slot;
                    cache_slot = -1;
                }
            }
        }
        __syncthreads();
        bool left_on_stack = false;
        cur_group = -1; cur_base = 0; cur_end = 0;
        next_batch();
        prefetch();
        for (int gi = 0; gi < groups; ++gi) {
            const int n_leaf = state[gi][0];
            left_on_stack |= state[gi][1] > 0;
            if (n_leaf == 0) continue;                                  // uniform over the workgroup
            evaluate_share(gi);
        }
        if (MODE == 0) {
            // forward: the wavefronts' partial sums are added in a fixed order, by wavefront g for group g (the
            // backward pass has added its dL/dx with atomics)
            __syncthreads();
            if (wave < groups && state[wave][0] > 0) {
                T v = T(0);
#pragma unroll
                for (int w = 0; w < kTravWaves; ++w) v += partial[wave][w][lane];
                result[wave][0][lane] += double(v);
            }
        }
        if (publish) {
            publish = false;
            bool fits = true;
            const int slot = n_pend > 0 ? __builtin_amdgcn_readfirstlane(piece_slot) : 0;
            if (n_pend > 0) {
                fits = slot + n_pend <= cache.pieces_max;
                wave_lds_fence();
                // slots in range are always filled: a helper must never read an unwritten piece
                if (lane < n_pend && slot + lane < cache.pieces_max)
                    cache.pieces[slot + lane] = fits ? make_int4(publish_slot, pend[wave][lane].x, pend[wave][lane].y, 0)
                                                     : make_int4(0, 0, 0, 0);
            }
            if (fits && lane == 0) {
                cache.stamp[publish_slot] = my_stamp;
                cache.piece_range[publish_slot] = make_int2(slot, n_pend);
                cache.count[publish_slot] = publish_flags;
            }
        }
        if (!left_on_stack) break;
        __syncthreads();                                                // every wavefront has read this round's state
        // a group without nodes left gathers nothing in later rounds
        if (wave < groups && sp == 0 && lane == 0) state[wave][0] = 0;
    }

    __syncthreads();
    if (wave >= groups) return;
    const int pid = pids[wave][lane];
    if (pid < 0) return;
    if (MODE == 0) {
        out[size_t(bl) * N + pid] = T(result[wave][0][lane]);
    } else if (NEED_GX) {
        const T g = pts[wave][D][lane];
        if (piece >= 0) {
#pragma unroll
            for (int d = 0; d < D; ++d) piece_gx[(size_t(piece) * D + d) * kWave + lane] = -g * T(result[0][d][lane]);
            return;
        }
        T* dst = grad_xes + (xseg * N + pid) * D;
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const T v = -g * T(result[wave][d][lane]);
            if (xes_shared) atomic_add(&dst[d], v); else dst[d] = v;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// small trees: all leaves against all points, the box test in front of every evaluation (no descent)
// ---------------------------------------------------------------------------------------------------------------
// A tree of a few dozen leaves has nothing to cull per 64-point group that a box test per leaf does not find faster:
// the descent, the candidate lists and the lane-by-lane evaluation cost more than they save.  Measured, 64 mixtures of
// 4096 points, forward / backward us without the tree against the traversal: 32 leaves 16 / 28 against 21 / 40 (6 % of
// the pairs inside a box; the same ratio at 0.1 %), 64 leaves 25 / 44 against 23 / 49, and with a quarter of the pairs
// inside (336 mixtures) 78 / 159 against 130 / 262; from 128 leaves on the traversal wins unless most boxes contain
// most points (22 / 42 against 39 / 56 at 0.6 % inside).  Mixtures of at most kAllPairsMax components are therefore
// evaluated without the tree: the leaf records of the mixture (own box + evaluation record,
// as the build left them) are staged in LDS, a wavefront owns P groups of 64 Morton-neighbouring points (lanes =
// points), walks over ALL leaves and applies the per-point rule of lbvh/aabb.h:39-47 itself; a leaf is evaluated for a
// group only when its box contains at least one of the group's points (one ballot: neighbouring points mostly agree).
// Same per-pair arithmetic as the traversal (centred form), same sums: the result is the sum over the Gaussians
// whose own box contains the point.  Backward: dL/dx in registers; the sums of a leaf are accumulated over the
// wavefront's P groups in registers, reduced over the wavefront once per leaf and added to the workgroup's LDS copy
// (double), which leaves with one global atomic per non-zero scalar; the wavefronts start at different leaves.
constexpr int kAllPairsMax = 64;
static int g_eval_path = 0;             // test knob (gmc_bvh_set_eval_path): 1 = always the traversal

template <typename T, int D, int P, int MODE, bool NEED_GM, bool NEED_GX>
__global__ __launch_bounds__(kBlock) void bvh_all_pairs_kernel(const T* __restrict__ xes, const int* __restrict__ p_order,
                                                              const T* __restrict__ leaf_rec, T* __restrict__ out,
                                                              const T* __restrict__ grad_out, T* __restrict__ sums,
                                                              T* __restrict__ grad_xes, int L, int M, int N, int Bx, int Lx,
                                                              int chunks, int xes_shared) {
    constexpr int LS = LeafRec<D>::kStride;
    constexpr int NR = BvhSums<D>::k;
    constexpr int kAmp = 2 * D + D + D * (D + 1) / 2;       // position of the amplitude inside a leaf record
    constexpr int kRec = kAmp - 2 * D + 1;                  // centre, symmetric matrix, amplitude
    __shared__ __attribute__((aligned(16))) T recs[kAllPairsMax * LS];
    __shared__ double lsum[MODE == 1 && NEED_GM ? kAllPairsMax * NR : 1];
    const T* exp2_tab = exp2_table<T>();                    // (published by the barrier below)
    const int bl = blockIdx.x / chunks, chunk = blockIdx.x - bl * chunks;
    const int b = bl / L, l = bl - b * L;
    const size_t xseg = size_t(b < Bx ? b : Bx - 1) * Lx + (l < Lx ? l : Lx - 1);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    {
        const T* src = leaf_rec + size_t(bl) * M * LS;
        for (int i = threadIdx.x; i < M * LS; i += kBlock) recs[i] = src[i];
        if (MODE == 1 && NEED_GM)
            for (int i = threadIdx.x; i < M * NR; i += kBlock) lsum[i] = 0.0;
    }
    T x[P][D], go[P], acc[P], gx[P][D];
    int pid[P];
    bool any_point = false;
#pragma unroll
    for (int p = 0; p < P; ++p) {
        const int j = ((chunk * (kBlock / kWave) + wave) * P + p) * kWave + lane;
        pid[p] = -1;
        if (j < N) {
            const int id = p_order[xseg * N + j];
            pid[p] = unsigned(id) < unsigned(N) ? id : 0;   // a permutation by construction; never index out of bounds
        }
        const size_t at = xseg * N + (pid[p] >= 0 ? pid[p] : 0);
#pragma unroll
        for (int d = 0; d < D; ++d) { x[p][d] = xes[at * D + d]; gx[p][d] = T(0); }
        go[p] = (MODE == 1 && pid[p] >= 0) ? grad_out[size_t(bl) * N + pid[p]] : T(0);
        acc[p] = T(0);
        any_point |= pid[p] >= 0;
    }
    __syncthreads();
    if (__ballot(any_point) != 0ull) {
        // the wavefronts of a workgroup start at different leaves: their additions to the LDS sums do not meet
        const int rot = wave * (M / (kBlock / kWave));
        for (int ii = 0; ii < M; ++ii) {
            int i = ii + rot;
            i -= i >= M ? M : 0;
            const T* r = recs + i * LS;
            T box[2 * D];
#pragma unroll
            for (int k = 0; k < 2 * D; ++k) box[k] = r[k];
            T rs[NR];
#pragma unroll
            for (int k = 0; k < NR; ++k) rs[k] = T(0);
            bool touched = false;
#pragma unroll
            for (int p = 0; p < P; ++p) {
                const bool in = (pid[p] >= 0) & inside_box<T, D>(x[p], box);
                if (__ballot(in) == 0ull) continue;
                touched = true;
                T rec[kRec];
#pragma unroll
                for (int k = 0; k < kRec; ++k) rec[k] = r[2 * D + k];
                T t[D], u[D];
                const T e = leaf_terms<T, D>(rec, exp2_tab, x[p], t, u);
                const T s = in ? rec[kRec - 1] * e : T(0);
                if (MODE == 0) {
                    acc[p] += s;
                } else {
                    if (NEED_GX) {
#pragma unroll
                        for (int d = 0; d < D; ++d) gx[p][d] = fma_(s, u[d], gx[p][d]);
                    }
                    if (NEED_GM) {
                        const T k0 = in ? e * go[p] : T(0);
                        rs[0] += k0;
                        T rt[D];
#pragma unroll
                        for (int d = 0; d < D; ++d) { rt[d] = k0 * t[d]; rs[1 + d] += rt[d]; }
                        int k = 1 + D;
#pragma unroll
                        for (int a = 0; a < D; ++a)
#pragma unroll
                            for (int c = a; c < D; ++c) { rs[k] = fma_(rt[a], t[c], rs[k]); ++k; }
                    }
                }
            }
            if (MODE == 1 && NEED_GM && touched) {
                // four sums at a time; the lane at the end of row r receives sum {0, 2, 1, 3}[r] of the four
                const int row = lane >> 4, mine = ((row & 1) << 1) | (row >> 1);
#pragma unroll
                for (int q0 = 0; q0 < NR; q0 += 4) {
                    const T total = wave_sum4_to_row_ends(rs[q0], q0 + 1 < NR ? rs[q0 + 1] : T(0), q0 + 2 < NR ? rs[q0 + 2] : T(0),
                                                          q0 + 3 < NR ? rs[q0 + 3] : T(0), lane);
                    if ((lane & 15) == 15 && q0 + mine < NR && total != T(0)) atomic_add(&lsum[i * NR + q0 + mine], double(total));
                }
            }
        }
    }
#pragma unroll
    for (int p = 0; p < P; ++p) {
        if (pid[p] < 0) continue;
        if (MODE == 0) {
            out[size_t(bl) * N + pid[p]] = acc[p];
        } else if (NEED_GX) {
            T* dst = grad_xes + (xseg * N + pid[p]) * D;
#pragma unroll
            for (int d = 0; d < D; ++d) {
                const T v = -go[p] * gx[p][d];
                if (xes_shared) atomic_add(&dst[d], v); else dst[d] = v;
            }
        }
    }
    if (MODE == 1 && NEED_GM) {
        __syncthreads();
        for (int s = threadIdx.x; s < M * NR; s += kBlock) {
            const T v = T(lsum[s]);
            if (v != T(0)) {
                const int i = s / NR, k = s - i * NR;
                int comp = reinterpret_cast<const int*>(recs + i * LS + kAmp + 1)[0];
                comp = unsigned(comp) < unsigned(M) ? comp : 0;
                atomic_add(&sums[(size_t(bl) * M + comp) * NR + k], v);
            }
        }
    }
}

// points per lane of the all-pairs kernels: as many as still leave a thousand workgroups
static int all_pairs_points(size_t BL, int N, int p_max) {
    const size_t groups = (size_t(N) + kWave - 1) / kWave;
    for (int P = p_max; P > 1; P >>= 1)
        if (BL * ((groups + 4 * P - 1) / (4 * P)) >= 1024) return P;
    return 1;
}

// (R0, sum r t, sum r t t^T) -> (dw, db, dC); see the dense epilogue for the formulas (here y = t, u = identity).
// covariance_form: the record holds S with C = (S^-1)^T; the matrix gradient is carried on to S as
// MatrixInverse.backward does (src/gmc/cpp/extensions/math/matrix_inverse.py:30-33: -S^-1 g S^-1 without transposes,
// which is the derivative for symmetric matrices only): dS = -(C dC C)^T.
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void bvh_bwd_epilogue_kernel(const T* __restrict__ mixture, T* __restrict__ sums,
                                                                 T* __restrict__ grad_mixture, size_t n,
                                                                 bool covariance_form, CandidateCache cache,
                                                                 const T* __restrict__ piece_gx,
                                                                 const int* __restrict__ p_order, T* __restrict__ grad_xes,
                                                                 const T* __restrict__ xes, unsigned gaussian_blocks, int L,
                                                                 int N, int Bx, int Lx) {
    constexpr int G = 1 + D + D * D;
    constexpr int NR = BvhSums<D>::k;
    // Workgroups behind the first `gaussian_blocks`: dL/dx of the pieces that helper workgroups of the traversal
    // worked on, one wavefront per piece, added to what the owners of the point groups have stored (several
    // pieces of a group meet here, hence atomics).
    if (blockIdx.x >= gaussian_blocks) {
        if (!cache.count) return;                           // the traversal had no helpers then
        const int published = cache.ctl[0] < cache.pieces_max ? cache.ctl[0] : cache.pieces_max;
        const int per_mixture = (N + kWave - 1) / kWave;
        const int lane = threadIdx.x & 63;
        const int p = int(blockIdx.x - gaussian_blocks) * (kBlock / kWave) + int(threadIdx.x >> 6);
        if (p >= published) return;
        const int4 desc = cache.pieces[p];
        if (desc.z <= 0) return;
        const int bl = desc.x / per_mixture, group = desc.x - bl * per_mixture;
        const int b = bl / L, l = bl - b * L;
        const size_t xseg = size_t(b < Bx ? b : Bx - 1) * Lx + (l < Lx ? l : Lx - 1);
        const int j = group * kWave + lane;
        if (j >= N) return;
        int pid = p_order[xseg * N + j];
        pid = unsigned(pid) < unsigned(N) ? pid : 0;
        for (int d = 0; d < D; ++d)
            atomic_add(&grad_xes[(xseg * N + pid) * D + d], piece_gx[(size_t(p) * D + d) * kWave + lane]);
        return;
    }
    const size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= n) return;
    const T* g = mixture + i * G;
    T rs[NR];
    for (int k = 0; k < NR; ++k) { rs[k] = sums[i * NR + k]; sums[i * NR + k] = T(0); }     // ready for the next backward pass
    T* o = grad_mixture + i * G;
    const double w = double(g[0]);
    double c[D][D];
    load_inverse_covariance<T, D>(g + 1 + D, covariance_form, c);
    const double det = determinant<T, D>(c);
    const double root = sqrt(det);
    const double norm = Kappa<D>::v * root;
    const double R0 = double(rs[0]);
    o[0] = T(norm * R0);
    double r1[D];
    for (int d = 0; d < D; ++d) r1[d] = double(rs[1 + d]);
    for (int r = 0; r < D; ++r) {
        double acc = 0.0;
        for (int q = 0; q < D; ++q) acc += 0.5 * (c[r][q] + c[q][r]) * r1[q];
        o[1 + r] = T(w * norm * acc);
    }
    double s2[D][D];
    int k = 1 + D;
    for (int a = 0; a < D; ++a)
        for (int q = a; q < D; ++q) { s2[a][q] = double(rs[k]); s2[q][a] = double(rs[k]); ++k; }
    const double kd = w * Kappa<D>::v * R0 / (2.0 * root);
    double gc[D][D];
    for (int r = 0; r < D; ++r)
        for (int q = 0; q < D; ++q) {
            double cof;
            if constexpr (D == 2) {
                cof = (r == q) ? c[1 - r][1 - q] : -c[q][r];
            } else {
                const int r1i = r == 0 ? 1 : 0, r2i = r == 2 ? 1 : 2, q1 = q == 0 ? 1 : 0, q2 = q == 2 ? 1 : 2;
                cof = (((r + q) & 1) ? -1.0 : 1.0) * (c[r1i][q1] * c[r2i][q2] - c[r1i][q2] * c[r2i][q1]);
            }
            gc[r][q] = -0.5 * w * norm * s2[r][q] + cof * kd;
        }
    if (!covariance_form) {
        for (int r = 0; r < D; ++r)
            for (int q = 0; q < D; ++q) o[1 + D + r * D + q] = T(gc[r][q]);
        return;
    }
    double x1[D][D];
    for (int r = 0; r < D; ++r)
        for (int q = 0; q < D; ++q) {
            double acc = 0.0;
            for (int t = 0; t < D; ++t) acc += c[r][t] * gc[t][q];
            x1[r][q] = acc;
        }
    for (int r = 0; r < D; ++r)
        for (int q = 0; q < D; ++q) {
            double acc = 0.0;
            for (int t = 0; t < D; ++t) acc += x1[r][t] * c[t][q];
            o[1 + D + q * D + r] = T(-acc);
        }
}

template <typename T, int D>
__global__ __launch_bounds__(kBlock) void export_nodes_kernel(const int2* __restrict__ children, const int* __restrict__ parent,
                                                             const int* __restrict__ leaf_comp, int32_t* __restrict__ nodes,
                                                             int M, size_t total) {
    const size_t t = size_t(blockIdx.x) * kBlock + threadIdx.x;
    if (t >= total) return;
    const size_t n_nodes = 2 * size_t(M) - 1;
    const size_t bl = t / n_nodes;
    const int node = int(t - bl * n_nodes);
    int32_t* o = nodes + t * 4;
    o[0] = parent[t];
    if (node < M - 1) {
        const int2 ch = children[bl * (M - 1) + node];
        o[1] = ch.x >= 0 ? ch.x : (M - 1) + ~ch.x;
        o[2] = ch.y >= 0 ? ch.y : (M - 1) + ~ch.y;
        o[3] = -1;
    } else {
        o[1] = -1; o[2] = -1;
        o[3] = leaf_comp[bl * M + (node - (M - 1))];
    }
}

// the boxes of the Gaussians in component order, from the boxes of the leaves (Morton order)
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void export_boxes_kernel(const T* __restrict__ node_box, const int* __restrict__ leaf_comp,
                                                             T* __restrict__ lower, T* __restrict__ upper, int M, size_t total) {
    const size_t t = size_t(blockIdx.x) * kBlock + threadIdx.x;
    if (t >= total) return;
    const size_t bl = t / M;
    const int leaf = int(t - bl * M);
    int comp = leaf_comp[t];
    comp = (comp >= 0 && comp < M) ? comp : 0;
    const T* box = node_box + (bl * (2 * size_t(M) - 1) + (M - 1) + leaf) * 2 * D;
    for (int d = 0; d < D; ++d) {
        if (lower) lower[(bl * M + comp) * D + d] = box[d];
        if (upper) upper[(bl * M + comp) * D + d] = box[D + d];
    }
}

template <typename T>
__global__ void copy_kernel(const T* __restrict__ src, T* __restrict__ dst, size_t n) {
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

__global__ void iota_segments_kernel(int* __restrict__ dst, int count, size_t total) {
    const size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < total) dst[i] = int(i % count);
}

// ---------------------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------------------
static unsigned grid_for(size_t n) { return unsigned((n + kBlock - 1) / kBlock); }

// Pass `pass` (8 key bits from `first_bit + 8 * pass` on) of the stable LSD radix sort of `segments` segments of
// `count` (key, value) pairs: input (ka, va) on even passes and (kb, vb) on odd ones, output the other pair, the
// last pass writes to (keys_out, vals_out).  A job without workgroups stands for "nothing to do in this pass".
static SortJob sort_job(uint32_t* ka, uint32_t* va, uint32_t* kb, uint32_t* vb, uint32_t* keys_out, uint32_t* vals_out,
                        uint32_t* hist, size_t segments, int count, int first_bit, int passes, int pass, int* err) {
    SortJob j = {};
    j.err = err;
    if (segments == 0 || count == 0 || pass >= passes) return j;
    const bool odd = pass & 1;
    j.keys_in = odd ? kb : ka; j.vals_in = odd ? vb : va;
    j.keys_out = odd ? ka : kb; j.vals_out = odd ? va : vb;
    if (pass == passes - 1) { j.keys_out = keys_out; j.vals_out = vals_out; }
    j.count = count;
    j.items = sort_items(size_t(count));
    j.blocks_per_seg = int(sort_blocks(size_t(count)));
    const size_t pass_words = segments * size_t(j.blocks_per_seg) * 256;
    j.hist = hist + size_t(pass) * pass_words;
    j.hist_next = pass + 1 < passes ? hist + size_t(pass + 1) * pass_words : nullptr;
    j.chunk_shift = 8;
    for (int it = j.items; it > 1; it >>= 1) ++j.chunk_shift;
    j.shift = first_bit + 8 * pass;
    j.blocks = unsigned(segments * size_t(j.blocks_per_seg));
    return j;
}

// Build of the trees and of the Morton order of the query points.  The two chains (boxes -> keys -> sort of the
// leaves; bounds -> keys -> sort of the points) do not depend on each other, so each launch serves both.
template <typename T, int D>
static int bvh_build_t(const T* mixture, const T* xes, char* bvh, const gmc_shape& s, const gmc_bvh_config& cfg,
                       hipStream_t st) {
    constexpr int G = 1 + D + D * D;
    const BvhLayout lay = bvh_layout(s);
    const size_t BL = size_t(s.B) * s.L, XL = size_t(s.Bx) * s.Lx;
    const int M = s.M, N = s.N;
    T* node_box = (T*)(bvh + lay.node_box); T* leaf_rec = (T*)(bvh + lay.leaf_rec);
    int2* children = (int2*)(bvh + lay.children); int* parent = (int*)(bvh + lay.parent);
    int2* node_range = (int2*)(bvh + lay.node_range);
    int* leaf_comp = (int*)(bvh + lay.leaf_comp);
    using Enc = typename OrderedInt<T>::type;
    Enc* run_box = (Enc*)(bvh + lay.run_box);
    uint32_t* ka = (uint32_t*)(bvh + lay.keys_a); uint32_t* kb = (uint32_t*)(bvh + lay.keys_b);
    uint32_t* va = (uint32_t*)(bvh + lay.vals_a); uint32_t* vb = (uint32_t*)(bvh + lay.vals_b);
    uint32_t* pka = (uint32_t*)(bvh + lay.pkeys_a); uint32_t* pkb = (uint32_t*)(bvh + lay.pkeys_b);
    uint32_t* pva = (uint32_t*)(bvh + lay.pvals_a); uint32_t* pvb = (uint32_t*)(bvh + lay.pvals_b);
    T* parts_g = (T*)(bvh + lay.parts_g); T* parts_p = (T*)(bvh + lay.parts_p);
    T* child_box = (T*)(bvh + lay.child_box);
    uint32_t* g_keys = (uint32_t*)(bvh + lay.g_keys);
    uint32_t* g_order = (uint32_t*)leaf_comp;                // the sorted payload IS the component id of every leaf
    int* p_order = (int*)(bvh + lay.p_order);
    const bool have_g = BL > 0 && M > 0, have_p = XL > 0 && N > 0;
    const bool sort_p = have_p && xes != nullptr;
    if (g_build_path == 0 && have_g && M <= kSmallTreeMax && (!sort_p || N <= kCoarseOrderMax) && BL + XL < (size_t(1) << 31)) {
        const CandidateCache cache = candidate_cache(bvh, lay);
        SmallBuild<T> a{node_box, child_box, leaf_rec, (T*)(bvh + lay.sums), children, parent, node_range,
                        leaf_comp, g_keys, (int*)(bvh + lay.frontier), p_order, cache.count, (int*)(bvh + lay.cand_ctl),
                        double(cfg.aabb_threshold), cfg.aabb_mode, cfg.covariance_form != 0 ? 1 : 0, M, N,
                        (N + kWave - 1) / kWave, sort_p ? 1 : 0, 0u};
        // trees of at most 64 leaves: one wavefront each, four per workgroup; of at most 128: two wavefronts each, two per
        // workgroup (no idle vector units while the leaves are written: the double arithmetic of a leaf's box and record is
        // the longest part of the chain); larger ones: one workgroup each, with one, two or four leaves per lane
        const int lanes = M <= kWave ? kWave : M <= 2 * kWave ? 2 * kWave : kBlock;      // lanes per tree
        a.tree_blocks = unsigned((BL + kBlock / lanes - 1) / (kBlock / lanes));
        const dim3 grid(a.tree_blocks + unsigned(have_p ? XL : 0));
        const int pp = !sort_p || N <= 4 * kBlock ? 4 : N <= 16 * kBlock ? 16 : 32;
#define GMC_SMALL(THREADS, K, PP) bvh_build_small_kernel<T, D, THREADS, K, PP><<<grid, dim3(kBlock), 0, st>>>(mixture, xes, a, BL)
#define GMC_SMALL_PP(THREADS, K) do { if (pp == 4) GMC_SMALL(THREADS, K, 4); else if (pp == 16) GMC_SMALL(THREADS, K, 16); else GMC_SMALL(THREADS, K, 32); } while (0)
        if (lanes == kWave) GMC_SMALL_PP(kWave, 1);
        else if (lanes == 2 * kWave) GMC_SMALL_PP(2 * kWave, 1);
        else if (M <= kBlock) GMC_SMALL_PP(kBlock, 1);
        else if (M <= 2 * kBlock) GMC_SMALL_PP(kBlock, 2);
        else GMC_SMALL_PP(kBlock, 4);
#undef GMC_SMALL_PP
#undef GMC_SMALL
        return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
    }
    const int bpm = (M + kBlock - 1) / kBlock;               // workgroups per mixture (boxes, keys)
    const int nbp = (N + kBoundsChunk - 1) / kBoundsChunk;   // partial bounds per point segment
    const unsigned box_blocks = have_g ? unsigned(BL * bpm) : 0u, bound_blocks = sort_p ? unsigned(XL * nbp) : 0u;
    if (box_blocks + bound_blocks > 0)
        bvh_bounds_kernel<T, D><<<dim3(box_blocks + bound_blocks), dim3(kBlock), 0, st>>>(
            mixture, M, bpm, parts_g, box_blocks, xes, N, nbp, parts_p, (int*)(bvh + lay.cand_ctl),
            (uint32_t*)(bvh + lay.hist_g), lay.hist_words);
    const int p_passes = N > kCoarseOrderMax ? 2 : 1;
    auto jobs_of_pass = [&](int pass, SortJob& jg, SortJob& jp) {
        jg = sort_job(ka, va, kb, vb, g_keys, g_order, (uint32_t*)(bvh + lay.hist_g), have_g ? BL : 0, M, 0, 4, pass, (int*)(bvh + lay.cand_ctl) + 2);
        jp = sort_job(pka, pva, pkb, pvb, p_passes == 1 ? pkb : pka, (uint32_t*)p_order,
                      (uint32_t*)(bvh + lay.hist_p), sort_p ? XL : 0, N, 30 - 8 * p_passes, p_passes, pass,
                      (int*)(bvh + lay.cand_ctl) + 2);
    };
    SortJob jg0, jp0;
    jobs_of_pass(0, jg0, jp0);
    MortonJob<T> mg = {}, mp = {};
    // one or two large trees: every value of the top 8 key bits gathered and sorted in LDS (bucket_sort_kernel)
    const bool bucket_sort = have_g && g_build_path != 2 && M > kSmallTreeMax && M <= kBucketSortMax &&
                             (BL == 1 || (BL == 2 && M <= kBucketSortMax / 2));
    // (a Morton workgroup per block of the first radix pass; without a radix sort behind it: 256 keys each)
    if (have_g) mg = MortonJob<T>{mixture, G, 1, M, bucket_sort ? 1 : jg0.items, bucket_sort ? bpm : jg0.blocks_per_seg, parts_g, bpm, ka, va,
                                  unsigned(BL * (bucket_sort ? bpm : jg0.blocks_per_seg)), bucket_sort ? nullptr : (uint32_t*)jg0.hist, jg0.shift};
    if (sort_p) mp = MortonJob<T>{xes, D, 0, N, jp0.items, jp0.blocks_per_seg, parts_p, nbp, pka, pva, unsigned(XL * jp0.blocks_per_seg),
                                  (uint32_t*)jp0.hist, jp0.shift};
    if (mg.blocks + mp.blocks > 0) morton_kernel<T, D><<<dim3(mg.blocks + mp.blocks), dim3(kBlock), 0, st>>>(mg, mp);
    // leaves: all 30 key bits; points: the top 16 Morton bits (65536 cells) are enough to make 64 consecutive
    // points neighbours, the top 8 bits for segments of at most kCoarseOrderMax points (32 points per cell; measured:
    // same traversal times, one sort pass less).  The sorted keys of the points are not needed afterwards: they
    // land in a spare buffer, which must not be the input of the last pass.
    // The launches of the leaves' four passes are bound by their latency and would take twice as long with the six
    // times more numerous points in them; the points' passes ride in the two longest launches of the tree
    // construction instead (leaf records + radix tree, boxes), which use a quarter of the compute units.
    const SortJob none = {};
    SortJob jp_first = none, jp_second = none;
    for (int pass = 0; pass < 4; ++pass) {
        SortJob jg, jp;
        jobs_of_pass(pass, jg, jp);
        if (pass == 0) jp_first = jp;
        if (pass == 1) jp_second = jp;
        if (jg.blocks == 0 || bucket_sort) continue;
        radix_scatter_kernel<<<dim3(jg.blocks), dim3(kBlock), 0, st>>>(jg, none);
    }
    if (bucket_sort) {
        const dim3 grid{unsigned(BL * 256)}, block{unsigned(kBucketSortLanes)};
        int* err = (int*)(bvh + lay.cand_ctl) + 2;
        if (M <= 2048) bucket_sort_kernel<2048><<<grid, block, 0, st>>>(ka, g_keys, g_order, M, err);
        else if (M <= 4096) bucket_sort_kernel<4096><<<grid, block, 0, st>>>(ka, g_keys, g_order, M, err);
        else if (M <= 8192) bucket_sort_kernel<8192><<<grid, block, 0, st>>>(ka, g_keys, g_order, M, err);
        else bucket_sort_kernel<16384><<<grid, block, 0, st>>>(ka, g_keys, g_order, M, err);
    }
    if (!have_g) {                                   // no trees to build: the points' passes are launches of their own
        if (jp_first.blocks > 0) radix_scatter_kernel<<<dim3(jp_first.blocks), dim3(kBlock), 0, st>>>(jp_first, none);
        if (jp_second.blocks > 0) radix_scatter_kernel<<<dim3(jp_second.blocks), dim3(kBlock), 0, st>>>(jp_second, none);
    }
    if (have_g) {
        const size_t n = BL * M;
        const unsigned leaf_blocks = unsigned((n + kBoxBlock - 1) / kBoxBlock);
        bvh_leaves_kernel<T, D><<<dim3(leaf_blocks + jp_first.blocks), dim3(kBlock), 0, st>>>(
            mixture, double(cfg.aabb_threshold), cfg.aabb_mode, g_order, g_keys, node_box, leaf_rec, run_box,
            children, parent, node_range, M, n, cfg.covariance_form != 0, (T*)(bvh + lay.sums), leaf_blocks, jp_first);
        if (M > 1) {
            const size_t nn = BL * (2 * size_t(M) - 1);
            const unsigned frontier_blocks = unsigned((BL + kBlock / kWave - 1) / (kBlock / kWave));
            bvh_child_boxes_kernel<T, D><<<dim3(grid_for(nn) + jp_second.blocks + frontier_blocks), dim3(kBlock), 0, st>>>(
                children, parent, node_range, run_box, node_box, child_box, M, nn, candidate_cache(bvh, lay), lay.point_groups,
                grid_for(nn), jp_second, (int*)(bvh + lay.frontier), BL);
        } else if (jp_second.blocks > 0) {           // single leaves have no boxes to merge
            radix_scatter_kernel<<<dim3(jp_second.blocks), dim3(kBlock), 0, st>>>(jp_second, none);
        }
    }
    if (have_p && !sort_p) iota_segments_kernel<<<dim3(grid_for(XL * N)), dim3(kBlock), 0, st>>>(p_order, N, XL * N);
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

// 64-point groups per traversal workgroup.  A forward pass on a new tree descends: more groups per workgroup overlap
// more descents (each a chain of memory round trips that leaves the vector units idle), and the launch should fit
// the resident workgroups in one go (measured on one mixture of 16384 Gaussians, groups -> best choice and time:
// 391 -> 1, 43 us; 782 -> 2, 39 us; 1563 -> 4, 46 us against 63 us with 2; 3125 ... 25000 -> 4).  A backward pass
// reads the candidate lists: small workgroups balance better over the compute units until the launch has many times
// more groups than resident workgroups (1563 -> 1, 77 us against 85 us with 4; 3125 -> 2; 6250 -> 3; 25000 -> 4).  (Four
// groups spread over exactly one round of resident workgroups are 3-6 % ahead at 1563 groups when the same backward
// pass is repeated on one tree, and not ahead in a step that builds, traverses forward and backward: not taken.)  The
// lists of many small trees are short and the fixed work of a workgroup weighs more: their backward launches take the
// forward rule (64 trees of 512 leaves, 4096 groups: 72 us with 4 against 79 with 3 and 98 with 1; 256 trees of 200
// leaves, 3328 groups: 44 us with 4, 46 with 2, 52 with 1).
static int g_traversal_groups[2] = {0, 0};      // test knob (gmc_bvh_set_traversal_groups): forward, backward; 0 = automatic
static int traversal_groups(size_t BL, int M, int N, bool backward) {
    const size_t per_mixture = (size_t(N) + kWave - 1) / kWave;
    const size_t total = BL * per_mixture, slots = size_t(kTravSlots);
    size_t g;
    if (g_traversal_groups[backward ? 1 : 0] > 0) g = size_t(g_traversal_groups[backward ? 1 : 0]);
    else if (backward && M > kSmallTreeMax) g = total < 4 * slots ? 1 : total < 8 * slots ? 2 : total < 16 * slots ? 3 : kGroupsMax;
    else g = total <= slots ? 1 : total <= 2 * slots ? 2 : kGroupsMax;
    if (g > per_mixture) g = per_mixture;
    return g < 1 ? 1 : int(g);
}

template <typename T, int D>
static int bvh_fwd_t(const T* xes, char* bvh, T* out, const gmc_shape& s, hipStream_t st) {
    const BvhLayout lay = bvh_layout(s);
    const size_t BL = size_t(s.B) * s.L;
    if (BL == 0 || s.N == 0) return GMC_OK;
    if (s.M == 0) {
        const size_t n = BL * s.N;
        fill_zero_kernel<T><<<dim3(grid_for(n) < 4096 ? grid_for(n) : 4096), dim3(kBlock), 0, st>>>(out, n);
        return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
    }
    if (g_eval_path != 1 && s.M <= kAllPairsMax) {
        const int P = all_pairs_points(BL, s.N, 4);
        const int chunks = int((size_t(s.N) + size_t(kBlock) * P - 1) / (size_t(kBlock) * P));
#define GMC_ALL(PP) bvh_all_pairs_kernel<T, D, PP, 0, false, false><<<dim3(unsigned(BL * chunks)), dim3(kBlock), 0, st>>>( \
        xes, (const int*)(bvh + lay.p_order), (const T*)(bvh + lay.leaf_rec), out, nullptr, nullptr, nullptr, s.L, s.M, s.N, \
        s.Bx, s.Lx, chunks, 0)
        if (P == 4) GMC_ALL(4); else if (P == 2) GMC_ALL(2); else GMC_ALL(1);
#undef GMC_ALL
        return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
    }
    const int groups = traversal_groups(BL, s.M, s.N, false);
    int chunks = (s.N + kWave * groups - 1) / (kWave * groups);
    // A launch that would leave resident slots empty is spread over all of them: workgroups whose last wavefront
    // finds no group left serve one group fewer (1563 groups: 512 workgroups of 3 or 4 instead of 391 of 4, 50.6 -> 46.5 us).
    if (groups > 1 && BL * size_t(chunks) < size_t(kTravSlots)) {
        const size_t per_mixture = (size_t(s.N) + kWave - 1) / kWave, fill = size_t(kTravSlots) / BL;
        chunks = int(fill < per_mixture ? fill : per_mixture);
    }
    bvh_traverse_kernel<T, D, 0, false, false><<<dim3(unsigned(BL * chunks)), dim3(kTravBlock), 0, st>>>(
        xes, (const int*)(bvh + lay.p_order), (const T*)(bvh + lay.child_box), (const int2*)(bvh + lay.children),
        (const T*)(bvh + lay.leaf_rec), out, nullptr, nullptr, nullptr, candidate_cache(bvh, lay), nullptr, 0,
        s.L, s.M, s.N, s.Bx, s.Lx, chunks, groups, 0, (const int*)(bvh + lay.frontier));
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

template <typename T, int D>
static int bvh_bwd_t(const T* grad_out, const T* mixture, const T* xes, char* bvh, T* grad_mixture, T* grad_xes,
                     T* sums, const gmc_shape& s, bool gm, bool gx, bool covariance_form, hipStream_t st) {
    constexpr int G = 1 + D + D * D;
    const BvhLayout lay = bvh_layout(s);
    const size_t BL = size_t(s.B) * s.L;
    const size_t n_g = BL * s.M, n_x = size_t(s.Bx) * s.Lx * s.N * D;
    const int xes_shared = (s.Bx != s.B || s.Lx != s.L) ? 1 : 0;
    auto zero = [&](T* p, size_t n) {
        if (n) fill_zero_kernel<T><<<dim3(grid_for(n) < 4096 ? grid_for(n) : 4096), dim3(kBlock), 0, st>>>(p, n);
    };
    if (BL == 0) return GMC_OK;
    if (s.N == 0 || s.M == 0) {
        if (gm) zero(grad_mixture, n_g * G);
        if (gx) zero(grad_xes, n_x);
        return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
    }
    sums = (T*)(bvh + lay.sums);                   // inside the object and all zero here; the caller's workspace is not used
    if (gx && xes_shared) zero(grad_xes, n_x);
    if (g_eval_path != 1 && s.M <= kAllPairsMax) {
        const int P = all_pairs_points(BL, s.N, sizeof(T) == 8 ? 2 : 4);
        const int chunks = int((size_t(s.N) + size_t(kBlock) * P - 1) / (size_t(kBlock) * P));
#define GMC_ALL(PP, GM, GX) bvh_all_pairs_kernel<T, D, PP, 1, GM, GX><<<dim3(unsigned(BL * chunks)), dim3(kBlock), 0, st>>>( \
        xes, (const int*)(bvh + lay.p_order), (const T*)(bvh + lay.leaf_rec), nullptr, grad_out, sums, grad_xes, s.L, s.M, s.N, \
        s.Bx, s.Lx, chunks, xes_shared)
#define GMC_ALL_P(GM, GX) do { if (P == 4) { if constexpr (sizeof(T) == 4) GMC_ALL(4, GM, GX); } else if (P == 2) GMC_ALL(2, GM, GX); else GMC_ALL(1, GM, GX); } while (0)
        if (gm && gx) GMC_ALL_P(true, true);
        else if (gm) GMC_ALL_P(true, false);
        else if (gx) GMC_ALL_P(false, true);
#undef GMC_ALL_P
#undef GMC_ALL
        if (gm) {
            bvh_bwd_epilogue_kernel<T, D><<<dim3(grid_for(n_g)), dim3(kBlock), 0, st>>>(
                mixture, sums, grad_mixture, n_g, covariance_form, candidate_cache(bvh, lay), nullptr, (const int*)(bvh + lay.p_order),
                grad_xes, xes, grid_for(n_g), s.L, s.N, s.Bx, s.Lx);
        }
        return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
    }
    const int groups = traversal_groups(BL, s.M, s.N, true);
    int chunks = (s.N + kWave * groups - 1) / (kWave * groups);
    if (groups > 1 && BL * size_t(chunks) < size_t(kTravSlots)) {       // (as in the forward pass: no resident slot left empty)
        const size_t per_mixture = (size_t(s.N) + kWave - 1) / kWave, fill = size_t(kTravSlots) / BL;
        chunks = int(fill < per_mixture ? fill : per_mixture);
    }
    // one helper workgroup per piece that a forward pass may have published, behind the owners
    const int helpers = lay.pieces_max;
    const dim3 grid(unsigned(BL * chunks + helpers));
    const CandidateCache cache = candidate_cache(bvh, lay);
    T* piece_gx = (T*)(bvh + lay.piece_gx);
#define GMC_TRAV(GM, GX) bvh_traverse_kernel<T, D, 1, GM, GX><<<grid, dim3(kTravBlock), 0, st>>>( \
        xes, (const int*)(bvh + lay.p_order), (const T*)(bvh + lay.child_box), (const int2*)(bvh + lay.children), \
        (const T*)(bvh + lay.leaf_rec), nullptr, grad_out, sums, grad_xes, cache, piece_gx, helpers, \
        s.L, s.M, s.N, s.Bx, s.Lx, chunks, groups, xes_shared, (const int*)(bvh + lay.frontier))
    if (gm && gx) GMC_TRAV(true, true);
    else if (gm) GMC_TRAV(true, false);
    else if (gx) GMC_TRAV(false, true);
#undef GMC_TRAV
    const bool pieces_gx = gx && helpers > 0;
    if (gm || pieces_gx) {
        const unsigned gaussian_blocks = gm ? grid_for(n_g) : 0u;
        const unsigned piece_blocks = pieces_gx ? unsigned((helpers + kBlock / kWave - 1) / (kBlock / kWave)) : 0u;
        bvh_bwd_epilogue_kernel<T, D><<<dim3(gaussian_blocks + piece_blocks), dim3(kBlock), 0, st>>>(
            mixture, sums, grad_mixture, n_g, covariance_form, cache, piece_gx, (const int*)(bvh + lay.p_order), grad_xes,
            xes, gaussian_blocks, s.L, s.N, s.Bx, s.Lx);
    }
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

template <typename T, int D>
static int bvh_export_t(const char* bvh, T* lower, T* upper, int32_t* nodes, T* node_boxes, const gmc_shape& s,
                        hipStream_t st) {
    const BvhLayout lay = bvh_layout(s);
    const size_t BL = size_t(s.B) * s.L;
    const size_t n = BL * s.M * D;
    auto copy = [&](const T* src, T* dst, size_t cnt) {
        if (cnt) copy_kernel<T><<<dim3(grid_for(cnt) < 4096 ? grid_for(cnt) : 4096), dim3(kBlock), 0, st>>>(src, dst, cnt);
    };
    if ((lower || upper) && n)
        export_boxes_kernel<T, D><<<dim3(grid_for(BL * s.M)), dim3(kBlock), 0, st>>>(
            (const T*)(bvh + lay.node_box), (const int*)(bvh + lay.leaf_comp), lower, upper, s.M, BL * s.M);
    if (s.M > 0) {
        const size_t nn = BL * (2 * size_t(s.M) - 1);
        if (nodes && nn)
            export_nodes_kernel<T, D><<<dim3(grid_for(nn)), dim3(kBlock), 0, st>>>(
                (const int2*)(bvh + lay.children), (const int*)(bvh + lay.parent), (const int*)(bvh + lay.leaf_comp), nodes,
                s.M, nn);
        if (node_boxes) copy((const T*)(bvh + lay.node_box), node_boxes, nn * 2 * D);
    }
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

}  // namespace gmc

extern "C" {

void gmc_bvh_set_traversal_groups(int forward, int backward) {
    gmc::g_traversal_groups[0] = forward >= 1 && forward <= gmc::kGroupsMax ? forward : 0;
    gmc::g_traversal_groups[1] = backward >= 1 && backward <= gmc::kGroupsMax ? backward : 0;
}
void gmc_bvh_set_build_path(int path) { gmc::g_build_path = path == 1 || path == 2 ? path : 0; }
void gmc_bvh_set_eval_path(int path) { gmc::g_eval_path = path == 1 ? 1 : 0; }

size_t gmc_bvh_bytes(const gmc_shape* shape) {
    if (gmc::check_shape(shape) != GMC_OK) return 0;
    return gmc::bvh_layout(*shape).total;
}

static int check_bvh_shape(const gmc_shape* shape) {
    const int rc = gmc::check_shape(shape);
    if (rc != GMC_OK) return rc;
    // leaf indices are stored bit-inverted in an int, traversal loop counters are ints
    if (shape->M > (1 << 30) || shape->N > (1 << 30)) return GMC_E_SHAPE;
    return GMC_OK;
}

int gmc_bvh_build(const void* mixture, const void* xes, void* bvh, size_t bvh_bytes, const gmc_shape* shape,
                  const gmc_bvh_config* config, void* stream) {
    const int rc = check_bvh_shape(shape);
    if (rc != GMC_OK) return rc;
    if (!config) return GMC_E_NULL;
    if (config->aabb_mode != GMC_AABB_REFERENCE && config->aabb_mode != GMC_AABB_TIGHT) return GMC_E_CONFIG;
    if (!(config->aabb_threshold > 0.0f)) return GMC_E_CONFIG;
    const size_t need = gmc::bvh_layout(*shape).total;
    if (need == 0) return GMC_OK;
    if (!bvh) return GMC_E_NULL;
    if (bvh_bytes < need) return GMC_E_WORKSPACE;
    if (!mixture && size_t(shape->B) * shape->L * shape->M > 0) return GMC_E_NULL;
#define ARGS(T) (const T*)mixture, (const T*)xes, (char*)bvh, *shape, *config, (hipStream_t)stream
    if (shape->dtype == GMC_F32) return shape->D == 2 ? gmc::bvh_build_t<float, 2>(ARGS(float)) : gmc::bvh_build_t<float, 3>(ARGS(float));
    return shape->D == 2 ? gmc::bvh_build_t<double, 2>(ARGS(double)) : gmc::bvh_build_t<double, 3>(ARGS(double));
#undef ARGS
}

int gmc_bvh_export_boxes(const void* bvh, void* lower, void* upper, const gmc_shape* shape, void* stream) {
    const int rc = check_bvh_shape(shape);
    if (rc != GMC_OK) return rc;
    if (size_t(shape->B) * shape->L * shape->M == 0) return GMC_OK;
    if (!bvh || !lower || !upper) return GMC_E_NULL;
#define ARGS(T) (const char*)bvh, (T*)lower, (T*)upper, (int32_t*)nullptr, (T*)nullptr, *shape, (hipStream_t)stream
    if (shape->dtype == GMC_F32) return shape->D == 2 ? gmc::bvh_export_t<float, 2>(ARGS(float)) : gmc::bvh_export_t<float, 3>(ARGS(float));
    return shape->D == 2 ? gmc::bvh_export_t<double, 2>(ARGS(double)) : gmc::bvh_export_t<double, 3>(ARGS(double));
#undef ARGS
}

int gmc_bvh_export_nodes(const void* bvh, int32_t* nodes, void* node_boxes, const gmc_shape* shape, void* stream) {
    const int rc = check_bvh_shape(shape);
    if (rc != GMC_OK) return rc;
    if (size_t(shape->B) * shape->L * shape->M == 0) return GMC_OK;
    if (!bvh || !nodes || !node_boxes) return GMC_E_NULL;
#define ARGS(T) (const char*)bvh, (T*)nullptr, (T*)nullptr, nodes, (T*)node_boxes, *shape, (hipStream_t)stream
    if (shape->dtype == GMC_F32) return shape->D == 2 ? gmc::bvh_export_t<float, 2>(ARGS(float)) : gmc::bvh_export_t<float, 3>(ARGS(float));
    return shape->D == 2 ? gmc::bvh_export_t<double, 2>(ARGS(double)) : gmc::bvh_export_t<double, 3>(ARGS(double));
#undef ARGS
}

int gmc_bvh_export_candidate_stats(const void* bvh, int32_t* stats, const gmc_shape* shape, void* stream) {
    const int rc = check_bvh_shape(shape);
    if (rc != GMC_OK) return rc;
    if (!stats) return GMC_E_NULL;
    const gmc::BvhLayout lay = gmc::bvh_layout(*shape);
    if (!bvh) return GMC_E_NULL;
    gmc::copy_kernel<int32_t><<<dim3(1), dim3(gmc::kBlock), 0, (hipStream_t)stream>>>(
        (const int32_t*)((const char*)bvh + lay.cand_ctl), stats, 4);
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

int gmc_bvh_export_leaf_order(const void* bvh, uint32_t* keys, int32_t* components, const gmc_shape* shape, void* stream) {
    const int rc = check_bvh_shape(shape);
    if (rc != GMC_OK) return rc;
    const size_t n = size_t(shape->B) * shape->L * shape->M;
    if (n == 0) return GMC_OK;
    if (!bvh || !keys || !components) return GMC_E_NULL;
    const gmc::BvhLayout lay = gmc::bvh_layout(*shape);
    const unsigned blocks = unsigned((n + gmc::kBlock - 1) / gmc::kBlock < 4096 ? (n + gmc::kBlock - 1) / gmc::kBlock : 4096);
    gmc::copy_kernel<uint32_t><<<dim3(blocks), dim3(gmc::kBlock), 0, (hipStream_t)stream>>>(
        (const uint32_t*)((const char*)bvh + lay.g_keys), keys, n);
    gmc::copy_kernel<int32_t><<<dim3(blocks), dim3(gmc::kBlock), 0, (hipStream_t)stream>>>(
        (const int32_t*)((const char*)bvh + lay.leaf_comp), components, n);
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

int gmc_eval_bvh_fwd(const void* mixture, const void* xes, void* bvh, void* out, const gmc_shape* shape,
                     void* stream) {
    (void)mixture;   // the leaf records inside the BVH hold everything the forward pass needs
    const int rc = check_bvh_shape(shape);
    if (rc != GMC_OK) return rc;
    if (size_t(shape->B) * shape->L * shape->N == 0) return GMC_OK;
    if (!out || !xes || (!bvh && shape->M > 0)) return GMC_E_NULL;
#define ARGS(T) (const T*)xes, (char*)bvh, (T*)out, *shape, (hipStream_t)stream
    if (shape->dtype == GMC_F32) return shape->D == 2 ? gmc::bvh_fwd_t<float, 2>(ARGS(float)) : gmc::bvh_fwd_t<float, 3>(ARGS(float));
    return shape->D == 2 ? gmc::bvh_fwd_t<double, 2>(ARGS(double)) : gmc::bvh_fwd_t<double, 3>(ARGS(double));
#undef ARGS
}

static int eval_bvh_bwd_impl(const void* grad_out, const void* mixture, const void* xes, void* bvh,
                             void* grad_mixture, void* grad_xes, void* workspace, size_t workspace_bytes,
                             const gmc_shape* shape, int need_grad_mixture, int need_grad_xes, bool covariance_form,
                             void* stream) {
    const int rc = check_bvh_shape(shape);
    if (rc != GMC_OK) return rc;
    const bool gm = need_grad_mixture != 0, gx = need_grad_xes != 0;
    if (!gm && !gx) return GMC_OK;
    const size_t n_g = size_t(shape->B) * shape->L * shape->M;
    const size_t n_x = size_t(shape->Bx) * shape->Lx * shape->N;
    if (gm && n_g > 0 && !grad_mixture) return GMC_E_NULL;
    if (gx && n_x > 0 && !grad_xes) return GMC_E_NULL;
    if (n_g > 0 && n_x > 0 && (!grad_out || !mixture || !xes || !bvh)) return GMC_E_NULL;
    (void)workspace_bytes;    // the per-Gaussian sums live inside the BVH object; a workspace is accepted and not used
#define ARGS(T) (const T*)grad_out, (const T*)mixture, (const T*)xes, (char*)bvh, (T*)grad_mixture, (T*)grad_xes, (T*)workspace, *shape, gm, gx, covariance_form, (hipStream_t)stream
    if (shape->dtype == GMC_F32) return shape->D == 2 ? gmc::bvh_bwd_t<float, 2>(ARGS(float)) : gmc::bvh_bwd_t<float, 3>(ARGS(float));
    return shape->D == 2 ? gmc::bvh_bwd_t<double, 2>(ARGS(double)) : gmc::bvh_bwd_t<double, 3>(ARGS(double));
#undef ARGS
}

int gmc_eval_bvh_bwd(const void* grad_out, const void* mixture, const void* xes, void* bvh, void* grad_mixture,
                     void* grad_xes, void* workspace, size_t workspace_bytes, const gmc_shape* shape,
                     int need_grad_mixture, int need_grad_xes, void* stream) {
    return eval_bvh_bwd_impl(grad_out, mixture, xes, bvh, grad_mixture, grad_xes, workspace, workspace_bytes, shape,
                             need_grad_mixture, need_grad_xes, false, stream);
}

int gmc_eval_bvh_cov_bwd(const void* grad_out, const void* mixture, const void* xes, void* bvh, void* grad_mixture,
                         void* grad_xes, void* workspace, size_t workspace_bytes, const gmc_shape* shape,
                         int need_grad_mixture, int need_grad_xes, void* stream) {
    return eval_bvh_bwd_impl(grad_out, mixture, xes, bvh, grad_mixture, grad_xes, workspace, workspace_bytes, shape,
                             need_grad_mixture, need_grad_xes, true, stream);
}

}  // extern "C"
