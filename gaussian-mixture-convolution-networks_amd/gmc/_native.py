"""Loader and thin ctypes front end of libgmc_hip.so (the C ABI declared in include/gmc_hip.h).

PyTorch is used for device memory and streams only: tensors are allocated with torch, raw device pointers and the
current HIP stream are handed to the library.  There is no CPU or pure-torch fallback: if the library is
missing, or a tensor does not live on a HIP device, the call raises.
"""
import ctypes
import os
import subprocess

import torch

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC_DIR = os.path.join(_PKG_DIR, "csrc")
LIB_PATH = os.path.join(CSRC_DIR, "libgmc_hip.so")

GMC_F32, GMC_F64 = 0, 1
GMC_AABB_REFERENCE, GMC_AABB_TIGHT = 0, 1
ABI_VERSION = 11
STATIC_SCRATCH_BYTES = 64 << 20


class Shape(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in ("B", "L", "M", "N", "D", "Bx", "Lx", "dtype")]


class ConvShape(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in ("B", "Cin", "Cout", "Nd", "Nk", "D", "dtype")]


class BvhConfigC(ctypes.Structure):
    _fields_ = [("aabb_mode", ctypes.c_int), ("aabb_threshold", ctypes.c_float), ("covariance_form", ctypes.c_int)]


def build(verbose: bool = False) -> str:
    """Compiles every HIP source of the library for gfx950 (hipcc cross-compiles without a GPU)."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.run(["make", "-B", "-j8", "-C", CSRC_DIR, "libgmc_hip.so"], check=True, stdout=out, stderr=out)
    global _lib
    _lib = None
    return LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()' "
                           f"or make -C {CSRC_DIR}); there is no fallback implementation")
    l = ctypes.CDLL(LIB_PATH)
    vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    shp = ctypes.POINTER(Shape)
    cfg = ctypes.POINTER(BvhConfigC)
    l.gmc_error_string.restype = ctypes.c_char_p
    l.gmc_error_string.argtypes = [ci]
    l.gmc_abi_version.restype = ci
    l.gmc_eval_fwd.argtypes = [vp, vp, vp, shp, vp]
    l.gmc_set_tuning.restype = None
    l.gmc_set_tuning.argtypes = [ci, ci]
    l.gmc_export_launch_clocks.argtypes = [ctypes.POINTER(ctypes.c_double)]
    l.gmc_eval_fwd_kernel_name.restype = ctypes.c_char_p
    l.gmc_eval_fwd_kernel_name.argtypes = [shp]
    l.gmc_eval_bwd_workspace_bytes.restype = sz
    l.gmc_eval_bwd_workspace_bytes.argtypes = [shp]
    l.gmc_eval_bwd.argtypes = [vp, vp, vp, vp, vp, vp, sz, shp, ci, ci, vp]
    l.gmc_eval_bwd_static.argtypes = [vp, vp, vp, vp, vp, shp, ci, ci, ci, vp]
    l.gmc_eval_cov_fwd.argtypes = [vp, vp, vp, shp, vp]
    l.gmc_eval_cov_bwd.argtypes = [vp, vp, vp, vp, vp, vp, sz, shp, ci, ci, vp]
    l.gmc_eval_componentwise_fwd.argtypes = [vp, vp, vp, shp, ci, vp]
    l.gmc_eval_componentwise_bwd.argtypes = [vp, vp, vp, vp, vp, vp, sz, shp, ci, ci, ci, vp]
    l.gmc_relu_fit_goal.argtypes = [vp, vp, vp, vp, shp, vp]
    l.gmc_relu_fit_step.argtypes = [vp, vp, vp, vp, shp, vp]
    l.gmc_eval_cov_moments_bytes.restype = sz
    l.gmc_eval_cov_moments_bytes.argtypes = [shp]
    l.gmc_eval_cov_moments.argtypes = [vp, vp, vp, vp, sz, vp, vp, vp, vp, vp, ctypes.c_double, shp, ci, vp]
    l.gmc_batch_norm_sampling_positions.argtypes = [vp, vp, shp, vp]
    l.gmc_validate_mixture.argtypes = [vp, vp, shp, vp]
    cshp = ctypes.POINTER(ConvShape)
    l.gmc_convolution_fwd.argtypes = [vp, vp, vp, cshp, vp]
    l.gmc_convolution_bwd.argtypes = [vp, vp, vp, vp, vp, cshp, ci, ci, vp]
    if hasattr(l, "gmc_bvh_bytes"):
        l.gmc_bvh_set_build_path.restype = None
        l.gmc_bvh_set_build_path.argtypes = [ci]
        l.gmc_bvh_set_eval_path.restype = None
        l.gmc_bvh_set_eval_path.argtypes = [ci]
        l.gmc_bvh_set_traversal_groups.restype = None
        l.gmc_bvh_set_traversal_groups.argtypes = [ci, ci]
        l.gmc_bvh_bytes.restype = sz
        l.gmc_bvh_bytes.argtypes = [shp]
        l.gmc_bvh_build.argtypes = [vp, vp, vp, sz, shp, cfg, vp]
        l.gmc_bvh_export_boxes.argtypes = [vp, vp, vp, shp, vp]
        l.gmc_bvh_export_nodes.argtypes = [vp, vp, vp, shp, vp]
        l.gmc_bvh_export_candidate_stats.argtypes = [vp, vp, shp, vp]
        l.gmc_bvh_export_leaf_order.argtypes = [vp, vp, vp, shp, vp]
        l.gmc_eval_bvh_fwd.argtypes = [vp, vp, vp, vp, shp, vp]
        l.gmc_eval_bvh_bwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, sz, shp, ci, ci, vp]
        l.gmc_eval_bvh_cov_bwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, sz, shp, ci, ci, vp]
    if l.gmc_abi_version() != ABI_VERSION:
        raise RuntimeError("libgmc_hip.so was built from a different include/gmc_hip.h; rebuild it")
    _lib = l
    return l


def check(code: int) -> None:
    if code != 0:
        raise RuntimeError("gmc_hip: " + lib().gmc_error_string(code).decode())


def n_dimensions(mixture: torch.Tensor) -> int:
    last = mixture.shape[-1]
    if last == 7:
        return 2
    if last == 13:
        return 3
    raise RuntimeError("mixture must have 7 or 13 elements in the last dimension")


def check_input(mixture: torch.Tensor, xes: torch.Tensor) -> Shape:
    """Same rules and messages as gpe::check_input_and_get_ns (src/gmc/cpp/extensions/util/mixture.h:107-127)
    plus the dtype dispatch of parallel_implementation.cu:78 (floating types only)."""
    if mixture.dim() != 4:
        raise RuntimeError("mixture must have 4 dimensions")
    d = n_dimensions(mixture)
    if not mixture.is_contiguous():
        raise RuntimeError("mixture must be contiguous")
    if not xes.is_contiguous():
        raise RuntimeError("xes must be contiguous")
    if xes.dim() != 4:
        raise RuntimeError("xes must have 4 dimensions")
    if xes.dtype != mixture.dtype:
        raise RuntimeError("mixture and xes must have the same dtype")
    if xes.device != mixture.device:
        raise RuntimeError("mixture and xes must have the same device")
    if mixture.dtype not in (torch.float32, torch.float64):
        raise RuntimeError("unsupported datatype: evaluate_inversed is implemented for float32 and float64")
    B, L, M, _ = mixture.shape
    Bx, Lx, N, Dx = xes.shape
    if Bx not in (1, B):
        raise RuntimeError("xes must have a batch dimension equal to one or the mixture")
    if Lx not in (1, L):
        raise RuntimeError("xes must have a layer dimension equal to one or the mixture")
    if Dx != d:
        raise RuntimeError("xes must have the last dimension equal to the number of dimensions of the mixture")
    if not mixture.is_cuda:
        raise RuntimeError("gmc_hip evaluates on an AMD GPU only: mixture and xes must be HIP ('cuda') tensors; "
                           "this build has no CPU implementation")
    return Shape(B, L, M, N, d, Bx, Lx, GMC_F32 if mixture.dtype == torch.float32 else GMC_F64)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device) -> int:
    """handle of torch's current HIP stream on `device` (the raw getter skips the construction of a Stream object)"""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


class _on:
    """Makes `device` the current HIP device for the duration of a call, like torch.cuda.device, but without its
    bookkeeping when the device is current already (the usual case; these wrappers sit on launch-bound paths)."""
    __slots__ = ("idx", "prev")

    def __init__(self, device):
        self.idx = device.index
        self.prev = -1

    def __enter__(self):
        cur = torch.cuda.current_device()
        if self.idx is not None and cur != self.idx:
            self.prev = cur
            torch.cuda.set_device(self.idx)

    def __exit__(self, *exc):
        if self.prev >= 0:
            torch.cuda.set_device(self.prev)
        return False


def _p(t):
    """device address as a plain int (ctypes converts it to void*); None (a null pointer) for absent or empty tensors"""
    return t.data_ptr() if t is not None and t.numel() > 0 else None


def eval_fwd(mixture: torch.Tensor, xes: torch.Tensor, covariance_form: bool = False) -> torch.Tensor:
    """`covariance_form`: the mixture holds covariances and the inversion happens inside the kernel"""
    shape = check_input(mixture, xes)
    out = torch.empty((shape.B, shape.L, shape.N), dtype=mixture.dtype, device=mixture.device)
    fn = lib().gmc_eval_cov_fwd if covariance_form else lib().gmc_eval_fwd
    with _on(mixture.device):
        check(fn(_p(mixture), _p(xes), _p(out), ctypes.byref(shape), _stream(mixture.device)))
    return out


def eval_bwd(grad_output, mixture, xes, need_mixture: bool, need_xes: bool, covariance_form: bool = False):
    shape = check_input(mixture, xes)
    if grad_output.dim() != 3:
        raise RuntimeError("grad_output has wrong number of dimensions")
    if grad_output.shape[0] != shape.B:
        raise RuntimeError("grad_output has wrong batch dimension")
    if grad_output.shape[1] != shape.L:
        raise RuntimeError("grad_output has wrong layer dimension")
    if grad_output.shape[2] != shape.N:
        raise RuntimeError("grad_output has wrong xes dimension")
    if grad_output.dtype != mixture.dtype:
        raise RuntimeError("grad_output dtype does not match with mixture dtype")
    if not grad_output.is_contiguous():
        raise RuntimeError("grad_output must be contiguous")
    _check_grad_output_device(grad_output, mixture)
    dev = mixture.device
    # both gradients are always returned, all-zero when not required (parallel_implementation.cu:120-121,175)
    grad_mixture = torch.empty_like(mixture) if need_mixture else torch.zeros_like(mixture)
    grad_xes = torch.empty_like(xes) if need_xes else torch.zeros_like(xes)
    if not (need_mixture or need_xes):
        return grad_mixture, grad_xes
    with _on(dev):
        ws_bytes = lib().gmc_eval_bwd_workspace_bytes(ctypes.byref(shape)) if need_mixture else 0
        ws = torch.empty((max(ws_bytes, 8) // 8,), dtype=torch.float64, device=dev)
        fn = lib().gmc_eval_cov_bwd if covariance_form else lib().gmc_eval_bwd
        check(fn(_p(grad_output), _p(mixture), _p(xes), _p(grad_mixture), _p(grad_xes), _p(ws), ws_bytes,
                 ctypes.byref(shape), int(need_mixture), int(need_xes), _stream(dev)))
    return grad_mixture, grad_xes


def eval_componentwise_fwd(mixture: torch.Tensor, xes: torch.Tensor, covariance_form: bool = False) -> torch.Tensor:
    """values [B, L, N, M] of every (point, component) pair"""
    shape = check_input(mixture, xes)
    out = torch.empty((shape.B, shape.L, shape.N, shape.M), dtype=mixture.dtype, device=mixture.device)
    with _on(mixture.device):
        check(lib().gmc_eval_componentwise_fwd(_p(mixture), _p(xes), _p(out), ctypes.byref(shape), int(covariance_form),
                                               _stream(mixture.device)))
    return out


def eval_componentwise_bwd(grad_output, mixture, xes, need_mixture: bool, need_xes: bool, covariance_form: bool = False):
    shape = check_input(mixture, xes)
    if tuple(grad_output.shape) != (shape.B, shape.L, shape.N, shape.M):
        raise RuntimeError("grad_output has wrong shape")
    _check_grad_output_device(grad_output, mixture)
    if grad_output.dtype != mixture.dtype:
        raise RuntimeError("grad_output dtype does not match with mixture dtype")
    if not grad_output.is_contiguous():
        raise RuntimeError("grad_output must be contiguous")
    dev = mixture.device
    grad_mixture = torch.empty_like(mixture) if need_mixture else torch.zeros_like(mixture)
    grad_xes = torch.empty_like(xes) if need_xes else torch.zeros_like(xes)
    if not (need_mixture or need_xes):
        return grad_mixture, grad_xes
    with _on(dev):
        ws_bytes = lib().gmc_eval_bwd_workspace_bytes(ctypes.byref(shape)) if need_mixture else 0
        ws = torch.empty((max(ws_bytes, 8) // 8,), dtype=torch.float64, device=dev)
        check(lib().gmc_eval_componentwise_bwd(_p(grad_output), _p(mixture), _p(xes), _p(grad_mixture), _p(grad_xes),
                                               _p(ws), ws_bytes, ctypes.byref(shape), int(need_mixture), int(need_xes),
                                               int(covariance_form), _stream(dev)))
    return grad_mixture, grad_xes


def _mixture_shape(mixture: torch.Tensor, n_points: int) -> Shape:
    if mixture.dim() != 4:
        raise RuntimeError("mixture must have 4 dimensions")
    d = n_dimensions(mixture)
    if not mixture.is_contiguous():
        raise RuntimeError("mixture must be contiguous")
    if mixture.dtype not in (torch.float32, torch.float64):
        raise RuntimeError("unsupported datatype: float32 and float64 only")
    if not mixture.is_cuda:
        raise RuntimeError("gmc_hip evaluates on an AMD GPU only; this build has no CPU implementation")
    B, L, M, _ = mixture.shape
    return Shape(B, L, M, n_points, d, B, L, GMC_F32 if mixture.dtype == torch.float32 else GMC_F64)


def _like(t: torch.Tensor, ref: torch.Tensor, shape, what: str) -> torch.Tensor:
    if tuple(t.shape) != tuple(shape) or t.dtype != ref.dtype or t.device != ref.device:
        raise RuntimeError(f"{what} must have shape {tuple(shape)} and the dtype and device of the mixture")
    return t.contiguous()


def validate_mixture(mixture: torch.Tensor, what: str = "mixture") -> None:
    """The reference's check_mixture (src/gmc/cpp/extensions/util/mixture.h:85-93) as one small launch and one read of
    a flag (this synchronises with the device, which is why it is optional everywhere): raises RuntimeError for NaNs,
    infinities and matrices with a determinant <= 0."""
    shape = _mixture_shape(mixture, 0)
    flag = torch.empty((1,), dtype=torch.int32, device=mixture.device)
    with _on(mixture.device):
        check(lib().gmc_validate_mixture(_p(mixture), _p(flag), ctypes.byref(shape), _stream(mixture.device)))
    bits = int(flag.item())
    if bits & 1:
        raise RuntimeError(f"{what} contains NaNs or infinities")
    if bits & 2:
        raise RuntimeError(f"{what} contains non positive definite covariances")


def relu_fit_goal(target_mixture: torch.Tensor, constant: torch.Tensor, fitting_mixture: torch.Tensor) -> torch.Tensor:
    """relu(evaluate(target, centres of fitting) + constant) - relu(constant), [B, L, n_fitting] (no gradients)"""
    shape = _mixture_shape(target_mixture, fitting_mixture.shape[2])
    B, L = shape.B, shape.L
    if fitting_mixture.dim() != 4 or fitting_mixture.shape[:2] != target_mixture.shape[:2] or \
            fitting_mixture.shape[3] != target_mixture.shape[3]:
        raise RuntimeError("target and fitting mixture must agree in batch, layers and dimensions")
    fitting_mixture = _like(fitting_mixture, target_mixture, fitting_mixture.shape, "fitting mixture")
    constant = _like(constant.expand(B, L), target_mixture, (B, L), "constant")
    goal = torch.empty((B, L, shape.N), dtype=target_mixture.dtype, device=target_mixture.device)
    with _on(target_mixture.device):
        check(lib().gmc_relu_fit_goal(_p(target_mixture), _p(constant), _p(fitting_mixture), _p(goal), ctypes.byref(shape),
                                      _stream(target_mixture.device)))
    return goal


def relu_fit_step(fitting_mixture: torch.Tensor, x: torch.Tensor, goal: torch.Tensor) -> torch.Tensor:
    """one multiplicative update |x| (goal + 0.05) / (evaluate(fitting with weights |x|, own centres) + 0.05)"""
    shape = _mixture_shape(fitting_mixture, fitting_mixture.shape[2])
    dims = (shape.B, shape.L, shape.M)
    x = _like(x, fitting_mixture, dims, "x")
    goal = _like(goal, fitting_mixture, dims, "goal")
    out = torch.empty_like(x)
    with _on(fitting_mixture.device):
        check(lib().gmc_relu_fit_step(_p(fitting_mixture), _p(x), _p(goal), _p(out), ctypes.byref(shape),
                                      _stream(fitting_mixture.device)))
    return out


def eval_cov_moments(mixture: torch.Tensor, constant: torch.Tensor, xes: torch.Tensor, per_sample: bool,
                     running_sd: torch.Tensor = None, running_mean: torch.Tensor = None, alpha: float = 0.0,
                     want_inverse: bool = False):
    """torch.std_mean of (evaluate(mixture, xes) + constant) over batch and samples per channel ([L], per_sample False)
    or over the samples of every (b, l) ([B, L]), without the values going to memory -> (sd, mean), or
    (sd, mean, 1 / max(sd, 0.001)) with want_inverse.  running_sd / running_mean: updated in place to
    (1 - alpha) * running + alpha * statistic and returned in place of the statistics."""
    shape = check_input(mixture, xes)
    if shape.Bx != shape.B or shape.Lx != shape.L:
        raise RuntimeError("the sampling positions must have the batch and layer dimensions of the mixture")
    B, L = shape.B, shape.L
    constant = _like(constant.expand(B, L), mixture, (B, L), "constant")
    dims = (B, L) if per_sample else (L,)
    if running_sd is not None:
        running_sd = _like(running_sd, mixture, dims, "running_sd")
        running_mean = _like(running_mean, mixture, dims, "running_mean")
    sd = torch.empty(dims, dtype=mixture.dtype, device=mixture.device)
    mean = torch.empty_like(sd)
    inv = torch.empty_like(sd) if want_inverse else None
    scratch = int(lib().gmc_eval_cov_moments_bytes(ctypes.byref(shape)))
    moments = torch.empty(max(scratch // 8, 1), dtype=torch.float64, device=mixture.device)
    with _on(mixture.device):
        check(lib().gmc_eval_cov_moments(_p(mixture), _p(constant), _p(xes), _p(moments), scratch, _p(sd), _p(mean), _p(inv),
                                         _p(running_sd), _p(running_mean), float(alpha), ctypes.byref(shape),
                                         int(per_sample), _stream(mixture.device)))
    return (sd, mean, inv) if want_inverse else (sd, mean)


def batch_norm_sampling_positions(mixture: torch.Tensor, uniform: torch.Tensor) -> torch.Tensor:
    """turns uniform numbers [B, L, N, D] in place into positions inside the box of all centres of their batch entry"""
    shape = check_input(mixture, uniform)
    if shape.Bx != shape.B or shape.Lx != shape.L:
        raise RuntimeError("the uniform numbers must have the batch and layer dimensions of the mixture")
    with _on(mixture.device):
        check(lib().gmc_batch_norm_sampling_positions(_p(mixture), _p(uniform), ctypes.byref(shape), _stream(mixture.device)))
    return uniform


# ---------------------------------------------------------------------------------------------------------------
# LBVH-culled variant
# ---------------------------------------------------------------------------------------------------------------

_AABB_MODES = {"reference": GMC_AABB_REFERENCE, "tight": GMC_AABB_TIGHT}


def _bvh_config(aabb_threshold: float, aabb_mode: str, covariance_form: bool = False) -> BvhConfigC:
    if aabb_mode not in _AABB_MODES:
        raise RuntimeError(f"unknown aabb_mode {aabb_mode!r}; expected 'reference' or 'tight'")
    if not aabb_threshold > 0:
        raise RuntimeError("aabb_threshold must be positive")
    return BvhConfigC(_AABB_MODES[aabb_mode], float(aabb_threshold), int(bool(covariance_form)))


class Bvh:
    """One LBVH per (batch, layer) mixture plus the Morton order of the query points, as an opaque device blob.
    covariance_form: the mixture holds covariances (as gm.evaluate takes them) instead of inverse covariances."""

    def __init__(self, mixture: torch.Tensor, xes: torch.Tensor, aabb_threshold: float = 0.001,
                 aabb_mode: str = "reference", covariance_form: bool = False):
        self.shape = check_input(mixture, xes)
        self.covariance_form = bool(covariance_form)
        self._cfg = _bvh_config(aabb_threshold, aabb_mode, covariance_form)
        dev = mixture.device
        with _on(dev):
            self._nbytes = lib().gmc_bvh_bytes(ctypes.byref(self.shape))
            self.blob = torch.empty((max(self._nbytes, 8),), dtype=torch.uint8, device=dev)
        self.dtype, self.device = mixture.dtype, dev
        self.rebuild(mixture, xes)

    def rebuild(self, mixture: torch.Tensor, xes: torch.Tensor):
        """Builds the trees of another mixture (same shape, dtype and device) into this object; all kept candidate
        lists are forgotten."""
        shape = check_input(mixture, xes)
        _check_bvh_shape(shape, self)
        if mixture.device != self.device:
            raise RuntimeError("the BVH lives on another device than the mixture")
        with _on(self.device):
            check(lib().gmc_bvh_build(_p(mixture), _p(xes), _p(self.blob), self._nbytes, ctypes.byref(self.shape),
                                      ctypes.byref(self._cfg), _stream(self.device)))
        # The object holds the Gaussians as they were now (leaf records, boxes): the forward pass reads only those,
        # the backward epilogue reads the mixture it is given.  Remember which values the tree belongs to.
        self._mixture_key = (mixture.data_ptr(), mixture._version)

    def check_mixture(self, mixture: torch.Tensor):
        """A Bvh is bound to the mixture values it was built from: other storage, or the same storage after an
        in-place update, needs a new Bvh (the forward pass would evaluate the old values otherwise)."""
        if (mixture.data_ptr(), mixture._version) != self._mixture_key:
            raise RuntimeError("the BVH was built from other mixture values (another tensor, or this one was modified "
                               "in place since): build a new Bvh")

    def boxes(self):
        """(lower, upper), each [B, L, M, D], in component order"""
        s = self.shape
        lo = torch.empty((s.B, s.L, s.M, s.D), dtype=self.dtype, device=self.device)
        up = torch.empty_like(lo)
        with _on(self.device):
            check(lib().gmc_bvh_export_boxes(_p(self.blob), _p(lo), _p(up), ctypes.byref(s), _stream(self.device)))
        return lo, up

    def nodes(self):
        """(nodes [B, L, 2M-1, 4] int32 = parent, left, right, component-or--1; node boxes [B, L, 2M-1, 2D])"""
        s = self.shape
        n = max(2 * s.M - 1, 0)
        nodes = torch.empty((s.B, s.L, n, 4), dtype=torch.int32, device=self.device)
        nb = torch.empty((s.B, s.L, n, 2 * s.D), dtype=self.dtype, device=self.device)
        with _on(self.device):
            check(lib().gmc_bvh_export_nodes(_p(self.blob), _p(nodes), _p(nb), ctypes.byref(s), _stream(self.device)))
        return nodes, nb

    def leaf_order(self):
        """(keys [B, L, M] int64 holding the 30-bit Morton codes of the leaves in sorted order, components [B, L, M]
        int32 = component id of every leaf)"""
        s = self.shape
        keys = torch.empty((s.B, s.L, s.M), dtype=torch.int32, device=self.device)
        comps = torch.empty((s.B, s.L, s.M), dtype=torch.int32, device=self.device)
        with _on(self.device):
            check(lib().gmc_bvh_export_leaf_order(_p(self.blob), _p(keys), _p(comps), ctypes.byref(s), _stream(self.device)))
        return keys.to(torch.int64) & 0xFFFFFFFF, comps

    def candidate_stats(self):
        """int32 [4]: pieces of long candidate lists published for the backward pass, pool ints in use, error flags
        (0 unless the library has a bug: 1 = a traversal dropped a node, 2 = a sort pass went out of range), 0"""
        stats = torch.empty((4,), dtype=torch.int32, device=self.device)
        with _on(self.device):
            check(lib().gmc_bvh_export_candidate_stats(_p(self.blob), _p(stats), ctypes.byref(self.shape),
                                                       _stream(self.device)))
        return stats


def _check_bvh_shape(shape: Shape, bvh: "Bvh"):
    """the layout of the opaque BVH object follows from the shape it was built for"""
    for name, _ in Shape._fields_:
        if getattr(shape, name) != getattr(bvh.shape, name):
            raise RuntimeError(f"the BVH was built for another shape or dtype ({name}: {getattr(bvh.shape, name)} at the "
                               f"build, {getattr(shape, name)} now)")


def _check_bvh_use(mixture, bvh: "Bvh", shape: Shape):
    _check_bvh_shape(shape, bvh)
    if bvh.device != mixture.device:
        raise RuntimeError("the BVH lives on another device than the mixture")
    bvh.check_mixture(mixture)


def _check_grad_output_device(grad_output, mixture):
    if grad_output.device != mixture.device:
        raise RuntimeError("grad_output must live on the device of the mixture")


def eval_bvh_fwd(mixture, xes, bvh: Bvh) -> torch.Tensor:
    """The forward pass evaluates the Gaussians stored in `bvh` at its build; `mixture` must be the tensor (and the
    values) the Bvh was built from."""
    shape = check_input(mixture, xes)
    _check_bvh_use(mixture, bvh, shape)
    out = torch.empty((shape.B, shape.L, shape.N), dtype=mixture.dtype, device=mixture.device)
    with _on(mixture.device):
        check(lib().gmc_eval_bvh_fwd(_p(mixture), _p(xes), _p(bvh.blob), _p(out), ctypes.byref(shape),
                                     _stream(mixture.device)))
    return out


def eval_bvh_bwd(grad_output, mixture, xes, bvh: Bvh, need_mixture: bool, need_xes: bool):
    shape = check_input(mixture, xes)
    _check_bvh_use(mixture, bvh, shape)
    _check_grad_output_device(grad_output, mixture)
    if tuple(grad_output.shape) != (shape.B, shape.L, shape.N):
        raise RuntimeError("grad_output has wrong shape")
    if grad_output.dtype != mixture.dtype:
        raise RuntimeError("grad_output dtype does not match with mixture dtype")
    if not grad_output.is_contiguous():
        raise RuntimeError("grad_output must be contiguous")
    dev = mixture.device
    grad_mixture = torch.empty_like(mixture) if need_mixture else torch.zeros_like(mixture)
    grad_xes = torch.empty_like(xes) if need_xes else torch.zeros_like(xes)
    if not (need_mixture or need_xes):
        return grad_mixture, grad_xes
    with _on(dev):
        fn = lib().gmc_eval_bvh_cov_bwd if bvh.covariance_form else lib().gmc_eval_bvh_bwd
        check(fn(_p(grad_output), _p(mixture), _p(xes), _p(bvh.blob), _p(grad_mixture), _p(grad_xes), None, 0,
                 ctypes.byref(shape), int(need_mixture), int(need_xes), _stream(dev)))
    return grad_mixture, grad_xes


def check_convolution_input(data: torch.Tensor, kernels: torch.Tensor) -> ConvShape:
    """Rules and messages of convolution::forward_impl_t (src/gmc/cpp/extensions/convolution/implementation_forward.h:35-43);
    its n_batch x n_layers < 65535 grid limit does not apply here."""
    if data.dim() != 4 or kernels.dim() != 4:
        raise RuntimeError("data and kernels must have 4 dimensions")
    d = n_dimensions(data)
    if data.shape[2] < 1 or kernels.shape[2] < 1:
        raise RuntimeError("number of components must be greater 1 for this implementation")
    if data.shape[1] != kernels.shape[1]:
        raise RuntimeError("number of input feature maps must agree with the second kernel dimension")
    if n_dimensions(kernels) != d:
        raise RuntimeError("number of dimensions of data and kernel must agree")
    if data.dtype != kernels.dtype:
        raise RuntimeError("kernel and data dtypes must agree")
    if data.dtype not in (torch.float32, torch.float64):
        raise RuntimeError("unsupported datatype: the convolution is implemented for float32 and float64")
    if data.device != kernels.device:
        raise RuntimeError("data and kernel devices must agree")
    if not data.is_contiguous() or not kernels.is_contiguous():
        raise RuntimeError("data and kernels must be contiguous")
    if not data.is_cuda:
        raise RuntimeError("gmc_hip convolves on an AMD GPU only: data and kernels must be HIP ('cuda') tensors; "
                           "this build has no CPU implementation")
    return ConvShape(data.shape[0], data.shape[1], kernels.shape[0], data.shape[2], kernels.shape[2], d,
                     GMC_F32 if data.dtype == torch.float32 else GMC_F64)


def convolution_fwd(data: torch.Tensor, kernels: torch.Tensor) -> torch.Tensor:
    shape = check_convolution_input(data, kernels)
    out = torch.empty((shape.B, shape.Cout, shape.Nd * shape.Cin * shape.Nk, data.shape[-1]), dtype=data.dtype,
                      device=data.device)
    with _on(data.device):
        check(lib().gmc_convolution_fwd(_p(data), _p(kernels), _p(out), ctypes.byref(shape), _stream(data.device)))
    return out


def convolution_bwd(grad_out: torch.Tensor, data: torch.Tensor, kernels: torch.Tensor, need_data: bool = True,
                    need_kernels: bool = True):
    """-> (grad_data, grad_kernels); a gradient that is not asked for comes back as zeros, like the reference's"""
    shape = check_convolution_input(data, kernels)
    expected = (shape.B, shape.Cout, shape.Nd * shape.Cin * shape.Nk, data.shape[-1])
    if tuple(grad_out.shape) != expected or grad_out.dtype != data.dtype or grad_out.device != data.device:
        raise RuntimeError("grad_output must have the shape, dtype and device of the convolution result")
    if not grad_out.is_contiguous():
        raise RuntimeError("grad_output must be contiguous")
    grad_data = torch.empty_like(data) if need_data else torch.zeros_like(data)
    grad_kernels = torch.empty_like(kernels) if need_kernels else torch.zeros_like(kernels)
    with _on(data.device):
        check(lib().gmc_convolution_bwd(_p(grad_out), _p(data), _p(kernels), _p(grad_data), _p(grad_kernels),
                                        ctypes.byref(shape), int(need_data), int(need_kernels), _stream(data.device)))
    return grad_data, grad_kernels
