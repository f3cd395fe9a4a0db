"""Host side of libsrwm_hip.so: loads the C-ABI library with ctypes and exposes the four
extension-level functions with the positional tensor lists of the reference's pybind
modules (supervised_learning/self_ref_v0/self_ref_v0.cu:1344-1356,
supervised_learning/fast_weight/fast_weight_cuda.cu:667-679):

    self_ref_forward(x, W_y, W_q, W_k, w_b, q, k, beta, y_diff, q_diff, k_diff, beta_diff, out)
    self_ref_backward(x, q, k, beta, y_diff, q_diff, k_diff, beta_diff, grad_out,
                      W_y, W_q, W_k, w_b, grad_x, grad_W_y, grad_W_q, grad_W_k, grad_w_b)
    fast_weight_forward(q, k, v, beta, v_old, v_insert, kv, out)
    fast_weight_backward(q, k, v, beta, v_old, v_insert, grad_out, kv,
                         grad_q, grad_k, grad_v, grad_beta)

PyTorch is used for device memory and streams only.  There is no CPU path: a missing
library, a CPU tensor or a non-float32 tensor raises.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_PKG = os.path.dirname(_HERE)
LIB_PATH = os.path.join(_PKG, "lib", "libsrwm_hip.so")
CSRC = os.path.join(_PKG, "csrc")

# flags of include/srwm_hip.h
GRAD_STATE_ZERO = 0
GRAD_STATE_IN = 1
GRAD_STATE_ACCUM = 2
FLAG_GENERIC = 16
FLAG_NO_FALLBACK = 8192    # raise where the register-resident kernels do not take the call instead of running the LDS-resident ones
FLAG_CHUNKWISE = 32     # delta forward: chunkwise MFMA kernel (E == M in {64, 128})
FLAG_EXACT_PRODUCTS = 512   # chunkwise kernels with bf16 inputs: every product from hi + lo operand pairs
FLAG_BF16_GRADS = 1024      # chunkwise delta backward with bf16 inputs: grad_q, grad_k, grad_v written as bf16 by the library
FLAG_SPARSE_V_OLD = 4096    # chunkwise delta forward: v_old only for steps with |beta| < 2^-24 (all a chunkwise backward reads of it)
FLAG_NORM_EPS = 2048        # delta_layer_prologue: 1e-5 added to the normalisers of q and k
FLAG_STATE_SHIFT = 64      # layer entry points: the state tensors hold W minus the shared weights
FLAG_FRESH_STATE = 128     # layer forward: start from the shared weights
FLAG_SOFTMAX_INPUT = 256   # layer entry points: x is given before its softmax

ABI_VERSION = 17

# True: a call that the register-resident kernels do not take (head size without an instantiation, misaligned
# base or strides) raises instead of running on the several times slower LDS-resident kernels
NO_FALLBACK = False

_lib = None

_F = ctypes.c_void_p      # device float*
_S = ctypes.POINTER(ctypes.c_int64)
_I = ctypes.c_int
_U = ctypes.c_uint

_SIGNATURES = {
    "srwm_forward_f32": [_F, _S] + [_F] * 12 + [_I] * 4 + [_U, ctypes.c_void_p],
    "srwm_forward_bf16": [_F, _S] + [_F] * 12 + [_I] * 4 + [_U, ctypes.c_void_p],
    "srwm_backward_bf16": [_F, _S] + [_F] * 7 + [_F, _S] + [_F] * 9 + [_I] * 4 + [_U, ctypes.c_void_p],
    "srwm_forward_wide_f32": [_F, _S] + [_F] * 12 + [_I] * 5 + [_U, ctypes.c_void_p],
    "srwm_backward_wide_f32": [_F, _S] + [_F] * 7 + [_F, _S] + [_F] * 9 + [_I] * 5 + [_U, ctypes.c_void_p],
    "srwm_layer_forward_f32": [_F, _S] + [_F] * 17 + [_S] + [_I] * 5 + [_U, ctypes.c_void_p],
    "srwm_layer_backward_f32": [_F, _S] + [_F] * 7 + [_F, _S] + [_F] * 9 + [_S] + [_F] * 8 + [_I] * 5 + [_U, ctypes.c_void_p],
    "srwm_layer_backward_noalloc_f32": [_F, _S] + [_F] * 7 + [_F, _S] + [_F] * 9 + [_S] + [_F] * 4 + [_I] * 5 + [_U, ctypes.c_void_p],
    "srwm_layer_forward_bf16": [_F, _S] + [_F] * 17 + [_S] + [_I] * 5 + [_U, ctypes.c_void_p],
    "srwm_layer_backward_bf16": [_F, _S] + [_F] * 7 + [_F, _S] + [_F] * 9 + [_S] + [_F] * 8 + [_I] * 5 + [_U, ctypes.c_void_p],
    "srwm_forward_steps_f32": [_F, _S] + [_F] * 17 + [_I] * 4 + [_U, ctypes.c_void_p],
    "srwm_readout_grad_wide_f32": [_F] * 5 + [_F, _S] + [_F] * 2 + [_I] * 5 + [_U, ctypes.c_void_p],
    "srwm_layer_readout_grad_f32": [_F, _S] + [_F] * 5 + [_F, _S] + [_F, _F, _S] + [_F] * 2 + [_I] * 5 + [_U, ctypes.c_void_p],
    "srwm_readout_grad_f32": [_F] * 5 + [_F, _S] + [_F] * 2 + [_I] * 4 + [_U, ctypes.c_void_p],
    "srwm_backward_f32": [_F, _S] + [_F] * 7 + [_F, _S] + [_F] * 9 + [_I] * 4 + [_U, ctypes.c_void_p],
    "delta_forward_steps_f32": [_F, _S] * 4 + [_F] * 5 + [_S] + [_I] * 5 + [_U, ctypes.c_void_p],
    "delta_readout_replay_f32": [_F, _S] + [_F, _F] + [_F, _S] + [_F, _F] + [_I] * 5 + [_U, ctypes.c_void_p],
    "delta_steps_backward_f32": [_F, _S] * 4 + [_F] * 3 + [_F, _S] + [_F] * 5 + [_I] * 5 + [_U, ctypes.c_void_p],
    "delta_forward_f32": [_F, _S] * 4 + [_F] * 4 + [_S] + [_I] * 5 + [_U, ctypes.c_void_p],
    "delta_backward_f32": [_F, _S] * 4 + [_F, _F] + [_F, _S] + [_F] * 6 + [_I] * 5 + [_U, ctypes.c_void_p],
    "delta_forward_bf16": [_F, _S] * 4 + [_F] * 4 + [_S] + [_I] * 5 + [_U, ctypes.c_void_p],
    "delta_backward_bf16": [_F, _S] * 4 + [_F, _F] + [_F, _S] + [_F] * 6 + [_I] * 5 + [_U, ctypes.c_void_p],
    "delta_layer_prologue_f32": [_F] * 6 + [_I] * 5 + [_U, ctypes.c_void_p],
    "delta_layer_prologue_grad_f32": [_F, _S] * 4 + [_F] * 5 + [_I] * 5 + [_U, ctypes.c_void_p],
    "delta_layer_prologue_bf16": [_F] * 6 + [_I] * 5 + [_U, ctypes.c_void_p],
    "delta_layer_prologue_grad_bf16": [_F, _S] * 4 + [_F] * 5 + [_I] * 5 + [_U, ctypes.c_void_p],
}


def build(verbose=False):
    """Compile libsrwm_hip.so for gfx950 with hipcc (always recompiles)."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.check_call(["make", "-C", CSRC, "-B", "-j8"], stdout=out, stderr=out)
    return LIB_PATH


def lib():
    """The loaded library.  Raises if it has not been built -- there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC}` "
                "(or __graft_entry__.build()); the HIP kernels have no CPU/PyTorch fallback")
        L = ctypes.CDLL(LIB_PATH)
        L.srwm_hip_abi_version.restype = _I
        if L.srwm_hip_abi_version() != ABI_VERSION:
            raise RuntimeError("libsrwm_hip.so ABI version mismatch; rebuild the library")
        for name, args in _SIGNATURES.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = _I
        L.srwm_hip_strerror.restype = ctypes.c_char_p
        L.srwm_hip_strerror.argtypes = [_I]
        L.srwm_hip_limits.argtypes = [ctypes.POINTER(_I)] * 3
        L.srwm_hip_limits.restype = _I
        L.srwm_hip_scratch_bytes.restype = ctypes.c_size_t
        L.srwm_hip_scratch_bytes.argtypes = []
        L.srwm_hip_fallback_calls.restype = ctypes.c_uint64
        L.srwm_hip_fallback_calls.argtypes = []
        _lib = L
    return _lib


def fallback_calls():
    """Calls since the library was loaded that the register-resident kernels did not take (head size, alignment) and the
    several times slower LDS-resident kernels served; calls that asked for those with FLAG_GENERIC are not counted."""
    return int(lib().srwm_hip_fallback_calls())


def limits(device=None):
    """(max E of SRWM forward, max E of SRWM backward, max E == M of the delta rule)."""
    a, b, c = _I(), _I(), _I()
    with torch.cuda.device(device):
        lib().srwm_hip_limits(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
    return a.value, b.value, c.value


def _check(code, what):
    if code != 0:
        msg = lib().srwm_hip_strerror(code).decode()
        raise RuntimeError(f"{what} failed with code {code}: {msg}")


def _require(t, name, shape=None, dtype=torch.float32):
    # runs some twenty times per operator call, on a path that is host-bound for single-step calls:
    # only attribute reads and identity / tuple comparisons on the success path
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got {t.device}); there is no CPU path")
    if t.dtype is not dtype:
        raise TypeError(f"{name} must be {dtype} (got {t.dtype})")
    if shape is not None and t.shape != shape:
        raise ValueError(f"{name} has shape {tuple(t.shape)}, expected {tuple(shape)}")


def _fam(flags):
    return flags | FLAG_NO_FALLBACK if NO_FALLBACK and not flags & FLAG_GENERIC else flags


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _rows_ok(t):
    """Can the kernels address this tensor through (n, h, l) strides: last axis contiguous, rows
    aligned to four elements."""
    ok = t.stride(-1) == 1 or t.shape[-1] == 1
    if ok and t.shape[-1] % 4 == 0:
        ok = t.data_ptr() % (4 * t.element_size()) == 0 and all(s % 4 == 0 for s in t.stride()[:3])
    return ok


def _strided(t):
    """A tensor the kernels can read through (n, h, l) strides.  Anything else is copied."""
    if not _rows_ok(t):
        t = t.contiguous()
    return t, (ctypes.c_int64 * 3)(*t.stride()[:3])


class _Dense:
    """Context for tensors the kernels address densely: contiguous ones pass through; others
    are staged through a contiguous copy that is written back on exit when `writeback`."""

    def __init__(self, tensors, writeback):
        self.orig = list(tensors)
        self.writeback = writeback
        self.work = [t if t.is_contiguous() else t.contiguous() for t in self.orig]

    def __enter__(self):
        return self.work

    def __exit__(self, *exc):
        if self.writeback and exc[0] is None:
            for o, w in zip(self.orig, self.work):
                if o is not w:
                    o.copy_(w)
        return False


def _has_bf16_kernel(E, M):
    return E == M and E in (8, 16, 32, 64, 128)


# torch's own fast path to the current stream's handle (what its compiled-code launchers use); the
# public Stream object costs several microseconds to build per call
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device):
    if _raw_stream is not None and device.index is not None:
        return ctypes.c_void_p(_raw_stream(device.index))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def self_ref_forward(x, W_y, W_q, W_k, w_b, q, k, beta, y_diff, q_diff, k_diff, beta_diff, out,
                     flags=0):
    """SRWM forward over the whole sequence.  W_y, W_q, W_k, w_b are overwritten with the
    final state; q ... out are overwritten with the per-step vectors.  W_y is (N, H, E, Y):
    Y = E for the plain operator, any other width (3E+1 in the reference's second variant)
    makes out and y_diff (N, H, L, Y).  x and out may both be bfloat16; everything else stays
    float32."""
    io = x.dtype if isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 else torch.float32
    _require(x, "x", None, io)
    N, H, L, E = x.shape
    _require(W_y, "W_y")
    Y = W_y.shape[-1]
    _require(W_y, "W_y", (N, H, E, Y))
    for t, nm in ((W_q, "W_q"), (W_k, "W_k")):
        _require(t, nm, (N, H, E, E))
    _require(w_b, "w_b", (N, H, E, 4))
    for t, nm in ((q, "q"), (k, "k"), (q_diff, "q_diff"), (k_diff, "k_diff")):
        _require(t, nm, (N, H, L, E))
    _require(y_diff, "y_diff", (N, H, L, Y))
    _require(out, "out", (N, H, L, Y), io)
    _require(beta, "beta", (N, H, L, 4))
    _require(beta_diff, "beta_diff", (N, H, L, 4))
    if x.numel() == 0 or Y == 0:
        return
    xs, xstr = _strided(x)
    null = ctypes.c_void_p(None)
    with torch.cuda.device(x.device), \
            _Dense([W_y, W_q, W_k, w_b, q, k, beta, y_diff, q_diff, k_diff, beta_diff, out], True) as d:
        if io == torch.bfloat16 and Y == E:
            name = "srwm_forward_bf16"
            code = lib().srwm_forward_bf16(_ptr(xs), xstr, *[_ptr(t) for t in d], N, H, L, E, _fam(flags),
                                           _stream(x.device))
        elif io == torch.bfloat16:   # wide output block: the layer entry point without any of its extras
            name = "srwm_layer_forward_bf16"
            code = lib().srwm_layer_forward_bf16(_ptr(xs), xstr, null, null, null, null, null,
                                                 *[_ptr(t) for t in d], None, N, H, L, E, Y, _fam(flags), _stream(x.device))
        elif Y == E:
            name = "srwm_forward_f32"
            code = lib().srwm_forward_f32(_ptr(xs), xstr, *[_ptr(t) for t in d], N, H, L, E, _fam(flags),
                                          _stream(x.device))
        else:
            name = "srwm_forward_wide_f32"
            code = lib().srwm_forward_wide_f32(_ptr(xs), xstr, *[_ptr(t) for t in d], N, H, L, E, Y,
                                               _fam(flags), _stream(x.device))
    _check(code, name)


def self_ref_forward_steps(x, keep, slow, W_y, W_q, W_k, w_b, q, k, beta, y_diff, q_diff, k_diff,
                           beta_diff, out, flags=0):
    """SRWM forward over all steps of an unroll with per-step resets: where keep[n, t] == 0 the
    state of batch row n is replaced, before step t, by the shared weights `slow` = (W_y, W_q,
    W_k: (1 or no batch axis, H, E, E), w_b: (..., H, E, 4)).  keep: (N, L) float32 or None.
    Otherwise as self_ref_forward.  A W_y of another width (N, H, E, Y) selects the wide-output form."""
    _require(x, "x")
    N, H, L, E = x.shape
    if isinstance(W_y, torch.Tensor) and W_y.dim() == 4 and W_y.shape[-1] != E:
        return self_ref_layer_forward(x, keep, slow, W_y, W_q, W_k, w_b, q, k, beta, y_diff, q_diff, k_diff,
                                      beta_diff, out, flags=flags)
    for t, nm in ((W_y, "W_y"), (W_q, "W_q"), (W_k, "W_k")):
        _require(t, nm, (N, H, E, E))
    _require(w_b, "w_b", (N, H, E, 4))
    for t, nm in ((q, "q"), (k, "k"), (y_diff, "y_diff"), (q_diff, "q_diff"), (k_diff, "k_diff"),
                  (out, "out")):
        _require(t, nm, (N, H, L, E))
    _require(beta, "beta", (N, H, L, 4))
    _require(beta_diff, "beta_diff", (N, H, L, 4))
    null = ctypes.c_void_p(None)
    sl = [null] * 4
    if keep is not None:
        _require(keep, "keep", (N, L))
        keep = keep.contiguous()
        shapes = ((H, E, E),) * 3 + ((H, E, 4),)
        sl = []
        for t, shp, nm in zip(slow, shapes, ("slow W_y", "slow W_q", "slow W_k", "slow w_b")):
            t = t.detach().reshape(shp) if isinstance(t, torch.Tensor) and t.numel() == H * E * shp[-1] else t
            _require(t, nm, shp)
            sl.append(t.contiguous())
    if x.numel() == 0:
        return
    xs, xstr = _strided(x)
    with torch.cuda.device(x.device), \
            _Dense([W_y, W_q, W_k, w_b, q, k, beta, y_diff, q_diff, k_diff, beta_diff, out], True) as d:
        code = lib().srwm_forward_steps_f32(
            _ptr(xs), xstr, _ptr(keep) if keep is not None else null,
            *[(_ptr(t) if keep is not None else t) for t in sl],
            *[_ptr(t) for t in d], N, H, L, E, _fam(flags), _stream(x.device))
    _check(code, "srwm_forward_steps_f32")


def self_ref_readout_grad(k, beta, y_diff, keep, slow_W_y, grad_out, W_y_entry, grad_x, flags=0):
    """grad_x[n, h, t] = W_y,t-1 grad_out[n, h, t] for an unroll whose carried state is detached
    between steps; W_y_entry is the (N, H, E, E) y block as it was before self_ref_forward_steps.
    flags: FLAG_GENERIC forces the LDS-resident kernel."""
    _require(k, "k")
    N, H, L, E = k.shape
    _require(y_diff, "y_diff")
    Y = y_diff.shape[-1]                      # width of the output block (E, or 3E+1 for the wide variant)
    _require(beta, "beta", (N, H, L, 4))
    _require(y_diff, "y_diff", (N, H, L, Y))
    _require(grad_out, "grad_out", (N, H, L, Y))
    _require(W_y_entry, "W_y_entry", (N, H, E, Y))
    _require(grad_x, "grad_x", (N, H, L, E))
    null = ctypes.c_void_p(None)
    if keep is not None:
        _require(keep, "keep", (N, L))
        keep = keep.contiguous()
        slow_W_y = slow_W_y.detach().reshape(H, E, Y).contiguous()
        _require(slow_W_y, "slow W_y", (H, E, Y))
    if k.numel() == 0:
        return
    gos, gstr = _strided(grad_out)
    with torch.cuda.device(k.device), _Dense([k, beta, y_diff, W_y_entry], False) as sv, \
            _Dense([grad_x], True) as gr:
        code = lib().srwm_readout_grad_wide_f32(
            _ptr(sv[0]), _ptr(sv[1]), _ptr(sv[2]), _ptr(keep) if keep is not None else null,
            _ptr(slow_W_y) if keep is not None else null, _ptr(gos), gstr, _ptr(sv[3]), _ptr(gr[0]),
            N, H, L, E, Y, _fam(flags), _stream(k.device))
    _check(code, "srwm_readout_grad_wide_f32")


def self_ref_layer_readout_grad(x, k, beta, y_diff, keep, slow_W_y, grad_out, W_y_entry, grad_x, grad_W_y,
                                grad_slow_W_y, flags=0):
    """self_ref_readout_grad plus the gradient of the shared W_y, for a layer's whole unroll:
    grad_x[n, h, t] = W_y,t-1 grad_out[n, h, t]; grad_W_y[n, h] = sum_t x_t (x) grad_out_t
    ((N, H, E, Y), written); grad_slow_W_y (H, E, Y) = its sum over the batch.  x: the operator's
    input (soft-maxed if the layer soft-maxes it), any strides.  flags: FLAG_STATE_SHIFT (W_y_entry
    is the carried shift from the shared weights), FLAG_GENERIC."""
    _require(k, "k")
    N, H, L, E = k.shape
    _require(y_diff, "y_diff")
    Y = y_diff.shape[-1]
    _require(x, "x", (N, H, L, E))
    _require(beta, "beta", (N, H, L, 4))
    _require(y_diff, "y_diff", (N, H, L, Y))
    _require(grad_out, "grad_out", (N, H, L, Y))
    _require(W_y_entry, "W_y_entry", (N, H, E, Y))
    _require(grad_x, "grad_x", (N, H, L, E))
    _require(grad_W_y, "grad_W_y", (N, H, E, Y))
    _require(grad_slow_W_y, "grad_slow_W_y", (H, E, Y))
    if not (grad_W_y.is_contiguous() and grad_slow_W_y.is_contiguous()):
        raise ValueError("grad_W_y and grad_slow_W_y must be contiguous")
    slow_W_y = slow_W_y.detach().reshape(H, E, Y).contiguous()
    _require(slow_W_y, "slow W_y", (H, E, Y))
    null = ctypes.c_void_p(None)
    if keep is not None:
        _require(keep, "keep", (N, L))
        keep = keep.contiguous()
    if k.numel() == 0:
        grad_W_y.zero_()
        grad_slow_W_y.zero_()
        return
    xs, xstr = _strided(x)
    gos, gstr = _strided(grad_out)
    with torch.cuda.device(k.device), _Dense([k, beta, y_diff, W_y_entry], False) as sv, \
            _Dense([] if grad_x.stride(-1) == 1 else [grad_x], True) as gr:
        gxt = gr[0] if gr else grad_x   # rows at any strides: a permuted buffer is written in place
        code = lib().srwm_layer_readout_grad_f32(
            _ptr(xs), xstr, _ptr(sv[0]), _ptr(sv[1]), _ptr(sv[2]), _ptr(keep) if keep is not None else null,
            _ptr(slow_W_y), _ptr(gos), gstr, _ptr(sv[3]), _ptr(gxt), (ctypes.c_int64 * 3)(*gxt.stride()[:3]),
            _ptr(grad_W_y), _ptr(grad_slow_W_y), N, H, L, E, Y, _fam(flags), _stream(k.device))
    _check(code, "srwm_layer_readout_grad_f32")


def self_ref_backward(x, q, k, beta, y_diff, q_diff, k_diff, beta_diff, grad_out,
                      W_y, W_q, W_k, w_b, grad_x, grad_W_y, grad_W_q, grad_W_k, grad_w_b,
                      flags=GRAD_STATE_ACCUM):
    """SRWM backward.  W_* must hold the final state the forward left behind.  By default
    behaves like the reference extension function: the grad_W buffers are read as the
    gradient w.r.t. the final state and the result is added to them (identical to a plain
    overwrite when they arrive zero-filled, which is how SelfRefv0.backward calls it).
    W_y (N, H, E, Y) fixes the width of y_diff, grad_out and grad_W_y.  x and grad_out may both be
    bfloat16; grad_x and everything else stay float32."""
    io = x.dtype if isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 else torch.float32
    _require(x, "x", None, io)
    N, H, L, E = x.shape
    _require(W_y, "W_y")
    Y = W_y.shape[-1]
    for t, nm in ((q, "q"), (k, "k"), (q_diff, "q_diff"), (k_diff, "k_diff"), (grad_x, "grad_x")):
        _require(t, nm, (N, H, L, E))
    _require(y_diff, "y_diff", (N, H, L, Y))
    _require(grad_out, "grad_out", (N, H, L, Y), io)
    _require(beta, "beta", (N, H, L, 4))
    _require(beta_diff, "beta_diff", (N, H, L, 4))
    for t, nm in ((W_y, "W_y"), (grad_W_y, "grad_W_y")):
        _require(t, nm, (N, H, E, Y))
    for t, nm in ((W_q, "W_q"), (W_k, "W_k"), (grad_W_q, "grad_W_q"), (grad_W_k, "grad_W_k")):
        _require(t, nm, (N, H, E, E))
    _require(w_b, "w_b", (N, H, E, 4))
    _require(grad_w_b, "grad_w_b", (N, H, E, 4))
    if x.numel() == 0 or Y == 0:
        # no steps: the state gradient passes through unchanged (zero when none came in)
        if (flags & 3) == GRAD_STATE_ZERO:
            for g in (grad_W_y, grad_W_q, grad_W_k, grad_w_b):
                g.zero_()
        return
    xs, xstr = _strided(x)
    gos, gstr = _strided(grad_out)
    with torch.cuda.device(x.device), \
            _Dense([q, k, beta, y_diff, q_diff, k_diff, beta_diff], False) as sv, \
            _Dense([W_y, W_q, W_k, w_b], False) as st, \
            _Dense([grad_x, grad_W_y, grad_W_q, grad_W_k, grad_w_b], True) as gr:
        if io == torch.bfloat16 and Y == E:
            name = "srwm_backward_bf16"
            code = lib().srwm_backward_bf16(_ptr(xs), xstr, *[_ptr(t) for t in sv], _ptr(gos), gstr,
                                            *[_ptr(t) for t in st], *[_ptr(t) for t in gr],
                                            N, H, L, E, _fam(flags), _stream(x.device))
        elif io == torch.bfloat16:
            null = ctypes.c_void_p(None)
            name = "srwm_layer_backward_bf16"
            code = lib().srwm_layer_backward_bf16(_ptr(xs), xstr, *[_ptr(t) for t in sv], _ptr(gos), gstr,
                                                  null, null, null, null, *[_ptr(t) for t in st],
                                                  _ptr(gr[0]), None, *[_ptr(t) for t in gr[1:]], null, null, null, null,
                                                  N, H, L, E, Y, _fam(flags), _stream(x.device))
        elif Y == E:
            name = "srwm_backward_f32"
            code = lib().srwm_backward_f32(_ptr(xs), xstr, *[_ptr(t) for t in sv], _ptr(gos), gstr,
                                           *[_ptr(t) for t in st], *[_ptr(t) for t in gr],
                                           N, H, L, E, _fam(flags), _stream(x.device))
        else:
            name = "srwm_backward_wide_f32"
            code = lib().srwm_backward_wide_f32(_ptr(xs), xstr, *[_ptr(t) for t in sv], _ptr(gos), gstr,
                                                *[_ptr(t) for t in st], *[_ptr(t) for t in gr],
                                                N, H, L, E, Y, _fam(flags), _stream(x.device))
    _check(code, name)


def _shared(slow, H, E, Y):
    """The layer's parameters as dense (H, E, .) tensors; a leading batch axis of 1 is dropped."""
    shapes = ((H, E, Y), (H, E, E), (H, E, E), (H, E, 4))
    out = []
    for t, shp, nm in zip(slow, shapes, ("shared W_y", "shared W_q", "shared W_k", "shared w_b")):
        _require(t, nm)
        if t.dim() == 4 and t.shape[0] == 1:
            t = t[0]
        _require(t, nm, shp)
        out.append(t if t.is_contiguous() else t.detach().contiguous())   # only its address is used
    return out


def self_ref_layer_forward(x, keep, slow, W_y, W_q, W_k, w_b, q, k, beta, y_diff, q_diff, k_diff,
                           beta_diff, out, flags=0):
    """SRWM forward with the layers' prologue and epilogue inside the kernel: `slow` = the shared
    weights (W_y: (1, H, E, Y) or (H, E, Y), ...), read without a repeat(); flags FLAG_FRESH_STATE
    (start from them, W_* are outputs), FLAG_STATE_SHIFT (W_* hold the state minus the shared
    weights, in and out), FLAG_SOFTMAX_INPUT (x is soft-maxed by the kernel); keep as in
    self_ref_forward_steps.  x and out may both be bfloat16."""
    io = x.dtype if isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 else torch.float32
    _require(x, "x", None, io)
    N, H, L, E = x.shape
    _require(W_y, "W_y")
    Y = W_y.shape[-1]
    _require(W_y, "W_y", (N, H, E, Y))
    for t, nm in ((W_q, "W_q"), (W_k, "W_k")):
        _require(t, nm, (N, H, E, E))
    _require(w_b, "w_b", (N, H, E, 4))
    for t, nm in ((q, "q"), (k, "k"), (q_diff, "q_diff"), (k_diff, "k_diff")):
        _require(t, nm, (N, H, L, E))
    _require(y_diff, "y_diff", (N, H, L, Y))
    _require(out, "out", (N, H, L, Y), io)
    _require(beta, "beta", (N, H, L, 4))
    _require(beta_diff, "beta_diff", (N, H, L, 4))
    sl = _shared(slow, H, E, Y)
    null = ctypes.c_void_p(None)
    if keep is not None:
        _require(keep, "keep", (N, L))
        keep = keep.contiguous()
    if x.numel() == 0:
        if flags & FLAG_FRESH_STATE:   # no steps: the state is the shared weights (a zero shift)
            for w, sw in zip((W_y, W_q, W_k, w_b), sl):
                if flags & FLAG_STATE_SHIFT:
                    w.zero_()
                else:
                    w.copy_(sw.unsqueeze(0).expand_as(w))
        return
    xs, xstr = _strided(x)
    by_strides = _rows_ok(out)   # a permuted buffer is written in place
    with torch.cuda.device(x.device), \
            _Dense([W_y, W_q, W_k, w_b, q, k, beta, y_diff, q_diff, k_diff, beta_diff], True) as d, \
            _Dense([] if by_strides else [out], True) as o:
        ot = out if by_strides else o[0]
        name = "srwm_layer_forward_bf16" if io == torch.bfloat16 else "srwm_layer_forward_f32"
        code = getattr(lib(), name)(
            _ptr(xs), xstr, _ptr(keep) if keep is not None else null, *[_ptr(t) for t in sl],
            *[_ptr(t) for t in d], _ptr(ot), (ctypes.c_int64 * 3)(*ot.stride()[:3]), N, H, L, E, Y, _fam(flags),
            _stream(x.device))
    _check(code, name)


def self_ref_layer_backward(x, q, k, beta, y_diff, q_diff, k_diff, beta_diff, grad_out, slow,
                            W_y, W_q, W_k, w_b, grad_x, grad_W, grad_slow, flags=GRAD_STATE_ZERO):
    """Backward of self_ref_layer_forward (without resets).  W_*: the final state as the forward
    left it; grad_W: four (N, H, E, .) tensors (SRWM_GRAD_STATE_* semantics, per batch row);
    grad_slow: four (H, E, .) tensors receiving the sum of grad_W over the batch, or None.
    x and grad_out may both be bfloat16; every gradient comes back in float32."""
    io = x.dtype if isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 else torch.float32
    _require(x, "x", None, io)
    N, H, L, E = x.shape
    _require(W_y, "W_y")
    Y = W_y.shape[-1]
    for t, nm in ((q, "q"), (k, "k"), (q_diff, "q_diff"), (k_diff, "k_diff"), (grad_x, "grad_x")):
        _require(t, nm, (N, H, L, E))
    _require(y_diff, "y_diff", (N, H, L, Y))
    _require(grad_out, "grad_out", (N, H, L, Y), io)
    _require(beta, "beta", (N, H, L, 4))
    _require(beta_diff, "beta_diff", (N, H, L, 4))
    shapes = ((N, H, E, Y), (N, H, E, E), (N, H, E, E), (N, H, E, 4))
    for t, g, shp in zip((W_y, W_q, W_k, w_b), grad_W, shapes):
        _require(t, "state", shp)
        _require(g, "grad_W", shp)
        if not g.is_contiguous():
            raise ValueError("grad_W tensors must be contiguous")
    sl = _shared(slow, H, E, Y)
    null = ctypes.c_void_p(None)
    gsl = [null] * 4
    if grad_slow is not None:
        for g, shp in zip(grad_slow, ((H, E, Y), (H, E, E), (H, E, E), (H, E, 4))):
            _require(g, "grad_slow", shp)
            if not g.is_contiguous():
                raise ValueError("grad_slow tensors must be contiguous")
        gsl = [_ptr(g) for g in grad_slow]
    if x.numel() == 0:
        if (flags & 3) == GRAD_STATE_ZERO:
            for g in grad_W:
                g.zero_()
        if grad_slow is not None:
            for gs_, g in zip(grad_slow, grad_W):
                gs_.copy_(g.sum(0))
        return
    xs, xstr = _strided(x)
    gos, gstr = _strided(grad_out)
    with torch.cuda.device(x.device), \
            _Dense([q, k, beta, y_diff, q_diff, k_diff, beta_diff], False) as sv, \
            _Dense([W_y, W_q, W_k, w_b], False) as st, \
            _Dense([] if grad_x.stride(-1) == 1 else [grad_x], True) as gx:
        gxt = gx[0] if gx else grad_x   # any row strides: the kernels store grad_x element by element
        name = "srwm_layer_backward_bf16" if io == torch.bfloat16 else "srwm_layer_backward_f32"
        code = getattr(lib(), name)(
            _ptr(xs), xstr, *[_ptr(t) for t in sv], _ptr(gos), gstr, *[_ptr(t) for t in sl],
            *[_ptr(t) for t in st], _ptr(gxt), (ctypes.c_int64 * 3)(*gxt.stride()[:3]), *[_ptr(g) for g in grad_W], *gsl,
            N, H, L, E, Y, _fam(flags), _stream(x.device))
    _check(code, name)


def scratch_bytes():
    """Size of the static device array behind self_ref_layer_backward_noalloc."""
    return int(lib().srwm_hip_scratch_bytes())


def self_ref_layer_backward_noalloc(x, q, k, beta, y_diff, q_diff, k_diff, beta_diff, grad_out, slow,
                                    W_y, W_q, W_k, w_b, grad_x, grad_slow, flags=0):
    """self_ref_layer_backward without the per-row gradient tensors: they live in a static device
    array inside the library, so the call allocates nothing (every tensor must already be dense where
    the kernels need it dense; nothing is copied here).  grad_slow: four (H, E, .) tensors, required.
    Raises when N*H*E*(Y+2E+4) floats exceed scratch_bytes().  Calls that overlap on one GPU share the
    array and race; calls on one stream are ordered."""
    _require(x, "x")
    N, H, L, E = x.shape
    _require(W_y, "W_y")
    Y = W_y.shape[-1]
    for t, nm in ((q, "q"), (k, "k"), (q_diff, "q_diff"), (k_diff, "k_diff"), (grad_x, "grad_x")):
        _require(t, nm, (N, H, L, E))
    _require(y_diff, "y_diff", (N, H, L, Y))
    _require(grad_out, "grad_out", (N, H, L, Y))
    _require(beta, "beta", (N, H, L, 4))
    _require(beta_diff, "beta_diff", (N, H, L, 4))
    for t, shp in zip((W_y, W_q, W_k, w_b), ((N, H, E, Y), (N, H, E, E), (N, H, E, E), (N, H, E, 4))):
        _require(t, "state", shp)
    if not all(isinstance(t, torch.Tensor) and t.is_contiguous() for t in slow):
        raise ValueError("self_ref_layer_backward_noalloc copies nothing: the shared weights must be contiguous")
    sl = _shared(slow, H, E, Y)
    for g, shp in zip(grad_slow, ((H, E, Y), (H, E, E), (H, E, E), (H, E, 4))):
        _require(g, "grad_slow", shp)
    dense = [q, k, beta, y_diff, q_diff, k_diff, beta_diff, W_y, W_q, W_k, w_b, grad_x, *grad_slow]
    if not all(t.is_contiguous() for t in dense):
        raise ValueError("self_ref_layer_backward_noalloc copies nothing: saved vectors, state and gradients "
                         "must be contiguous")
    (xs, xstr), (gos, gstr) = _strided(x), _strided(grad_out)
    if xs is not x or gos is not grad_out:
        raise ValueError("self_ref_layer_backward_noalloc copies nothing: x and grad_out need a contiguous, "
                         "16-byte aligned last axis")
    with torch.cuda.device(x.device):
        code = lib().srwm_layer_backward_noalloc_f32(
            _ptr(x), xstr, *[_ptr(t) for t in (q, k, beta, y_diff, q_diff, k_diff, beta_diff)], _ptr(grad_out), gstr,
            *[_ptr(t) for t in sl], *[_ptr(t) for t in (W_y, W_q, W_k, w_b)], _ptr(grad_x), None,
            *[_ptr(g) for g in grad_slow], N, H, L, E, Y, _fam(flags), _stream(x.device))
    _check(code, "srwm_layer_backward_noalloc_f32")


# names of the extension functions of the reference's wide-output variant
# (reinforcement_learning/torchbeast/self_ref_v1/__init__.py:31-32): same call, W_y is (N,H,E,3E+1)
self_ref_forward_v1 = self_ref_forward
self_ref_backward_v1 = self_ref_backward


def fast_weight_forward(q, k, v, beta, v_old, v_insert, kv, out, flags=0):
    """Delta-rule forward.  kv ([N,H,E,M], fp32) is overwritten with the final memory.
    q, k, v, beta and out are all float32 or all bfloat16; v_old, v_insert and kv are float32.
    out may have any strides with a contiguous last axis (a permuted buffer is written in place)."""
    io = q.dtype if isinstance(q, torch.Tensor) and q.dtype == torch.bfloat16 else torch.float32
    _require(q, "q", None, io)
    N, H, L, E = q.shape
    _require(k, "k", (N, H, L, E), io)
    _require(v, "v", None, io)
    M = v.shape[-1]
    _require(v, "v", (N, H, L, M), io)
    _require(beta, "beta", (N, H, L, 1), io)
    _require(out, "out", (N, H, L, M), io)
    for t, nm in ((v_old, "v_old"), (v_insert, "v_insert")):
        _require(t, nm, (N, H, L, M))
    _require(kv, "kv", (N, H, E, M))
    if q.numel() == 0 or v.numel() == 0:
        return
    if io == torch.bfloat16 and not _has_bf16_kernel(E, M):
        # no bf16 kernel for this size: widen, run the fp32 kernels, round the output
        o32 = torch.empty(out.shape, device=out.device, dtype=torch.float32)
        fast_weight_forward(q.float(), k.float(), v.float(), beta.float(), v_old, v_insert, kv, o32, flags)
        out.copy_(o32)
        return
    fn = lib().delta_forward_bf16 if io == torch.bfloat16 else lib().delta_forward_f32
    (qs, qstr), (ks, kstr), (vs, vstr), (bs, bstr) = (_strided(t) for t in (q, k, v, beta))
    by_strides = _rows_ok(out)
    with torch.cuda.device(q.device), _Dense([v_old, v_insert, kv], True) as d, _Dense([] if by_strides else [out], True) as o:
        ot = out if by_strides else o[0]
        code = fn(_ptr(qs), qstr, _ptr(ks), kstr, _ptr(vs), vstr, _ptr(bs), bstr,
                  *[_ptr(t) for t in d], _ptr(ot), (ctypes.c_int64 * 3)(*ot.stride()[:3]), N, H, L, E, M, _fam(flags),
                  _stream(q.device))
    _check(code, fn.__name__)


def fast_weight_forward_steps(q, k, v, beta, keep, v_old, v_insert, kv, out, flags=0):
    """Delta-rule forward over all steps of an unroll; the memory is zeroed before step t of batch
    row n where keep[n, t] == 0 (keep: (N, L) float32 or None).  float32 only."""
    _require(q, "q")
    N, H, L, E = q.shape
    _require(k, "k", (N, H, L, E))
    _require(v, "v")
    M = v.shape[-1]
    _require(v, "v", (N, H, L, M))
    _require(beta, "beta", (N, H, L, 1))
    for t, nm in ((v_old, "v_old"), (v_insert, "v_insert"), (out, "out")):
        _require(t, nm, (N, H, L, M))
    _require(kv, "kv", (N, H, E, M))
    null = ctypes.c_void_p(None)
    if keep is not None:
        _require(keep, "keep", (N, L))
        keep = keep.contiguous()
    if q.numel() == 0 or v.numel() == 0:
        return
    (qs, qstr), (ks, kstr), (vs, vstr), (bs, bstr) = (_strided(t) for t in (q, k, v, beta))
    by_strides = _rows_ok(out)
    with torch.cuda.device(q.device), _Dense([v_old, v_insert, kv], True) as d, _Dense([] if by_strides else [out], True) as o:
        ot = out if by_strides else o[0]
        code = lib().delta_forward_steps_f32(_ptr(qs), qstr, _ptr(ks), kstr, _ptr(vs), vstr, _ptr(bs), bstr,
                                             _ptr(keep) if keep is not None else null,
                                             *[_ptr(t) for t in d], _ptr(ot), (ctypes.c_int64 * 3)(*ot.stride()[:3]),
                                             N, H, L, E, M, _fam(flags), _stream(q.device))
    _check(code, "delta_forward_steps_f32")


def fast_weight_readout_replay(k, v_insert, keep, grad_out, kv_entry, u, flags=0):
    """u[n, h, t] = W_{t-1} grad_out[n, h, t] for an unroll whose memory carries no gradient;
    kv_entry is the (N, H, E, M) memory as it was before fast_weight_forward_steps.
    flags: FLAG_GENERIC forces the LDS-resident kernel."""
    _require(k, "k")
    N, H, L, E = k.shape
    _require(v_insert, "v_insert")
    M = v_insert.shape[-1]
    _require(v_insert, "v_insert", (N, H, L, M))
    _require(grad_out, "grad_out", (N, H, L, M))
    _require(kv_entry, "kv_entry", (N, H, E, M))
    _require(u, "u", (N, H, L, E))
    null = ctypes.c_void_p(None)
    if keep is not None:
        _require(keep, "keep", (N, L))
        keep = keep.contiguous()
    if k.numel() == 0:
        return
    (ks, kstr), (gos, gstr) = _strided(k), _strided(grad_out)
    with torch.cuda.device(k.device), _Dense([v_insert, kv_entry], False) as sv, _Dense([u], True) as d:
        code = lib().delta_readout_replay_f32(_ptr(ks), kstr, _ptr(sv[0]), _ptr(keep) if keep is not None else null,
                                              _ptr(gos), gstr, _ptr(sv[1]), _ptr(d[0]), N, H, L, E, M, _fam(flags),
                                              _stream(k.device))
    _check(code, "delta_readout_replay_f32")


def fast_weight_steps_backward(q, k, v, beta, keep, v_old, v_insert, grad_out, kv_entry, grad_q, grad_k, grad_v,
                               grad_beta, flags=0):
    """The whole backward of fast_weight_forward_steps (the memory carries no gradient): the replay
    of fast_weight_readout_replay and the per-step formulas, two launches.  grad_q, grad_k: (N, H, L, E);
    grad_v: (N, H, L, M); grad_beta: (N, H, L, 1); all overwritten."""
    _require(q, "q")
    N, H, L, E = q.shape
    _require(v, "v")
    M = v.shape[-1]
    _require(k, "k", (N, H, L, E))
    _require(v, "v", (N, H, L, M))
    _require(beta, "beta", (N, H, L, 1))
    for t, nm in ((v_old, "v_old"), (v_insert, "v_insert"), (grad_out, "grad_out"), (grad_v, "grad_v")):
        _require(t, nm, (N, H, L, M))
    _require(kv_entry, "kv_entry", (N, H, E, M))
    _require(grad_q, "grad_q", (N, H, L, E))
    _require(grad_k, "grad_k", (N, H, L, E))
    _require(grad_beta, "grad_beta", (N, H, L, 1))
    null = ctypes.c_void_p(None)
    if keep is not None:
        _require(keep, "keep", (N, L))
        keep = keep.contiguous()
    if q.numel() == 0:
        return
    (qs, qstr), (ks, kstr), (vs, vstr), (bs, bstr), (gos, gstr) = (_strided(t) for t in (q, k, v, beta, grad_out))
    with torch.cuda.device(q.device), _Dense([v_old, v_insert, kv_entry], False) as sv, \
            _Dense([grad_q, grad_k, grad_v, grad_beta], True) as d:
        code = lib().delta_steps_backward_f32(
            _ptr(qs), qstr, _ptr(ks), kstr, _ptr(vs), vstr, _ptr(bs), bstr, _ptr(keep) if keep is not None else null,
            _ptr(sv[0]), _ptr(sv[1]), _ptr(gos), gstr, _ptr(sv[2]), *[_ptr(t) for t in d], N, H, L, E, M, _fam(flags),
            _stream(q.device))
    _check(code, "delta_steps_backward_f32")


def delta_layer_prologue(rows, E, M, eps=False):
    """rows: (L, N, H, 2E+M+1) float32 or bfloat16, contiguous -- the delta-rule layers' projection [q~ | k~ | v | b~].
    Returns q, k: (L, N, H, E) normalised (elu + 1 over its sum, plus 1e-5 when `eps`), v: (L, N, H, M),
    beta: (L, N, H) = sigmoid, in the type of `rows`, and sums: (L, N, H, 2) float32; all freshly allocated and
    contiguous, from one launch."""
    io = rows.dtype if isinstance(rows, torch.Tensor) and rows.dtype == torch.bfloat16 else torch.float32
    _require(rows, "rows", None, io)
    L, N, H, W = rows.shape
    if W != 2 * E + M + 1 or not rows.is_contiguous():
        raise ValueError(f"rows must be contiguous with last axis 2E+M+1 = {2 * E + M + 1} (got {tuple(rows.shape)})")
    new = lambda *sh: torch.empty(sh, device=rows.device, dtype=io)
    q, k, v, beta = new(L, N, H, E), new(L, N, H, E), new(L, N, H, M), new(L, N, H)
    sums = torch.empty((L, N, H, 2), device=rows.device, dtype=torch.float32)
    if rows.numel():
        fn = lib().delta_layer_prologue_bf16 if io == torch.bfloat16 else lib().delta_layer_prologue_f32
        with torch.cuda.device(rows.device):
            code = fn(_ptr(rows), _ptr(q), _ptr(k), _ptr(v), _ptr(beta), _ptr(sums),
                      N, H, L, E, M, FLAG_NORM_EPS if eps else 0, _stream(rows.device))
        _check(code, fn.__name__)
    return q, k, v, beta, sums


def delta_layer_prologue_grad(grad_q, grad_k, grad_v, grad_beta, q, k, beta, sums):
    """Backward of delta_layer_prologue.  grad_q, grad_k: (N, H, L, E), grad_v: (N, H, L, M), grad_beta:
    (N, H, L, 1), any strides with a contiguous last axis (the operator's gradients as they are);
    q, k, beta, sums as delta_layer_prologue returned them.  Returns the gradient of `rows`, (L, N, H, 2E+M+1)."""
    L, N, H, E = q.shape
    M = grad_v.shape[-1]
    io = q.dtype if isinstance(q, torch.Tensor) and q.dtype == torch.bfloat16 else torch.float32
    _require(q, "q", None, io)
    _require(k, "k", (L, N, H, E), io)
    _require(beta, "beta", (L, N, H), io)
    _require(sums, "sums", (L, N, H, 2))
    gs = []
    for t, nm, w in ((grad_q, "grad_q", E), (grad_k, "grad_k", E), (grad_v, "grad_v", M), (grad_beta, "grad_beta", 1)):
        _require(t, nm, (N, H, L, w), io)
        if w > 1 and t.stride(-1) != 1:
            t = t.contiguous()
        gs.append((t, (ctypes.c_int64 * 3)(*t.stride()[:3])))
    q, k, beta, sums = (t.contiguous() for t in (q, k, beta, sums))
    grad_rows = torch.empty((L, N, H, 2 * E + M + 1), device=q.device, dtype=io)
    if grad_rows.numel():
        fn = lib().delta_layer_prologue_grad_bf16 if io == torch.bfloat16 else lib().delta_layer_prologue_grad_f32
        with torch.cuda.device(q.device):
            code = fn(*[a for t, st in gs for a in (_ptr(t), st)], _ptr(q), _ptr(k), _ptr(beta), _ptr(sums),
                      _ptr(grad_rows), N, H, L, E, M, 0, _stream(q.device))
        _check(code, fn.__name__)
    return grad_rows


def fast_weight_backward(q, k, v, beta, v_old, v_insert, grad_out, kv, grad_q, grad_k, grad_v,
                         grad_beta, grad_kv=None, flags=GRAD_STATE_ZERO):
    """Delta-rule backward.  kv must hold the final memory and is reverted to the initial
    one.  grad_kv (optional, beyond the reference's list): gradient of the memory, see
    the SRWM_GRAD_STATE_* flags."""
    io = q.dtype if isinstance(q, torch.Tensor) and q.dtype == torch.bfloat16 else torch.float32
    _require(q, "q", None, io)
    N, H, L, E = q.shape
    _require(k, "k", (N, H, L, E), io)
    _require(v, "v", None, io)
    M = v.shape[-1]
    _require(beta, "beta", (N, H, L, 1), io)
    for t, nm in ((v_old, "v_old"), (v_insert, "v_insert")):
        _require(t, nm, (N, H, L, M))
    _require(grad_out, "grad_out", (N, H, L, M), io)
    _require(kv, "kv", (N, H, E, M))
    # the library writes fp32 gradients; with bf16 inputs the caller may pass fp32 tensors
    # (used as they are) or bf16 ones (filled through an fp32 temporary)
    gdt = lambda t: torch.float32 if (isinstance(t, torch.Tensor) and t.dtype == torch.float32) else io
    _require(grad_q, "grad_q", (N, H, L, E), gdt(grad_q))
    _require(grad_k, "grad_k", (N, H, L, E), gdt(grad_k))
    _require(grad_v, "grad_v", (N, H, L, M), gdt(grad_v))
    _require(grad_beta, "grad_beta", (N, H, L, 1), gdt(grad_beta))
    if grad_kv is not None:
        _require(grad_kv, "grad_kv", (N, H, E, M))
    if q.numel() == 0 or v.numel() == 0:
        if grad_kv is not None and (flags & 3) == GRAD_STATE_ZERO:
            grad_kv.zero_()
        return
    if io == torch.bfloat16 and not _has_bf16_kernel(E, M):
        g32 = [torch.empty(t.shape, device=t.device, dtype=torch.float32)
               for t in (grad_q, grad_k, grad_v, grad_beta)]
        fast_weight_backward(q.float(), k.float(), v.float(), beta.float(), v_old, v_insert,
                             grad_out.float(), kv, *g32, grad_kv=grad_kv, flags=flags)
        for dst, src in zip((grad_q, grad_k, grad_v, grad_beta), g32):
            dst.copy_(src)
        return
    fn = lib().delta_backward_bf16 if io == torch.bfloat16 else lib().delta_backward_f32
    (qs, qstr), (ks, kstr), (vs, vstr), (bs, bstr), (gos, gstr) = (
        _strided(t) for t in (q, k, v, beta, grad_out))
    if io == torch.bfloat16:
        bf_outs = (grad_q, grad_k, grad_v, grad_beta)
        # The chunkwise kernels round grad_q, grad_k, grad_v themselves when all three are bf16, no
        # gradient of the memory is asked for and single products are allowed; grad_beta is fp32 there.
        native = (bool(flags & FLAG_CHUNKWISE) and not flags & FLAG_EXACT_PRODUCTS and grad_kv is None and
                  all(t.dtype == torch.bfloat16 for t in bf_outs[:3]))
        if native:
            flags |= FLAG_BF16_GRADS
        # otherwise the library returns every gradient in fp32 and bf16 destinations are rounded here
        grad_q, grad_k, grad_v, grad_beta = (
            t if t.dtype == torch.float32 or (native and i < 3)
            else torch.empty(t.shape, device=t.device, dtype=torch.float32)
            for i, t in enumerate(bf_outs))
    outs = [kv, grad_q, grad_k, grad_v, grad_beta] + ([grad_kv] if grad_kv is not None else [])
    with torch.cuda.device(q.device), _Dense([v_old, v_insert], False) as sv, _Dense(outs, True) as d:
        gkv = _ptr(d[5]) if grad_kv is not None else ctypes.c_void_p(None)
        code = fn(_ptr(qs), qstr, _ptr(ks), kstr, _ptr(vs), vstr, _ptr(bs), bstr,
                  _ptr(sv[0]), _ptr(sv[1]), _ptr(gos), gstr,
                  *[_ptr(t) for t in d[:5]], gkv, N, H, L, E, M, _fam(flags), _stream(q.device))
    _check(code, fn.__name__)
    if io == torch.bfloat16:
        for dst, src in zip(bf_outs, (grad_q, grad_k, grad_v, grad_beta)):
            if dst is not src:
                dst.copy_(src)
