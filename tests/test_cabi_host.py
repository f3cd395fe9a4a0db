"""CPU-side checks of the boundary: the shared library loads, exports every symbol that
include/srwm_hip.h declares, and the host layer refuses what it must refuse.  No kernel is
launched here."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "srwm_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    return re.findall(r"^SRWM_API\s+(?:const\s+)?\w+\s*\*?\s*(\w+)\s*\(", text, flags=re.M)


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ("srwm_forward_f32", "srwm_backward_f32", "delta_forward_f32", "delta_backward_f32",
                 "srwm_hip_limits", "srwm_hip_strerror", "srwm_hip_abi_version"):
        assert must in names


def test_library_exports_every_declared_symbol():
    import srwm_hip
    assert os.path.exists(srwm_hip.LIB_PATH), "build the library first (make -C modern-srwm_amd/csrc)"
    L = ctypes.CDLL(srwm_hip.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(L, name), name
    assert srwm_hip.lib().srwm_hip_abi_version() == srwm_hip.ABI_VERSION


def _prototypes():
    """name -> list of parameter declarations, parsed from the header."""
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    text = "\n".join(line for line in text.split("\n") if not line.lstrip().startswith("#"))
    out = {}
    for m in re.finditer(r"SRWM_API\s+(?:const\s+)?\w+\s*\*?\s*(\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        params = [p.strip() for p in m.group(2).split(",")]
        out[m.group(1)] = [] if params == ["void"] else params
    return out


def test_ctypes_signatures_match_the_header():
    """The host layer binds every compute entry point with the parameter list the header declares:
    same count, pointers where the header has pointers or arrays, ints where it has ints."""
    import srwm_hip
    protos = _prototypes()
    aux = {"srwm_hip_abi_version", "srwm_hip_strerror", "srwm_hip_limits", "srwm_hip_lds_probe",
           "srwm_hip_latency_probe", "srwm_hip_scratch_bytes", "srwm_hip_fallback_calls"}
    assert set(protos) - aux == set(srwm_hip._SIGNATURES), set(protos) - aux ^ set(srwm_hip._SIGNATURES)
    for name, args in srwm_hip._SIGNATURES.items():
        params = protos[name]
        assert len(params) == len(args), (name, len(params), len(args))
        for decl, ct in zip(params, args):
            if "*" in decl or "[" in decl:
                assert ct in (ctypes.c_void_p, srwm_hip._S), (name, decl)
            elif decl.startswith("unsigned"):
                assert ct is ctypes.c_uint, (name, decl)
            else:
                assert decl.startswith("int ") and ct is ctypes.c_int, (name, decl)


def test_error_strings():
    import srwm_hip
    L = srwm_hip.lib()
    assert b"success" in L.srwm_hip_strerror(0)
    assert b"invalid" in L.srwm_hip_strerror(-1)
    assert b"not supported" in L.srwm_hip_strerror(-2)
    assert b"stride" in L.srwm_hip_strerror(-3)


def test_cpu_tensors_are_refused_loudly():
    """There is no CPU or PyTorch fallback behind the operators."""
    import srwm_hip
    from self_ref_v0 import self_ref_v0
    from fast_weight import fast_weight_delta
    x = torch.zeros(1, 1, 2, 8)
    W = [torch.zeros(1, 1, 8, 8) for _ in range(3)] + [torch.zeros(1, 1, 8, 4)]
    with pytest.raises(KeyError):          # same failure as the reference: no "cpu" entry in .dot
        self_ref_v0(x, *W)
    outs = [torch.zeros(1, 1, 2, 8)] * 2 + [torch.zeros(1, 1, 2, 4)] + [torch.zeros(1, 1, 2, 8)] * 3 + \
           [torch.zeros(1, 1, 2, 4), torch.zeros(1, 1, 2, 8)]
    with pytest.raises(RuntimeError, match="no CPU path"):
        srwm_hip.self_ref_forward(x, *W, *outs)
    q = torch.zeros(1, 1, 2, 8)
    with pytest.raises((RuntimeError, AssertionError)):
        fast_weight_delta(q, q, q, torch.zeros(1, 1, 2, 1), torch.zeros(1, 1, 8, 8))


def test_shape_asserts_match_the_reference_wording():
    from self_ref_v0 import SelfRefv0, StatefulSelfRefv0, self_ref_v0, stateful_self_ref_v0
    x = torch.zeros(2, 3, 4, 8)
    good = torch.zeros(2, 3, 8, 8)
    with pytest.raises(AssertionError, match="Reshape/unsqueeze if needed."):
        self_ref_v0(x, good, good, good, torch.zeros(2, 3, 8, 3))
    with pytest.raises(AssertionError, match="Reshape/unsqueeze if needed."):
        stateful_self_ref_v0(x, good[:1], good, good, torch.zeros(2, 3, 8, 4))
    assert set(SelfRefv0.dot) == {"cuda"} and set(StatefulSelfRefv0.dot_backward) == {"cuda"}


def test_host_layer_uses_no_oracle_and_no_torch_math():
    """The product path must not import the oracle (it is test infrastructure)."""
    pkg = os.path.join(ROOT, "modern-srwm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text, f


def test_argument_validation_needs_no_gpu():
    """Every entry point rejects bad arguments before it touches the device, so the checks can be
    exercised here with placeholder pointers that are never dereferenced (all calls below return a
    negative code; nothing is launched)."""
    import srwm_hip
    L = srwm_hip.lib()
    P = ctypes.c_void_p
    fake = lambda: P(0x1000)                      # non-null, 16-byte aligned, never read
    ok_strides = (ctypes.c_int64 * 3)(64 * 16, 16, 16 * 8)
    huge = (ctypes.c_int64 * 3)(1 << 41, 16, 16)
    N, H, Ls, E = 2, 8, 4, 16
    srwm_f = lambda x, xs, n, e, flags: L.srwm_forward_f32(x, xs, *[fake() for _ in range(12)], n, H, Ls, e, flags, P(None))
    assert srwm_f(P(None), ok_strides, N, E, 0) == -1          # SRWM_EINVAL: null input
    assert srwm_f(fake(), None, N, E, 0) == -1                 # null stride array
    assert srwm_f(fake(), ok_strides, 0, E, 0) == -1           # empty batch
    assert srwm_f(fake(), ok_strides, N, -3, 0) == -1          # negative head size
    assert srwm_f(fake(), ok_strides, N, E, 32) == -1          # the chunkwise flag means nothing to the SRWM
    assert srwm_f(fake(), ok_strides, N, E, 1 << 20) == -1     # unknown flag bit
    assert srwm_f(fake(), ok_strides, N, E, 16 | 8192) == -1   # the LDS-resident kernels asked for and forbidden at once
    assert srwm_f(fake(), ok_strides, N, 6, 8192) == -4        # SRWM_ENOKERNEL: no register-resident kernel serves E = 6, and no fallback wanted
    assert srwm_f(P(0x1004), ok_strides, N, E, 8192) == -4     # nor for a base that is not 16-byte aligned
    assert srwm_f(fake(), huge, N, E, 0) == -3                 # SRWM_ESTRIDE: extent overflows the 2^40 bound
    assert srwm_f(fake(), ok_strides, N, 4096, 0) == -2        # SRWM_ESIZE: 4096 x 12292 floats fit no CU
    srwm_b = lambda flags: L.srwm_backward_f32(fake(), ok_strides, *[fake() for _ in range(7)], fake(), ok_strides,
                                               *[fake() for _ in range(9)], N, H, Ls, E, flags, P(None))
    assert srwm_b(3) == -1                                     # grad-state mode 3 does not exist
    delta_f = lambda flags, m, os=None: L.delta_forward_f32(*[a for _ in range(4) for a in (fake(), ok_strides)],
                                                            *[fake() for _ in range(4)], os, N, H, Ls, E, m, flags, P(None))
    assert delta_f(16 | 32, E) == -1                           # generic and chunkwise exclude each other
    assert delta_f(0, 0) == -1                                 # value width 0
    assert delta_f(32, E) == -4                                # SRWM_ENOKERNEL: no chunkwise kernel for E = M = 16
    assert delta_f(4096, E) == -1                              # v_old for the tiny betas only: a mode of the chunkwise kernels
    assert delta_f(32 | 4096, E) == -4                         # accepted with them
    i3 = lambda *v: (ctypes.c_int64 * 3)(*v)
    assert delta_f(32, E, i3(H * E, E, N * H * E)) == -4       # out as a [L,N,H,M] buffer: accepted
    assert delta_f(32, E, i3(H * E, E // 2, N * H * E)) == -3  # SRWM_ESTRIDE: rows of out overlap
    assert delta_f(32, E, i3(0, E, N * H * E)) == -3           # batch rows on top of each other
    assert delta_f(32, E, i3(H * E, E, -N * H * E)) == -3      # an output is not written backwards
    delta_b = lambda gW, flags: L.delta_backward_f32(*[a for _ in range(4) for a in (fake(), ok_strides)],
                                                     fake(), fake(), fake(), ok_strides, fake(), fake(), fake(), fake(),
                                                     fake(), gW, N, H, Ls, E, E, flags, P(None))
    assert delta_b(P(None), 1) == -1                           # an incoming state gradient needs the buffer
    assert delta_b(P(None), 32 | 1024) == -1                   # rounded gradients exist with bf16 inputs only
    delta_bb = lambda gW, flags, e: L.delta_backward_bf16(*[a for _ in range(4) for a in (fake(), ok_strides)],
                                                          fake(), fake(), fake(), ok_strides, fake(), fake(), fake(),
                                                          fake(), fake(), gW, N, H, Ls, e, e, flags, P(None))
    assert delta_bb(P(None), 1024, E) == -1                    # ... and in the chunkwise kernels only,
    assert delta_bb(P(None), 32 | 512 | 1024, E) == -1         # with single products,
    assert delta_bb(fake(), 32 | 1024, E) == -1                # and without the gradient of the memory
    assert delta_bb(P(None), 32 | 1024, E) == -4               # accepted; SRWM_ENOKERNEL: E = M = 16 has no chunkwise kernel
    # "the forward left rows of v_old out" (4096): refused by every backward that reads all rows of it
    assert delta_b(P(None), 4096) == -1                        # the step-by-step sweep
    assert delta_b(P(None), 16 | 4096) == -1                   # the LDS-resident one
    assert delta_b(P(None), 32 | 4096) == -4                   # chunkwise, fp32: accepted (no kernel at E = M = 16)
    assert delta_bb(P(None), 4096, E) == -1                    # bf16 step-by-step
    assert delta_bb(P(None), 32 | 4096, E) == -1               # chunkwise with single products and fp32 gradients
    assert delta_bb(P(None), 32 | 512 | 4096, E) == -4         # operand pairs everywhere: accepted
    assert delta_bb(P(None), 32 | 1024 | 4096, E) == -4        # rounded gradients: accepted
    layer_f = lambda sw, flags, os=None: L.srwm_layer_forward_f32(fake(), ok_strides, P(None), sw, sw, sw, sw,
                                                                  *[fake() for _ in range(12)], os, N, H, Ls, E, E, flags,
                                                                  P(None))
    assert layer_f(P(None), 64) == -1                          # the shift form needs the shared weights
    assert layer_f(P(None), 128) == -1                         # so does a fresh start
    assert layer_f(fake(), 128, (ctypes.c_int64 * 3)(H * E, E // 2, N * H * E)) == -3   # SRWM_ESTRIDE: rows of out overlap
    layer_b = lambda gxs: L.srwm_layer_backward_f32(
        fake(), ok_strides, *[fake() for _ in range(7)], fake(), ok_strides, *[fake() for _ in range(9)], gxs,
        *[fake() for _ in range(8)], N, H, Ls, E, E, 3, P(None))
    assert layer_b(None) == -1                                 # grad-state mode 3 does not exist (dense grad_x accepted)
    assert layer_b((ctypes.c_int64 * 3)(0, E, N * H * E)) == -1   # the flags are checked before the strides
    noalloc = lambda n, flags, gs: L.srwm_layer_backward_noalloc_f32(
        fake(), ok_strides, *[fake() for _ in range(7)], fake(), ok_strides, *[fake() for _ in range(9)], None,
        gs, gs, gs, gs, n, H, Ls, E, E, flags, P(None))
    assert noalloc(N, 0, P(None)) == -1                        # the batch sums are what it is for
    assert noalloc(N, 1, fake()) == -1                         # no buffer for an incoming state gradient
    assert noalloc(1 << 16, 0, fake()) == -5                   # SRWM_ESCRATCH: 2^16 x 8 rows of 16 x 52 floats > 32 MiB
    readout = lambda sw, gs, flags, gxs=None: L.srwm_layer_readout_grad_f32(
        fake(), ok_strides, fake(), fake(), fake(), P(None), sw, fake(), ok_strides, fake(), fake(), gxs, fake(), gs,
        N, H, Ls, E, E, flags, P(None))
    assert readout(P(None), fake(), 64) == -1                  # the shared W_y is always needed
    assert readout(fake(), P(None), 0) == -1                   # its gradient is what the call is for
    assert readout(fake(), fake(), 128) == -1                  # a fresh start has no entry state to replay from
    assert readout(fake(), fake(), 0, (ctypes.c_int64 * 3)(H * E, E // 2, N * H * E)) == -3   # SRWM_ESTRIDE: rows of grad_x overlap
    dsteps = lambda gq, flags: L.delta_steps_backward_f32(
        *[a for _ in range(4) for a in (fake(), ok_strides)], P(None), fake(), fake(), fake(), ok_strides, fake(),
        gq, fake(), fake(), fake(), N, H, Ls, E, E, flags, P(None))
    assert dsteps(P(None), 0) == -1                            # every gradient buffer is required
    assert dsteps(fake(), 32) == -1                            # there is no chunkwise form of the step mode
    prologue = lambda rows, flags, e: L.delta_layer_prologue_f32(rows, *[fake() for _ in range(5)], N, H, Ls, e, e, flags, P(None))
    assert prologue(P(None), 0, E) == -1                       # every buffer is required
    assert prologue(fake(), 32, E) == -1                       # the only flag it knows is the 1e-5 of the RL tree's normalisation
    assert prologue(fake(), 2048, 0) == -1                     # empty rows
    pgrad = lambda st, flags: L.delta_layer_prologue_grad_bf16(*[a for _ in range(4) for a in (fake(), st)],
                                                               *[fake() for _ in range(5)], N, H, Ls, E, E, flags, P(None))
    assert pgrad(None, 0) == -1                                # gradients come with their strides
    assert pgrad(ok_strides, 2048) == -1                       # the backward takes no flag
    assert pgrad(huge, 0) == -3                                # SRWM_ESTRIDE
    assert L.srwm_hip_scratch_bytes() == 32 << 20
    assert b"scratch" in L.srwm_hip_strerror(-5)


def test_layout_helpers_of_the_host_layer():
    """The helpers that decide memory layouts, on CPU tensors: output rows follow the row order of a step-major
    input view (so that the layers' reshape back is a view) and stay dense otherwise; the keep flags of the step
    mode are the transposed, converted notdone mask."""
    import layer
    import self_ref_v0
    L, N, H, E, Y = 5, 3, 2, 4, 13
    h = torch.randn(L, N, H * E)
    x = h.reshape(L, N, H, E).permute(1, 2, 0, 3)                      # what the layers hand to the operator
    out = self_ref_v0._rows_like(x, Y, torch.float32)
    assert out.shape == (N, H, L, Y) and out.stride() == (H * Y, Y, N * H * Y, 1)
    chain = out.transpose(1, 2).reshape(N, L, H * Y).transpose(0, 1)  # supervised_learning/layer.py:184-186
    assert chain.is_contiguous() and chain.data_ptr() == out.data_ptr()
    assert self_ref_v0._rows_like(x.contiguous(), Y, torch.float32).is_contiguous()
    assert self_ref_v0._rows_like(x[:, :, :1], Y, torch.float32).is_contiguous()          # one step: nothing to reorder
    assert self_ref_v0._rows_like(x[..., ::2], Y, torch.bfloat16).is_contiguous()         # rows not contiguous: dense
    notdone = torch.rand(L, N) > 0.3
    keep = layer._keep_rows(notdone, torch.float32)
    assert keep.shape == (N, L) and keep.is_contiguous() and keep.dtype == torch.float32
    assert torch.equal(keep, notdone.t().float())
