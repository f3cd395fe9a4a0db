"""srwm_layer_backward_noalloc_f32, the entry point that allocates nothing: its per-row state
gradients live in a static device array inside the library.  It must return exactly what
srwm_layer_backward_f32 returns (same kernels, same summation order), on calls in a row that
share the array, the second smaller than the first."""
import math

import pytest
import torch

import srwm_hip

pytestmark = pytest.mark.gpu


def _case(N, H, L, E, Y, seed, shift, generic=False, poison=False, check_memory=False):
    """Layer forward on the GPU, then the backward through both entry points.  poison: the upstream gradient of the
    no-alloc call is NaN, so every per-row gradient it leaves in the static array is NaN (nothing is compared).
    check_memory: the no-alloc call must leave the device's free memory and torch's allocator as they were."""
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(seed)
    std = 1.0 / math.sqrt(E)
    x = torch.randn(N, H, L, E, generator=g).to(dev)
    slow = [(torch.randn(H, E, w, generator=g) * std).to(dev) for w in (Y, E, E, 4)]
    go = torch.randn(N, H, L, Y, generator=g).to(dev)
    f32 = dict(device=dev, dtype=torch.float32)
    if shift:
        state = [(torch.randn(N, H, E, w, generator=g) * 0.1).to(dev) for w in (Y, E, E, 4)]
    else:
        state = [torch.empty(N, H, E, w, **f32) for w in (Y, E, E, 4)]
    saved = [torch.empty(N, H, L, w, **f32) for w in (E, E, 4, Y, E, E, 4)]
    out = torch.empty(N, H, L, Y, **f32)
    base = srwm_hip.FLAG_STATE_SHIFT | srwm_hip.FLAG_SOFTMAX_INPUT | (srwm_hip.FLAG_GENERIC if generic else 0)
    srwm_hip.self_ref_layer_forward(x, None, slow, *state, *saved, out,
                                    flags=base | (0 if shift else srwm_hip.FLAG_FRESH_STATE))
    # existing entry point: per-row gradients in caller-provided tensors
    gx_ref = torch.empty(N, H, L, E, **f32)
    gW = [torch.empty(N, H, E, w, **f32) for w in (Y, E, E, 4)]
    gs_ref = [torch.empty(H, E, w, **f32) for w in (Y, E, E, 4)]
    srwm_hip.self_ref_layer_backward(x, *saved, go, slow, *state, gx_ref, gW, gs_ref,
                                     flags=base | srwm_hip.GRAD_STATE_ZERO)
    # the entry point under test: poisoned outputs, so that a skipped write shows
    gx = torch.full((N, H, L, E), float("nan"), **f32)
    gs = [torch.full((H, E, w), float("nan"), **f32) for w in (Y, E, E, 4)]
    if poison:
        go = torch.full_like(go, float("nan"))
    torch.cuda.synchronize()
    before = (torch.cuda.mem_get_info(dev)[0], torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev))
    srwm_hip.self_ref_layer_backward_noalloc(x, *saved, go, slow, *state, gx, gs, flags=base)
    torch.cuda.synchronize()
    after = (torch.cuda.mem_get_info(dev)[0], torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev))
    if check_memory:
        assert after == before, (before, after)
    if poison:
        assert bool(torch.isnan(gs[0]).all())
        return
    assert torch.isfinite(gx_ref).all() and all(torch.isfinite(t).all() for t in gs_ref)
    assert torch.equal(gx, gx_ref)
    for a, b, per_row in zip(gs, gs_ref, gW):
        assert torch.equal(a, b)
        # and the batch sums are sums of THIS call's rows, not of what an earlier call left in the array
        assert torch.allclose(a, per_row.sum(0), rtol=1e-5, atol=1e-6 * float(per_row.abs().max()) * N)


def test_noalloc_backward_equals_the_allocating_one_on_calls_in_a_row():
    print("case no-alloc layer backward: large, then smaller, then wide, then LDS-resident kernels", flush=True)
    _case(8, 8, 40, 32, 32, seed=1, shift=False)
    _case(8, 8, 40, 32, 32, seed=1, shift=False, check_memory=True)   # kernels loaded by now: nothing may be allocated
    _case(8, 8, 40, 32, 32, seed=7, shift=False, poison=True)         # leaves NaN in every word the next calls reuse
    _case(3, 4, 17, 32, 32, seed=2, shift=True, check_memory=True)    # smaller input right after: the array still holds the NaNs
    _case(2, 16, 33, 64, 64, seed=3, shift=False)      # headline head size
    _case(3, 4, 12, 32, 97, seed=4, shift=True)        # wide output block
    _case(2, 3, 9, 12, 12, seed=5, shift=False, generic=True)
    _case(1, 1, 5, 8, 8, seed=6, shift=False)          # smallest


def test_noalloc_wrapper_copies_nothing():
    """The Python wrapper refuses tensors it would have to copy (a copy allocates), the shared weights included."""
    print("case no-alloc layer backward: non-contiguous shared weights", flush=True)
    dev = torch.device("cuda:0")
    N, H, L, E = 2, 2, 3, 8
    z = lambda *s: torch.zeros(*s, device=dev)
    saved = [z(N, H, L, w) for w in (E, E, 4, E, E, E, 4)]
    state = [z(N, H, E, w) for w in (E, E, E, 4)]
    slow = [z(H, E, w) for w in (E, E, E, 4)]
    slow[1] = z(H, E, 2 * E)[:, :, ::2]
    gs = [z(H, E, w) for w in (E, E, E, 4)]
    with pytest.raises(ValueError, match="copies nothing"):
        srwm_hip.self_ref_layer_backward_noalloc(z(N, H, L, E), *saved, z(N, H, L, E), slow, *state, z(N, H, L, E), gs)


def test_noalloc_backward_refuses_what_does_not_fit():
    print("case no-alloc layer backward: size limit", flush=True)
    dev = torch.device("cuda:0")
    N, H, L, E = 1024, 16, 1, 64          # 1024 * 16 * 64 * 196 floats = 784 MiB of per-row gradients
    assert N * H * E * (3 * E + 4) * 4 > srwm_hip.scratch_bytes()
    z = lambda *s: torch.zeros(*s, device=dev)
    saved = [z(N, H, L, w) for w in (E, E, 4, E, E, E, 4)]
    state = [z(N, H, E, w) for w in (E, E, E, 4)]
    slow = [z(H, E, w) for w in (E, E, E, 4)]
    gs = [torch.full((H, E, w), 7.0, device=dev) for w in (E, E, E, 4)]
    with pytest.raises(RuntimeError, match="-5"):
        srwm_hip.self_ref_layer_backward_noalloc(z(N, H, L, E), *saved, z(N, H, L, E), slow, *state,
                                                 z(N, H, L, E), gs)
    torch.cuda.synchronize()
    assert all(bool((t == 7.0).all()) for t in gs)     # nothing was launched
