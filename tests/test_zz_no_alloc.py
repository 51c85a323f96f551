"""bdh_state_step_noalloc (the decode step for callers that cannot allocate device memory) against
bdh_state_step, through the C ABI.

Both entry points launch the same kernels, so the bar is bit equality of every output (readout, updated
state, active bitmask, touched-row counts); the oracle is checked on the first call as well (f32 state:
1e-3 relative, observed far tighter).  Two calls in a row on the same device, the second on a smaller
input: the fixed scratch array keeps the first call's partials, and the second call must not read them.
A shape whose partials exceed the array is rejected with a clear error.
"""
import numpy as np
import pytest
import torch

from oracle import bdh_oracle as orc

pytestmark = pytest.mark.gpu


def _inputs(seed, B, h, N, d, density, Nq):
    from scipy.stats import norm

    rng = np.random.default_rng(seed)
    x = np.maximum(rng.standard_normal((B, h, N)) + norm.ppf(density), 0).astype(np.float32)
    v = rng.standard_normal((B, d)).astype(np.float32)
    rho = (0.01 * rng.standard_normal((B, h, Nq, d))).astype(np.float32)
    return x, v, rho


def _call(ffi, ctx, fn, x, v, rho, freqs, position, rotary, dtype, check_no_allocation=False):
    dev = "cuda:0"
    B, h, N = x.shape
    d = v.shape[1]
    xt, vt, ft = (torch.from_numpy(a).to(dev) for a in (x, v, freqs))
    rt = torch.from_numpy(rho).to(dev).to(dtype).contiguous()
    out = torch.empty((B, h, d), dtype=torch.float32, device=dev)
    bm = torch.zeros((B, h, (N + 63) // 64), dtype=torch.int64, device=dev)
    rows = torch.zeros((B, h), dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    ctx.set_stream(torch.cuda.current_stream(0).cuda_stream)
    print(f"{fn.__name__} B={B} h={h} N={N} d={d} rotary={rotary} dtype={dtype}", flush=True)
    free_before = torch.cuda.mem_get_info(0)[0]  # every tensor of the call exists already
    ctx.check(fn(ctx.handle, B, h, N, d, rotary, ffi.ptr(xt), ffi.ptr(vt), ffi.ptr(ft), position, None, None,
                 ffi.ptr(rt), ffi.F32 if dtype == torch.float32 else ffi.BF16, ffi.ptr(out), ffi.ptr(bm), ffi.ptr(rows)))
    torch.cuda.synchronize()
    if check_no_allocation:  # the driver's count of free device memory has not moved: no hipMalloc, no workspace growth
        assert torch.cuda.mem_get_info(0)[0] == free_before
    return out.cpu().numpy(), rt.float().cpu().numpy(), bm.cpu().numpy(), rows.cpu().numpy()


@pytest.mark.parametrize("rotary,dtype", [(orc.ROPE, torch.float32), (orc.ROPE, torch.bfloat16),
                                          (orc.ALIBI, torch.float32), (orc.POPE, torch.float32)])
def test_noalloc_step_equals_the_allocating_step_twice_in_a_row(corc, rotary, dtype):
    if not torch.cuda.is_available():
        pytest.fail("no HIP device: the GPU tests must run on the MI355X box")
    from burn_dragon_amd import ffi

    lib = ffi.load_library()
    ctx = ffi.Context(0)  # a fresh context: its workspace is empty, and the new entry point never grows it
    ctx_ref = ffi.Context(0)  # the allocating entry point runs on a context of its own
    try:
        # first call large (many workgroups per slice), second call smaller in every dimension
        for seed, (B, h, N, d, density) in enumerate([(4, 4, 4096, 256, 0.05), (2, 2, 640, 256, 0.3)]):
            x, v, rho = _inputs(40 + seed, B, h, N, d, density, 2 * N if rotary == orc.POPE else N)
            freqs = corc.build_freqs(N, rotary=rotary) if rotary != orc.ALIBI else np.zeros(N, np.float32)
            position = 777 + seed
            got = _call(ffi, ctx, lib.bdh_state_step_noalloc, x, v, rho, freqs, position, rotary, dtype,
                        check_no_allocation=True)
            ref = _call(ffi, ctx_ref, lib.bdh_state_step, x, v, rho, freqs, position, rotary, dtype)
            for a, b, name in zip(got, ref, ("out", "rho", "bitmask", "rows_touched")):
                assert np.array_equal(a, b), (name, seed)
            if dtype == torch.float32:
                q = corc.rotate(x[:, :, None, :], freqs, rotary, position)
                decay = corc.alibi_decay(corc.default_alibi_slopes(h)) if rotary == orc.ALIBI else None
                out_ref, rho_ref = corc.recurrent_attention(q, v[:, None, :], rho, decay=decay)
                assert np.abs(got[0] - out_ref[:, :, 0]).max() <= 1e-3 * np.abs(out_ref).max()
                assert np.abs(got[1] - rho_ref).max() <= 1e-3 * np.abs(rho_ref).max()
    finally:
        ctx.close()
        ctx_ref.close()


def test_noalloc_step_rejects_a_shape_beyond_its_scratch():
    if not torch.cuda.is_available():
        pytest.fail("no HIP device: the GPU tests must run on the MI355X box")
    from burn_dragon_amd import ffi

    lib = ffi.load_library()
    ctx = ffi.Context(0)
    try:
        # B*h = 4096 slices of N = 16384 at d = 512 would need 256 MiB of partials; the pointers are never
        # dereferenced because the size check comes before any launch
        B, h, N, d = 512, 8, 16384, 512
        dummy = torch.zeros(1024, dtype=torch.float32, device="cuda:0")
        rc = lib.bdh_state_step_noalloc(ctx.handle, B, h, N, d, ffi.ROPE, ffi.ptr(dummy), ffi.ptr(dummy), ffi.ptr(dummy),
                                        0, None, None, ffi.ptr(dummy), ffi.F32, ffi.ptr(dummy), None, None)
        assert rc == ffi.E_SHAPE
        assert b"scratch" in lib.bdh_last_error(ctx.handle)
    finally:
        ctx.close()
