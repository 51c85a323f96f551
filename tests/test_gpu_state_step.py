"""GPU parity of the recurrent state step (bdh_state_step / bdh_recurrent_attention) against the
CPU oracle, through the C ABI.

Tolerances: BASELINE north_star asks 1e-3 relative for an f32 state and 2e-2 for a bf16 state;
the f32 checks here are much tighter (the only differences are the device sincos, <= 2 ulp, and
the summation order of the readout).  Index artefacts (active bitmask, touched-row counts) are
bit-exact.  Untouched state rows must be bit-identical.
"""
import numpy as np
import pytest
import torch

from oracle import bdh_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.fail("no HIP device: the GPU tests must run on the MI355X box")
    from burn_dragon_amd import ffi
    from burn_dragon_amd.recurrent import recurrent_attention

    return ffi, recurrent_attention


def make_inputs(seed, B, h, T, N, d, density, rho_scale=0.01):
    rng = np.random.default_rng(seed)
    if density >= 1.0:
        x = (np.abs(rng.standard_normal((B, h, T, N))) + 0.1).astype(np.float32)
    elif density <= 0.0:
        x = np.zeros((B, h, T, N), np.float32)
    else:
        from scipy.stats import norm

        mu = norm.ppf(density)
        x = np.maximum(rng.standard_normal((B, h, T, N)) + mu, 0).astype(np.float32)
    v = rng.standard_normal((B, T, d)).astype(np.float32)
    rho = (rho_scale * rng.standard_normal((B, h, N, d))).astype(np.float32)
    return x, v, rho


def rel_err(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def run_gpu(recurrent_attention, x, v, rho, freqs, position, rotary, slopes=None, positions=None, dtype=torch.float32):
    dev = "cuda:0"
    xt, vt = torch.from_numpy(x).to(dev), torch.from_numpy(v).to(dev)
    rt = torch.from_numpy(rho).to(dev).to(dtype).contiguous()
    ft = torch.from_numpy(freqs).to(dev)
    pt = None if positions is None else torch.from_numpy(np.asarray(positions, np.int32)).to(dev)
    from burn_dragon_amd.positional import RotaryEmbedding

    out, bm, rows = recurrent_attention(xt, vt, rt, ft, position, RotaryEmbedding(rotary), slopes, pt,
                                        want_bitmask=True, want_rows=True)
    torch.cuda.synchronize()
    return out.cpu().numpy(), rt.float().cpu().numpy(), bm.cpu().numpy().view(np.uint64), rows.cpu().numpy()


@pytest.fixture(params=[0, 1], ids=["pairs256", "pairs64"])
def split(request, gpu):
    """Runs a test under both workgroup shapes of the wave-per-pair kernels."""
    ffi, _ = gpu
    ctx = ffi.default_context(0)
    ctx.set_option("state_step.split", request.param)
    yield request.param
    ctx.set_option("state_step.split", -1)


@pytest.mark.parametrize("d", [256, 512])
@pytest.mark.parametrize("N,density", [(512, 0.05), (640, 0.5), (130, 1.0), (1024, 0.0), (2048, 0.02)])
def test_fast_path_decode_step_matches_oracle(gpu, corc, split, N, d, density):
    _, recurrent_attention = gpu
    B, h, T = 3, 2, 1
    x, v, rho = make_inputs(100 + N + d, B, h, T, N, d, density)
    freqs = corc.build_freqs(N)
    position = 1234
    q = corc.rotate(x, freqs, orc.ROPE, position)
    out_ref, rho_ref = corc.recurrent_attention(q, v, rho)
    out, rho_new, bm, rows = run_gpu(recurrent_attention, x, v, rho, freqs, position, orc.ROPE)
    assert rel_err(out, out_ref) < 2e-5
    assert rel_err(rho_new, rho_ref) < 1e-6
    # bit-exact index artefacts
    assert np.array_equal(bm[:, :, 0], orc.active_bitmask(np.pad(x[:, :, 0], ((0, 0), (0, 0), (0, (-N) % 64)))))
    assert np.array_equal(rows[:, :, 0], orc.pair_closed_rows(x[:, :, 0]))
    # rows of inactive pairs are bit-identical to the input state
    inactive = ~np.repeat((x[:, :, 0] != 0).reshape(B, h, N // 2, 2).any(-1), 2, axis=-1)
    assert np.array_equal(rho_new[inactive], rho[inactive])


def test_update_is_bit_exact_when_rotation_is_exact(gpu, corc, split):
    """At position 0 cos = 1 and sin = 0 exactly, so q == x on both sides and the rank-1 update
    rho + (q*v) (product rounded, then added: src/model/bdh.rs:298) must agree bit for bit."""
    _, recurrent_attention = gpu
    B, h, N, d = 2, 2, 512, 256
    x, v, rho = make_inputs(7, B, h, 1, N, d, 0.3)
    freqs = corc.build_freqs(N)
    _, rho_ref = corc.recurrent_attention(corc.rotate(x, freqs, orc.ROPE, 0), v, rho)
    _, rho_new, _, _ = run_gpu(recurrent_attention, x, v, rho, freqs, 0, orc.ROPE)
    assert np.array_equal(rho_new, rho_ref)


def test_first_token_reads_zero_state_and_writes_outer_product(gpu, corc):
    _, recurrent_attention = gpu
    B, h, N, d = 2, 2, 256, 256
    x, v, _ = make_inputs(8, B, h, 1, N, d, 0.2)
    freqs = corc.build_freqs(N)
    out, rho_new, _, _ = run_gpu(recurrent_attention, x, v, np.zeros((B, h, N, d), np.float32), freqs, 0, orc.ROPE)
    assert not out.any()
    assert np.array_equal(rho_new, x[:, :, 0, :, None] * v[:, None, 0, None, :])


@pytest.mark.parametrize("rotary", [orc.ROPE, orc.ALIBI, orc.POPE])
def test_generic_path_small_shapes_all_rotaries(gpu, corc, rotary):
    """tests/model_paths.rs shapes (N=32, d=16): the generic kernel, T > 1, all three rotaries."""
    _, recurrent_attention = gpu
    B, h, T, N, d = 2, 2, 5, 32, 16
    x, v, rho = make_inputs(20 + rotary, B, h, T, N, d, 0.4)
    freqs = corc.build_freqs(N, 65536.0, rotary)
    slopes = np.array([0.5, 0.125], np.float32) if rotary == orc.ALIBI else None
    decay = None if slopes is None else corc.alibi_decay(slopes)
    Nq = 2 * N if rotary == orc.POPE else N
    rho = (0.01 * np.random.default_rng(1).standard_normal((B, h, Nq, d))).astype(np.float32)
    q = corc.rotate(x, freqs, rotary, 17)
    out_ref, rho_ref = corc.recurrent_attention(q, v, rho, decay)
    out, rho_new, bm, rows = run_gpu(recurrent_attention, x, v, rho, freqs, 17, rotary, slopes)
    assert rel_err(out, out_ref) < 2e-5
    assert rel_err(rho_new, rho_ref) < 2e-6
    assert np.array_equal(bm, orc.active_bitmask(np.pad(x, ((0, 0), (0, 0), (0, 0), (0, 32)))))
    expect_rows = orc.pair_closed_rows(x) if rotary == orc.ROPE else np.full((B, h, T), Nq)
    assert np.array_equal(rows, expect_rows)


def test_prefill_loop_equals_sequential_steps_and_causal_closed_form(gpu, corc, split):
    _, recurrent_attention = gpu
    B, h, T, N, d = 2, 2, 6, 256, 256
    x, v, _ = make_inputs(31, B, h, T, N, d, 0.1)
    rho0 = np.zeros((B, h, N, d), np.float32)
    freqs = corc.build_freqs(N)
    out, rho_new, _, _ = run_gpu(recurrent_attention, x, v, rho0, freqs, 40, orc.ROPE)
    q = corc.rotate(x, freqs, orc.ROPE, 40)
    out_ref, rho_ref = corc.recurrent_attention(q, v, rho0, sparse=True)
    assert rel_err(out, out_ref) < 2e-5 and rel_err(rho_new, rho_ref) < 1e-6
    # closed forms in float64: out = tril(-1)(QQ^T)V, final state = Q^T V
    q64, v64 = q.astype(np.float64), v.astype(np.float64)
    assert rel_err(out, orc.causal_unnormalised(q64, v64)) < 1e-5
    assert rel_err(rho_new, np.einsum("bhtn,btd->bhnd", q64, v64)) < 1e-5
    # chunk consistency on the device: [0,2) then [2,6) == one call
    dev = "cuda:0"
    from burn_dragon_amd.positional import RotaryEmbedding

    rt = torch.zeros((B, h, N, d), device=dev)
    xt, vt, ft = torch.from_numpy(x).to(dev), torch.from_numpy(v).to(dev), torch.from_numpy(freqs).to(dev)
    o1 = recurrent_attention(xt[:, :, :2].contiguous(), vt[:, :2].contiguous(), rt, ft, 40, RotaryEmbedding.ROPE)
    o2 = recurrent_attention(xt[:, :, 2:].contiguous(), vt[:, 2:].contiguous(), rt, ft, 42, RotaryEmbedding.ROPE)
    torch.cuda.synchronize()
    assert np.array_equal(torch.cat([o1, o2], 2).cpu().numpy(), out)
    assert np.array_equal(rt.cpu().numpy(), rho_new)


def test_per_sequence_positions(gpu, corc):
    _, recurrent_attention = gpu
    B, h, N, d = 3, 2, 256, 256
    x, v, rho = make_inputs(41, B, h, 1, N, d, 0.2)
    freqs = corc.build_freqs(N)
    positions = [5, 900, 4095]
    out, rho_new, _, _ = run_gpu(recurrent_attention, x, v, rho, freqs, 0, orc.ROPE, positions=positions)
    for b, p in enumerate(positions):
        q = corc.rotate(x[b : b + 1], freqs, orc.ROPE, p)
        o_ref, r_ref = corc.recurrent_attention(q, v[b : b + 1], rho[b : b + 1])
        assert rel_err(out[b : b + 1], o_ref) < 2e-5 and rel_err(rho_new[b : b + 1], r_ref) < 1e-6


@pytest.mark.parametrize("N,d", [(256, 256), (384, 512), (32, 16)])
def test_bf16_state_within_tolerance(gpu, corc, split, N, d):
    """bf16 storage, f32 accumulate: 2e-2 relative (north_star).  d=256/512 take the wave-per-pair
    kernel, d=16 the generic one."""
    _, recurrent_attention = gpu
    B, h, T = 2, 2, 4
    x, v, rho = make_inputs(51 + d, B, h, T, N, d, 0.2, rho_scale=0.05)
    rho_b = torch.from_numpy(rho).to(torch.bfloat16).float().numpy()  # the state both sides start from
    freqs = corc.build_freqs(N)
    out, rho_new, bm, rows = run_gpu(recurrent_attention, x, v, rho_b, freqs, 9, orc.ROPE, dtype=torch.bfloat16)
    out_ref, rho_ref = corc.recurrent_attention(corc.rotate(x, freqs, orc.ROPE, 9), v, rho_b)
    assert rel_err(out, out_ref) < 2e-2 and rel_err(rho_new, rho_ref) < 2e-2
    assert np.array_equal(rows, orc.pair_closed_rows(x))
    assert np.array_equal(bm, orc.active_bitmask(np.pad(x, ((0, 0), (0, 0), (0, 0), (0, (-N) % 64)))))
    # one step from an exactly representable state: the only error is the final rounding to bf16
    x1, v1 = x[:, :, :1], v[:, :1]
    _, rho_1, _, _ = run_gpu(recurrent_attention, x1, v1, rho_b, freqs, 0, orc.ROPE, dtype=torch.bfloat16)
    _, rho_1_ref = corc.recurrent_attention(corc.rotate(x1, freqs, orc.ROPE, 0), v1, rho_b)
    assert np.array_equal(rho_1, torch.from_numpy(rho_1_ref).to(torch.bfloat16).float().numpy())


def test_deterministic_across_runs(gpu, corc):
    _, recurrent_attention = gpu
    B, h, N, d = 4, 4, 2048, 256
    x, v, rho = make_inputs(61, B, h, 1, N, d, 0.05)
    freqs = corc.build_freqs(N)
    a = run_gpu(recurrent_attention, x, v, rho, freqs, 77, orc.ROPE)
    b = run_gpu(recurrent_attention, x, v, rho, freqs, 77, orc.ROPE)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_argument_errors_do_not_abort(gpu):
    ffi, _ = gpu
    ctx = ffi.default_context(0)
    lib = ctx.lib
    t = torch.zeros(1024, device="cuda:0")
    p = t.data_ptr()
    # odd latent with RoPE (src/model/attention.rs:310 would fail the reshape)
    assert lib.bdh_state_step(ctx.handle, 1, 1, 3, 4, ffi.ROPE, p, p, p, 0, None, None, p, ffi.F32, p, None, None) == ffi.E_SHAPE
    assert b"even" in lib.bdh_last_error(ctx.handle)
    assert lib.bdh_state_step(ctx.handle, 1, 1, 4, 4, 9, p, p, p, 0, None, None, p, ffi.F32, p, None, None) == ffi.E_INVAL
    assert lib.bdh_state_step(ctx.handle, 1, 1, 4, 4, ffi.ROPE, p, p, p, -1, None, None, p, ffi.F32, p, None, None) == ffi.E_INVAL
    assert lib.bdh_state_step(ctx.handle, 1, 1, 4, 4, ffi.ROPE, None, p, p, 0, None, None, p, ffi.F32, p, None, None) == ffi.E_INVAL
    assert lib.bdh_state_step(ctx.handle, 1, 1, 4, 4, ffi.ROPE, p, p, p, 0, None, None, p + 4, ffi.F32, p, None, None) == ffi.E_ALIGN
    # empty batch is a no-op
    assert lib.bdh_state_step(ctx.handle, 0, 4, 8, 4, ffi.ROPE, None, None, None, 0, None, None, None, ffi.F32, None, None, None) == ffi.OK


def test_full_size_config2_properties(gpu, corc):
    """BASELINE config 2 at its real shape: rho f32 [32,4,8192,256] (1 GiB), 5 % density.
    Checked (a) against the oracle on one batch entry, (b) everywhere against an f32 torch
    statement of the same step, (c) by the invariant that inactive rows keep their bits."""
    _, recurrent_attention = gpu
    from burn_dragon_amd.positional import RotaryEmbedding

    B, h, N, d = 32, 4, 8192, 256
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(5)
    rho = 0.01 * torch.randn((B, h, N, d), device=dev, generator=g)
    x = torch.relu(torch.randn((B, h, 1, N), device=dev, generator=g) - 1.6449)
    v = torch.randn((B, 1, d), device=dev, generator=g)
    freqs_np = corc.build_freqs(N)
    freqs = torch.from_numpy(freqs_np).to(dev)
    position = 3071
    rho_before = rho.clone()
    out, bm, rows = recurrent_attention(x, v, rho, freqs, position, RotaryEmbedding.ROPE, want_bitmask=True, want_rows=True)
    torch.cuda.synchronize()
    x_np = x.cpu().numpy()
    # (a) oracle on batch entry 0 (dense faithful form)
    q_np = corc.rotate(x_np, freqs_np, orc.ROPE, position)
    o_ref, r_ref = corc.recurrent_attention(q_np[:1], v[:1].cpu().numpy(), rho_before[:1].cpu().numpy())
    assert rel_err(out[:1].cpu().numpy(), o_ref) < 2e-5
    assert rel_err(rho[:1].cpu().numpy(), r_ref) < 1e-6
    # (b) torch f32 statement on every element, q taken from the oracle's rotate
    q = torch.from_numpy(q_np).to(dev)[:, :, 0]
    out_t = torch.einsum("bhnd,bhn->bhd", rho_before, q)
    assert rel_err(out[:, :, 0].cpu().numpy(), out_t.cpu().numpy()) < 5e-5
    rho_t = rho_before + q[..., None] * v[:, None, 0, None, :]
    assert float((rho - rho_t).abs().max()) < 1e-6
    # (c) index artefacts and untouched rows
    assert np.array_equal(bm.cpu().numpy().view(np.uint64)[:, :, 0], orc.active_bitmask(x_np[:, :, 0]))
    assert np.array_equal(rows.cpu().numpy()[:, :, 0], orc.pair_closed_rows(x_np[:, :, 0]))
    active_rows = torch.from_numpy(np.repeat((x_np[:, :, 0] != 0).reshape(B, h, N // 2, 2).any(-1), 2, axis=-1)).to(dev)
    assert torch.equal(rho[~active_rows], rho_before[~active_rows])
    frac = float(active_rows.float().mean())
    assert 0.09 < frac < 0.105  # 1 - 0.95^2 = 9.75 % of the rows


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.bfloat16, 2e-2)], ids=["f32", "bf16"])
@pytest.mark.parametrize("density", [0.01, 0.05, 0.20])
def test_config5_shapes_max_relative_error(gpu, corc, dtype, tol, density):
    """BASELINE config 5 (the config-4 layer shape h=8, N=16384, d=512) at B=1: the step of every
    density of the sweep, f32 and bf16 state, against the oracle started from the same (bf16-rounded,
    where it applies) state.  The printed errors are the max-rel-err column of the sweep table."""
    _, recurrent_attention = gpu
    B, h, N, d = 1, 8, 16384, 512
    x, v, rho = make_inputs(int(density * 100), B, h, 1, N, d, density)
    if dtype == torch.bfloat16:
        rho = torch.from_numpy(rho).to(torch.bfloat16).float().numpy()
    freqs = corc.build_freqs(N)
    out, rho_new, bm, rows = run_gpu(recurrent_attention, x, v, rho, freqs, 4000, orc.ROPE, dtype=dtype)
    out_ref, rho_ref = corc.recurrent_attention(corc.rotate(x, freqs, orc.ROPE, 4000), v, rho)
    e_out, e_rho = rel_err(out, out_ref), rel_err(rho_new, rho_ref)
    print(f"config-5 shape B=1 density {density:.0%} {dtype}: readout rel err {e_out:.2e}, state rel err {e_rho:.2e}")
    assert e_out < tol and e_rho < tol
    assert np.array_equal(rows, orc.pair_closed_rows(x))
    assert np.array_equal(bm, orc.active_bitmask(x))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.bfloat16, 2e-2)], ids=["f32", "bf16"])
@pytest.mark.parametrize("N,d,density", [(128, 128, 0.35), (1024, 256, 0.05), (200, 48, 0.5), (512, 512, 0.0),
                                         (651, 256, 0.3), (650, 256, 0.3), (1536, 512, 0.1)])
@pytest.mark.parametrize("byproducts", [True, False], ids=["bitmask+rows", "plain"])
def test_lazy_alibi_decay_matches_the_eager_reference_semantics(gpu, corc, dtype, tol, N, d, density, byproducts):
    """ALiBi state kept lazily decayed (only active rows touched, decay applied when a row is next
    used) against the oracle's eager `rho *= exp(-slope)` after every token (src/model/bdh.rs:299-301):
    every readout along the way, and the state after bdh_alibi_materialize."""
    _, recurrent_attention = gpu
    from burn_dragon_amd.recurrent import alibi_materialize, recurrent_attention_lazy_alibi

    B, h, T = 2, 4, 9
    x, v, rho0 = make_inputs(int(1000 * density) + d, B, h, T, N, d, density, rho_scale=0.05)
    if dtype == torch.bfloat16:
        rho0 = torch.from_numpy(rho0).to(torch.bfloat16).float().numpy()
    slopes = corc.default_alibi_slopes(h)
    clock0 = 37  # the state arrives up to date as of 37 tokens
    dev = "cuda:0"
    rho = torch.from_numpy(rho0).to(dev).to(dtype).contiguous()
    stamps = torch.full((B, h, N), clock0, device=dev, dtype=torch.int32)
    xt, vt = torch.from_numpy(x).to(dev), torch.from_numpy(v).to(dev)
    # first five tokens in one call, the rest one by one with per-sequence clocks on the device
    # (without by-products a kernel may walk the five tokens in one launch)
    if byproducts:
        out_a, bm, rows = recurrent_attention_lazy_alibi(xt[:, :, :5].contiguous(), vt[:, :5].contiguous(), rho, stamps,
                                                         clock0, None, None, want_bitmask=True, want_rows=True)
    else:
        out_a = recurrent_attention_lazy_alibi(xt[:, :, :5].contiguous(), vt[:, :5].contiguous(), rho, stamps, clock0,
                                               None, None)
    outs = [out_a]
    clocks = torch.full((B,), clock0 + 5, device=dev, dtype=torch.int32)
    for t in range(5, T):
        outs.append(recurrent_attention_lazy_alibi(xt[:, :, t:t + 1].contiguous(), vt[:, t:t + 1].contiguous(), rho,
                                                   stamps, 0, None, clocks))
        clocks += 1
    untouched = torch.from_numpy(~(x != 0).any(axis=2)).to(dev)  # rows no token activated
    assert torch.equal(rho[untouched].float(), torch.from_numpy(rho0).to(dev)[untouched])  # never read or written
    assert (stamps[untouched] == clock0).all()
    alibi_materialize(rho, stamps, clock0 + T)
    torch.cuda.synchronize()
    assert (stamps == clock0 + T).all()
    out = torch.cat(outs, 2).cpu().numpy()
    out_ref, rho_ref = corc.recurrent_attention(x, v, rho0, decay=corc.alibi_decay(slopes))
    assert rel_err(out, out_ref) < tol
    assert rel_err(rho.float().cpu().numpy(), rho_ref) < tol
    if byproducts:
        assert np.array_equal(rows.cpu().numpy(), (x[:, :, :5] != 0).sum(-1))
        assert np.array_equal(bm.cpu().numpy().view(np.uint64),
                              orc.active_bitmask(np.pad(x[:, :, :5], ((0, 0), (0, 0), (0, 0), (0, (-N) % 64)))))
    # the eager entry point on the same inputs gives the same values to rounding
    rho_e = torch.from_numpy(rho0).to(dev).to(dtype).contiguous()
    from burn_dragon_amd.positional import RotaryEmbedding

    out_e = recurrent_attention(xt, vt, rho_e, torch.zeros(N, device=dev), 0, RotaryEmbedding.ALIBI)
    assert rel_err(out, out_e.cpu().numpy()) < tol and rel_err(rho.float().cpu().numpy(), rho_e.float().cpu().numpy()) < tol


@pytest.fixture
def dense_chunks(gpu):
    """Forces the many-token dense form (f32 matrix cores) for the duration of a test."""
    ffi, _ = gpu
    ctx = ffi.default_context(0)
    ctx.set_option("state_step.dense_chunks", 1)
    yield ctx
    ctx.set_option("state_step.dense_chunks", -1)


def _run_plain(recurrent_attention, x, v, rho, freqs, position, rotary, positions=None):
    from burn_dragon_amd.positional import RotaryEmbedding

    dev = "cuda:0"
    rt = torch.from_numpy(rho).to(dev).contiguous()
    pt = None if positions is None else torch.from_numpy(np.asarray(positions, np.int32)).to(dev)
    out = recurrent_attention(torch.from_numpy(x).to(dev), torch.from_numpy(v).to(dev), rt,
                              torch.from_numpy(freqs).to(dev), position, RotaryEmbedding(rotary), None, pt)
    torch.cuda.synchronize()
    return out.cpu().numpy(), rt.cpu().numpy()


@pytest.mark.parametrize("rotary", [orc.ROPE, orc.POPE])
@pytest.mark.parametrize("B,h,T,N,d,density", [
    (2, 2, 130, 64, 32, 0.3),     # one chunk, partial tiles everywhere
    (1, 3, 600, 40, 20, 0.5),     # two chunks (512 + 88), d and N not multiples of the tile or of 8
    (2, 4, 257, 256, 256, 0.05),  # the headline row width, sparse activations
    (1, 1, 5, 34, 6, 1.0),        # tiny, d not a multiple of 4 (scalar loads)
])
def test_dense_chunk_form_matches_sequential_oracle(gpu, corc, dense_chunks, rotary, B, h, T, N, d, density):
    """out = tril(-1)(Q Q^T) V + Q rho0 and rho += Q^T V on the f32 matrix cores against the oracle's
    token-by-token loop (src/model/bdh.rs:286-303), from a non-zero state at a non-zero position."""
    _, recurrent_attention = gpu
    x, v, _ = make_inputs(7 * T + N + d, B, h, T, N, d, density)
    Nq = 2 * N if rotary == orc.POPE else N
    rho0 = (0.05 * np.random.default_rng(5).standard_normal((B, h, Nq, d))).astype(np.float32)
    freqs = corc.build_freqs(N, rotary=rotary)
    position = 37
    out, rho_new = _run_plain(recurrent_attention, x, v, rho0, freqs, position, rotary)
    out_ref, rho_ref = corc.recurrent_attention(corc.rotate(x, freqs, rotary, position), v, rho0.copy())
    assert out.shape == out_ref.shape
    assert rel_err(out, out_ref) < 2e-5, rel_err(out, out_ref)
    assert rel_err(rho_new, rho_ref) < 2e-5, rel_err(rho_new, rho_ref)


def test_dense_chunk_form_split_products_keep_f32_accuracy(gpu, corc, dense_chunks):
    """The big-tile products of the dense form run on the bf16 matrix instructions with every f32 operand
    split into three bf16 terms (six instructions per f32 one).  Against a float64 evaluation of the same
    sums from the same rotated activations, the error must stay at the level of f32 rounding: a dropped
    cross term (2^-16 of a product) would show up as several 1e-6 here.
    64 slices of 256 tokens: every product takes the 128 x 128 / 256 x 256 tiles."""
    _, recurrent_attention = gpu
    B, h, T, N, d = 8, 8, 256, 256, 256
    x, v, rho0 = make_inputs(4242, B, h, T, N, d, 0.5, rho_scale=0.05)
    rng = np.random.default_rng(17)
    x *= np.exp2(rng.integers(-6, 7, (1, h, 1, N))).astype(np.float32)   # operands of mixed magnitude
    v *= np.exp2(rng.integers(-6, 7, (1, 1, d))).astype(np.float32)
    freqs = corc.build_freqs(N)
    position = 11
    out, rho_new = _run_plain(recurrent_attention, x, v, rho0, freqs, position, orc.ROPE)
    q = corc.rotate(x, freqs, orc.ROPE, position).astype(np.float64)
    v64, r64 = v.astype(np.float64), rho0.astype(np.float64)
    scores = np.tril(np.einsum("bhtn,bhsn->bhts", q, q), -1)
    out_ref = np.einsum("bhts,bsd->bhtd", scores, v64) + np.einsum("bhtn,bhnd->bhtd", q, r64)
    rho_ref = r64 + np.einsum("bhtn,btd->bhnd", q, v64)

    def rms_err(a, b):
        return float(np.sqrt(np.mean((a.astype(np.float64) - b) ** 2)) / np.sqrt(np.mean(b ** 2)))

    # measured: 2.35e-7 and 2.42e-7 (the f32 matrix instructions: 2.74e-7 and 2.53e-7)
    assert rms_err(out, out_ref) < 6e-7, rms_err(out, out_ref)
    assert rms_err(rho_new, rho_ref) < 6e-7, rms_err(rho_new, rho_ref)
    assert rel_err(out, out_ref) < 2e-6 and rel_err(rho_new, rho_ref) < 2e-6


def test_dense_chunk_form_equals_step_kernels_and_handles_device_positions(gpu, corc):
    """The same call through the sparse step kernels and through the dense form; per-sequence device
    positions; T = 128 takes the dense form by default once the products have enough tiles to cover the
    chip (B*h = 96 slices here; with a handful of slices the multi-token f32 RoPE kernel is kept)."""
    ffi, recurrent_attention = gpu
    ctx = ffi.default_context(0)
    B, h, T, N, d = 24, 4, 128, 128, 256
    x, v, rho = make_inputs(99, B, h, T, N, d, 0.1, rho_scale=0.05)
    freqs = corc.build_freqs(N)
    positions = [int(p) for p in np.random.default_rng(1).integers(0, 4000, B)]
    try:
        ctx.set_option("state_step.dense_chunks", 0)
        out_s, rho_s = _run_plain(recurrent_attention, x, v, rho, freqs, 0, orc.ROPE, positions)
    finally:
        ctx.set_option("state_step.dense_chunks", -1)
    out_d, rho_d = _run_plain(recurrent_attention, x, v, rho, freqs, 0, orc.ROPE, positions)
    assert rel_err(out_d, out_s) < 2e-5 and rel_err(rho_d, rho_s) < 2e-5
    assert not np.array_equal(out_d, out_s)  # different summation order: the dense form did run
    # a handful of slices at the same shape: the default keeps the token loop (identical bits)
    try:
        ctx.set_option("state_step.dense_chunks", 0)
        out_few_loop, _ = _run_plain(recurrent_attention, x[:1], v[:1], rho[:1], freqs, 5, orc.ROPE)
    finally:
        ctx.set_option("state_step.dense_chunks", -1)
    out_few, _ = _run_plain(recurrent_attention, x[:1], v[:1], rho[:1], freqs, 5, orc.ROPE)
    assert np.array_equal(out_few, out_few_loop)
    for b, pos in list(enumerate(positions))[:3]:
        o_ref, r_ref = corc.recurrent_attention(corc.rotate(x[b : b + 1], freqs, orc.ROPE, pos), v[b : b + 1],
                                                rho[b : b + 1].copy())
        assert rel_err(out_d[b : b + 1], o_ref) < 2e-5 and rel_err(rho_d[b : b + 1], r_ref) < 2e-5


@pytest.mark.parametrize("B,h,T,N,d,density", [(2, 3, 130, 64, 32, 0.3), (1, 2, 600, 40, 20, 0.5), (2, 4, 200, 256, 256, 0.05)])
def test_dense_chunk_form_alibi_matches_sequential_oracle(gpu, corc, dense_chunks, B, h, T, N, d, density):
    """ALiBi in the many-token form: S[t,s] *= decay^(t-s), out_t gets decay^t (q_t . rho0), the state ends as
    decay^T rho0 + sum_s decay^(T-s) q_s (x) v_s — against the oracle's loop (src/model/bdh.rs:286-303).
    decay^k is exp(k log decay) here and k roundings of a product there: 1e-4 relative."""
    _, recurrent_attention = gpu
    from burn_dragon_amd.positional import RotaryEmbedding

    x, v, rho0 = make_inputs(3 * T + N, B, h, T, N, d, density, rho_scale=0.05)
    slopes = np.array([0.05 * (i + 1) for i in range(h)], np.float32)  # slow decay: old tokens still matter
    dev = "cuda:0"
    rt = torch.from_numpy(rho0).to(dev).contiguous()
    out = recurrent_attention(torch.from_numpy(x).to(dev), torch.from_numpy(v).to(dev), rt,
                              torch.zeros(N, device=dev), 11, RotaryEmbedding.ALIBI, slopes)
    torch.cuda.synchronize()
    out_ref, rho_ref = corc.recurrent_attention(x, v, rho0.copy(), corc.alibi_decay(slopes))
    assert rel_err(out.cpu().numpy(), out_ref) < 1e-4, rel_err(out.cpu().numpy(), out_ref)
    assert rel_err(rt.cpu().numpy(), rho_ref) < 1e-4, rel_err(rt.cpu().numpy(), rho_ref)


@pytest.mark.parametrize("rotary", [orc.ROPE, orc.POPE, orc.ALIBI])
def test_dense_chunk_form_big_tiles_on_ragged_shapes(gpu, corc, dense_chunks, rotary):
    """64 slices put every product on the 128 x 128 / 256 x 256 tiles (split-bf16 products); T, N and d are
    no multiples of a tile, of the 16-wide k stage or of 8, so every edge tile takes the checked loads, and a
    600-token call adds a second chunk with a carried state.  Against the oracle's token loop
    (src/model/bdh.rs:286-303)."""
    _, recurrent_attention = gpu
    from burn_dragon_amd.positional import RotaryEmbedding

    B, h, N, d = 8, 8, 138, 202
    for T in (200, 600):
        x, v, rho0 = make_inputs(77 + T, B, h, T, N, d, 0.3, rho_scale=0.05)
        Nq = 2 * N if rotary == orc.POPE else N
        rho0 = (0.05 * np.random.default_rng(9).standard_normal((B, h, Nq, d))).astype(np.float32)
        if rotary == orc.ALIBI:
            slopes = np.array([0.02 * (i + 1) for i in range(h)], np.float32)
            dev = "cuda:0"
            rt = torch.from_numpy(rho0).to(dev).contiguous()
            out = recurrent_attention(torch.from_numpy(x).to(dev), torch.from_numpy(v).to(dev), rt,
                                      torch.zeros(N, device=dev), 5, RotaryEmbedding.ALIBI, slopes)
            torch.cuda.synchronize()
            out, rho_new = out.cpu().numpy(), rt.cpu().numpy()
            out_ref, rho_ref = corc.recurrent_attention(x, v, rho0.copy(), corc.alibi_decay(slopes))
            tol = 1e-4
        else:
            freqs = corc.build_freqs(N, rotary=rotary)
            out, rho_new = _run_plain(recurrent_attention, x, v, rho0, freqs, 5, rotary)
            out_ref, rho_ref = corc.recurrent_attention(corc.rotate(x, freqs, rotary, 5), v, rho0.copy())
            tol = 2e-5
        assert rel_err(out, out_ref) < tol, (T, rel_err(out, out_ref))
        assert rel_err(rho_new, rho_ref) < tol, (T, rel_err(rho_new, rho_ref))


def test_dense_chunk_form_on_a_lazily_decayed_alibi_state(gpu, corc):
    """T = 150 on a state with pending decay: the call applies it, runs the dense form (default from T = 128)
    and leaves every stamp at clock + T; a following single-token lazy step continues correctly."""
    from burn_dragon_amd.recurrent import alibi_materialize, recurrent_attention_lazy_alibi

    rng = np.random.default_rng(12)
    B, h, T, N, d = 2, 2, 150, 128, 256
    x, v, rho0 = make_inputs(77, B, h, T + 1, N, d, 0.1, rho_scale=0.05)
    slopes = np.array([0.02, 0.3], np.float32)
    clock = 60
    stamps0 = rng.integers(0, clock + 1, (B, h, N)).astype(np.int32)
    dev = "cuda:0"
    rt, st = torch.from_numpy(rho0).to(dev).contiguous(), torch.from_numpy(stamps0).to(dev)
    xt, vt = torch.from_numpy(x).to(dev), torch.from_numpy(v).to(dev)
    out = recurrent_attention_lazy_alibi(xt[:, :, :T].contiguous(), vt[:, :T].contiguous(), rt, st, clock, slopes)
    out1 = recurrent_attention_lazy_alibi(xt[:, :, T:].contiguous(), vt[:, T:].contiguous(), rt, st, clock + T, slopes)
    alibi_materialize(rt, st, clock + T + 1, slopes)
    torch.cuda.synchronize()
    # oracle: the state the stamps stand for, then the eager loop over all T + 1 tokens
    decay = corc.alibi_decay(slopes).astype(np.float64)
    start = rho0.astype(np.float64) * (decay[None, :, None] ** (clock - stamps0))[..., None]
    out_ref, rho_ref = corc.recurrent_attention(x, v, start.astype(np.float32), corc.alibi_decay(slopes))
    assert rel_err(out.cpu().numpy(), out_ref[:, :, :T]) < 1e-4
    assert rel_err(out1.cpu().numpy(), out_ref[:, :, T:]) < 1e-4
    assert rel_err(rt.cpu().numpy(), rho_ref) < 1e-4
    assert (st.cpu().numpy() == clock + T + 1).all()


def test_dense_chunk_form_equals_token_loop_on_ragged_shapes(gpu, corc):
    """Sixteen seeded shapes with every dimension ragged (tile edges, odd d, a single token, more than one
    chunk), all three rotaries: the dense form and the token loop of the step kernels agree to f32
    reassociation on the device, and the first shapes also against the oracle."""
    ffi, recurrent_attention = gpu
    from burn_dragon_amd.positional import RotaryEmbedding

    ctx = ffi.default_context(0)
    rng = np.random.default_rng(2024)
    dev = "cuda:0"
    for case in range(16):
        B, h = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        T = int(rng.choice([1, 2, 17, 127, 128, 129, 255, 300, 513, 640]))
        N = 2 * int(rng.integers(1, 100))
        d = int(rng.choice([1, 3, 4, 8, 20, 33, 64, 70, 128, 132]))
        rotary = int(rng.integers(0, 3))
        density = float(rng.choice([0.0, 0.1, 0.5, 1.0]))
        x, v, _ = make_inputs(1000 + case, B, h, T, N, d, density)
        Nq = 2 * N if rotary == orc.POPE else N
        rho0 = (0.05 * rng.standard_normal((B, h, Nq, d))).astype(np.float32)
        freqs = corc.build_freqs(N, rotary=rotary)
        slopes = np.array([0.03 * (i + 1) for i in range(h)], np.float32) if rotary == orc.ALIBI else None
        position = int(rng.integers(0, 5000))
        label = f"case {case}: B={B} h={h} T={T} N={N} d={d} rotary={rotary} density={density}"
        print(label, flush=True)
        res = []
        for mode in (0, 1):
            ctx.set_option("state_step.dense_chunks", mode)
            try:
                rt = torch.from_numpy(rho0).to(dev).contiguous()
                out = recurrent_attention(torch.from_numpy(x).to(dev), torch.from_numpy(v).to(dev), rt,
                                          torch.from_numpy(freqs).to(dev), position, RotaryEmbedding(rotary), slopes)
                torch.cuda.synchronize()
            finally:
                ctx.set_option("state_step.dense_chunks", -1)
            res.append((out.cpu().numpy(), rt.cpu().numpy()))
        tol = 1e-4 if rotary == orc.ALIBI else 2e-5
        scale_o = max(np.abs(res[0][0]).max(), 1e-6)
        scale_r = max(np.abs(res[0][1]).max(), 1e-6)
        assert np.abs(res[1][0] - res[0][0]).max() <= tol * scale_o, label
        assert np.abs(res[1][1] - res[0][1]).max() <= tol * scale_r, label
        if case < 6:
            q = corc.rotate(x, freqs, rotary, position)
            out_ref, rho_ref = corc.recurrent_attention(q, v, rho0.copy(), None if slopes is None else corc.alibi_decay(slopes))
            assert np.abs(res[1][0] - out_ref).max() <= tol * max(np.abs(out_ref).max(), 1e-6), label
            assert np.abs(res[1][1] - rho_ref).max() <= tol * max(np.abs(rho_ref).max(), 1e-6), label


@pytest.mark.parametrize("rotary", [orc.ROPE, orc.ALIBI])
def test_dense_chunk_form_with_a_bf16_state(gpu, corc, rotary):
    """bf16 storage in the many-token form: the state is widened to f32 for the call and rounded once at its
    end, so it lands within one bf16 rounding of the f32 result (the token loop rounds after every token);
    2e-2 relative (north_star) against the oracle."""
    _, recurrent_attention = gpu
    from burn_dragon_amd.positional import RotaryEmbedding

    B, h, T, N, d = 2, 2, 200, 128, 64
    x, v, rho0 = make_inputs(321, B, h, T, N, d, 0.2, rho_scale=0.05)
    rho_b = torch.from_numpy(rho0).to(torch.bfloat16)
    freqs = corc.build_freqs(N, rotary=rotary)
    slopes = np.array([0.02, 0.05], np.float32) if rotary == orc.ALIBI else None
    dev = "cuda:0"
    rt = rho_b.to(dev).contiguous()
    out = recurrent_attention(torch.from_numpy(x).to(dev), torch.from_numpy(v).to(dev), rt,
                              torch.from_numpy(freqs).to(dev), 5, RotaryEmbedding(rotary), slopes)
    torch.cuda.synchronize()
    assert rt.dtype == torch.bfloat16
    q = corc.rotate(x, freqs, rotary, 5)
    out_ref, rho_ref = corc.recurrent_attention(q, v, rho_b.float().numpy().copy(),
                                                None if slopes is None else corc.alibi_decay(slopes))
    assert rel_err(out.cpu().numpy(), out_ref) < 1e-4  # the readouts never see a rounded state inside the call
    got = rt.float().cpu().numpy()
    assert rel_err(got, rho_ref) < 2e-2
    # exactly the f32 result rounded to bf16, up to f32 reassociation before the rounding
    want = torch.from_numpy(rho_ref).to(torch.bfloat16).float().numpy()
    assert (got != want).mean() < 0.02


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rotary", [orc.POPE, orc.ALIBI])
@pytest.mark.parametrize("N,d", [(130, 256), (96, 512)])
def test_dense_streaming_kernel_equals_generic_kernel_and_oracle(gpu, corc, rotary, N, d, dtype):
    """PoPE and eager ALiBi at d in {256,512} take k_step_dense: the same operations per element in the same
    order as the generic kernel (bit-identical state and readout), and the oracle's values."""
    ffi, recurrent_attention = gpu
    from burn_dragon_amd.positional import RotaryEmbedding

    ctx = ffi.default_context(0)
    B, h, T = 2, 3, 3
    x, v, _ = make_inputs(55 + N + d, B, h, T, N, d, 0.3)
    Nq = 2 * N if rotary == orc.POPE else N
    rho0 = (0.05 * np.random.default_rng(6).standard_normal((B, h, Nq, d))).astype(np.float32)
    rho0 = torch.from_numpy(rho0).to(dtype).float().numpy()  # representable in the storage type
    freqs = corc.build_freqs(N, rotary=rotary)
    slopes = np.array([0.1, 0.4, 0.9], np.float32) if rotary == orc.ALIBI else None
    dev = "cuda:0"
    res = []
    for mode in (1, 0):
        ctx.set_option("state_step.dense_kernel", mode)
        try:
            rt = torch.from_numpy(rho0).to(dev).to(dtype).contiguous()
            out, rows = recurrent_attention(torch.from_numpy(x).to(dev), torch.from_numpy(v).to(dev), rt,
                                            torch.from_numpy(freqs).to(dev), 77, RotaryEmbedding(rotary), slopes,
                                            want_rows=True)
            torch.cuda.synchronize()
        finally:
            ctx.set_option("state_step.dense_kernel", 1)
        res.append((out.cpu().numpy(), rt.float().cpu().numpy(), rows.cpu().numpy()))
    assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1], res[1][1])
    assert (res[0][2] == Nq).all() and (res[1][2] == Nq).all()  # every row is touched on every token
    q = corc.rotate(x, freqs, rotary, 77)
    out_ref, rho_ref = corc.recurrent_attention(q, v, rho0.copy(), None if slopes is None else corc.alibi_decay(slopes))
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert rel_err(res[0][0], out_ref) < tol and rel_err(res[0][1], rho_ref) < tol
