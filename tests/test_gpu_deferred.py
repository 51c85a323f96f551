"""GPU parity of the deferred-update decode step (bdh_state_step_deferred / bdh_state_flush) through the C ABI.

What is checked, per step and after flushes:
  - the readout of EVERY step against the CPU oracle's token loop (BDH::recurrent_attention,
    src/model/bdh.rs:258-307): 1e-3 relative for an f32 state, 2e-2 for a bf16 state (north_star's bounds);
  - the active bitmask and the touched-row counts: bit-exact against the oracle's index artefacts;
  - the FLUSHED state: `array_equal` to the state the eager entry point bdh_state_step leaves after the same
    steps (the flush applies the logged updates in step order with the eager step's operations);
  - log capacities 1, 8, 32, 64 and 128, a flush in the middle of a log, f32 and bf16 states, d = 256 and 512,
    a latent size that leaves the last workgroup's unit partly empty, per-sequence device positions.
"""
import ctypes

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
    from burn_dragon_amd import recurrent

    return ffi, recurrent


def rel_err(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def make_steps(seed, steps, B, h, N, d, density):
    from scipy.stats import norm

    rng = np.random.default_rng(seed)
    mu = norm.ppf(density)
    xs = np.maximum(rng.standard_normal((steps, B, h, N)) + mu, 0).astype(np.float32)
    vs = rng.standard_normal((steps, B, d)).astype(np.float32)
    rho = (0.01 * rng.standard_normal((B, h, N, d))).astype(np.float32)
    return xs, vs, rho


def eager_steps(recurrent, xs, vs, rho_t, freqs_t, p0):
    """The same steps through bdh_state_step on a copy of the state; returns (outs, final state)."""
    from burn_dragon_amd.positional import RotaryEmbedding

    rho_e = rho_t.clone()
    outs = []
    for t in range(xs.shape[0]):
        o = recurrent.recurrent_attention(xs[t].unsqueeze(2), vs[t].unsqueeze(1), rho_e, freqs_t, p0 + t,
                                          RotaryEmbedding.ROPE)
        outs.append(o[:, :, 0])
    return outs, rho_e


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.bfloat16, 2e-2)], ids=["f32", "bf16"])
@pytest.mark.parametrize("capacity", [1, 8, 32, 128])
@pytest.mark.parametrize("N,d,density,steps", [(1024, 256, 0.05, 70), (640, 512, 0.3, 40), (1024, 256, 0.3, 150)])
def test_deferred_steps_match_oracle_and_flushed_state_equals_eager(gpu, corc, capacity, N, d, density, steps, dtype, tol):
    ffi, recurrent = gpu
    B, h, p0 = 2, 2, 1000
    xs, vs, rho = make_steps(11 + N + capacity, steps, B, h, N, d, density)
    freqs = corc.build_freqs(N)
    dev = "cuda:0"
    xt, vt, ft = (torch.from_numpy(a).to(dev) for a in (xs, vs, freqs))
    rho_t = torch.from_numpy(rho).to(dev).to(dtype).contiguous()
    outs_e, rho_e = eager_steps(recurrent, xt, vt, rho_t, ft, p0)

    if capacity * d > 32768:
        pytest.skip("capacity * d <= 32768")
    print(f"deferred capacity={capacity} N={N} d={d} dtype={dtype}", flush=True)
    log = recurrent.StateLog(B, h, N, d, dtype, capacity)
    rho_ref = rho_t.float().cpu().numpy()  # the oracle walks the same (rounded) initial state in f32
    flush_mid = steps // 2 + 1  # a flush that does not fall on a multiple of the capacity
    for t in range(steps):
        if t == flush_mid:
            log.flush(rho_t)
            assert log.pending == 0
        out, bm, rows = recurrent.state_step_deferred(log, xt[t], vt[t], rho_t, ft, p0 + t, want_bitmask=True,
                                                      want_rows=True)
        torch.cuda.synchronize()
        q = corc.rotate(xs[t][:, :, None, :], freqs, orc.ROPE, p0 + t)
        out_ref, rho_ref = corc.recurrent_attention(q, vs[t][:, None, :], rho_ref)
        assert rel_err(out.cpu().numpy(), out_ref[:, :, 0]) < tol, f"step {t}"
        if dtype == torch.float32:  # same state on both sides: the deferred readout is the eager one reassociated
            assert rel_err(out.cpu().numpy(), outs_e[t].cpu().numpy()) < 2e-5, f"step {t}"
        assert np.array_equal(bm.cpu().numpy().view(np.uint64),
                              orc.active_bitmask(np.pad(xs[t], ((0, 0), (0, 0), (0, (-N) % 64))))), f"step {t}"
        assert np.array_equal(rows.cpu().numpy(), orc.pair_closed_rows(xs[t])), f"step {t}"
        assert 1 <= log.pending <= capacity
    log.flush(rho_t)
    torch.cuda.synchronize()
    assert log.pending == 0
    assert torch.equal(rho_t, rho_e), "the flushed state must hold the bits of the eager steps"
    if dtype == torch.float32:
        assert rel_err(rho_t.cpu().numpy(), rho_ref) < 1e-6
    log.close()


@pytest.mark.parametrize("steps", [64, 128])
def test_full_log_dense_activity_and_device_positions(gpu, corc, steps):
    """Every pair active in every step (the flush applies `steps` updates to every row), per-sequence positions."""
    ffi, recurrent = gpu
    B, h, N, d = 3, 2, 512, 256
    rng = np.random.default_rng(5)
    xs = (np.abs(rng.standard_normal((steps, B, h, N))) + 0.1).astype(np.float32)
    vs = rng.standard_normal((steps, B, d)).astype(np.float32)
    rho = (0.01 * rng.standard_normal((B, h, N, d))).astype(np.float32)
    freqs = corc.build_freqs(N)
    starts = np.array([5, 900, 4000], np.int32)
    dev = "cuda:0"
    xt, vt, ft = (torch.from_numpy(a).to(dev) for a in (xs, vs, freqs))
    rho_t = torch.from_numpy(rho).to(dev)
    pos_t = torch.from_numpy(starts).to(dev)
    log = recurrent.StateLog(B, h, N, d, torch.float32, steps)
    rho_ref = rho.copy()
    for t in range(steps):
        out = recurrent.state_step_deferred(log, xt[t], vt[t], rho_t, ft, 0, positions=pos_t + t)
        torch.cuda.synchronize()
        q = np.concatenate([corc.rotate(xs[t][b:b + 1, :, None, :], freqs, orc.ROPE, int(starts[b]) + t) for b in range(B)])
        out_ref, rho_ref = corc.recurrent_attention(q, vs[t][:, None, :], rho_ref)
        assert rel_err(out.cpu().numpy(), out_ref[:, :, 0]) < 1e-3, f"step {t}"
    assert log.pending == steps
    assert torch.equal(rho_t, torch.from_numpy(rho).to(dev)), "no step may write the state before the flush"
    log.flush(rho_t)
    torch.cuda.synchronize()
    assert rel_err(rho_t.cpu().numpy(), rho_ref) < 1e-6
    log.close()


def test_log_contract_and_argument_errors(gpu, corc):
    ffi, recurrent = gpu
    ctx = ffi.default_context(0)
    for bad in [dict(N=512, d=128, capacity=8), dict(N=512, d=256, capacity=0), dict(N=512, d=256, capacity=129),
                dict(N=512, d=512, capacity=65), dict(N=511, d=256, capacity=8)]:
        with pytest.raises(ffi.BdhError) as e:
            recurrent.StateLog(1, 1, bad["N"], bad["d"], torch.float32, bad["capacity"])
        assert e.value.status in (ffi.E_SHAPE, ffi.E_INVAL)
    B, h, N, d = 1, 2, 512, 256
    xs, vs, rho = make_steps(3, 3, B, h, N, d, 0.2)
    dev = "cuda:0"
    xt, vt = torch.from_numpy(xs).to(dev), torch.from_numpy(vs).to(dev)
    ft = torch.from_numpy(corc.build_freqs(N)).to(dev)
    rho_a, rho_b = torch.from_numpy(rho).to(dev), torch.from_numpy(rho).to(dev)
    log = recurrent.StateLog(B, h, N, d, torch.float32, 4)
    assert log.pending == 0 and log.nbytes > 0
    log.flush(rho_a)  # nothing pending: no-op
    recurrent.state_step_deferred(log, xt[0], vt[0], rho_a, ft, 0)
    assert log.pending == 1
    with pytest.raises(ffi.BdhError) as e:  # pending steps belong to rho_a
        recurrent.state_step_deferred(log, xt[1], vt[1], rho_b, ft, 1)
    assert e.value.status == ffi.E_INVAL and log.pending == 1
    with pytest.raises(ffi.BdhError):
        log.flush(rho_b)
    log.flush(rho_a)
    recurrent.state_step_deferred(log, xt[1], vt[1], rho_b, ft, 1)  # an empty log takes any state
    log.flush(rho_b)
    rc = ctx.lib.bdh_state_step_deferred(ctx.handle, None, ffi.ptr(xt), ffi.ptr(vt), ffi.ptr(ft), 0, None, ffi.ptr(rho_a),
                                         ffi.ptr(rho_b), None, None)
    assert rc == ffi.E_INVAL
    torch.cuda.synchronize()
    log.close()


def test_deferred_readout_is_deterministic(gpu, corc):
    ffi, recurrent = gpu
    B, h, N, d, steps = 2, 4, 2048, 256, 20
    xs, vs, rho = make_steps(9, steps, B, h, N, d, 0.1)
    dev = "cuda:0"
    xt, vt = torch.from_numpy(xs).to(dev), torch.from_numpy(vs).to(dev)
    ft = torch.from_numpy(corc.build_freqs(N)).to(dev)
    runs = []
    for _ in range(2):
        rho_t = torch.from_numpy(rho).to(dev)
        log = recurrent.StateLog(B, h, N, d, torch.float32, 16)
        outs = [recurrent.state_step_deferred(log, xt[t], vt[t], rho_t, ft, 77 + t).clone() for t in range(steps)]
        log.flush(rho_t)
        torch.cuda.synchronize()
        runs.append((torch.stack(outs), rho_t))
        log.close()
    assert torch.equal(runs[0][0], runs[1][0]) and torch.equal(runs[0][1], runs[1][1])


@pytest.mark.parametrize("K", [64, 128])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.bfloat16, 2e-2)], ids=["f32", "bf16"])
def test_deferred_full_size_config2_against_the_eager_step(gpu, corc, dtype, tol, K):
    """BASELINE config 2 at its full size (rho [32,4,8192,256], 5 % active), log capacities 64 and 128 (bench.py runs 128):
    70 steps (one flush by the step itself, one by the caller) against the eager entry point on a second copy of
    the state -- readouts within tolerance on every step, flushed state bit-identical."""
    ffi, recurrent = gpu
    from scipy.stats import norm

    B, h, N, d, steps = 32, 4, 8192, 256, K + 6
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(21)
    rho_t = (0.01 * torch.randn((B, h, N, d), device=dev, generator=g)).to(dtype).contiguous()
    mu = float(norm.ppf(0.05))
    ft = torch.from_numpy(corc.build_freqs(N)).to(dev)
    from burn_dragon_amd.positional import RotaryEmbedding

    rho_e = rho_t.clone()
    log = recurrent.StateLog(B, h, N, d, dtype, K)
    print(f"deferred config 2 dtype={dtype} log bytes={log.nbytes}", flush=True)
    worst = 0.0
    for t in range(steps):
        x = torch.relu(torch.randn((B, h, N), device=dev, generator=g) + mu).contiguous()
        v = torch.randn((B, d), device=dev, generator=g).contiguous()
        out_e, rows_e = recurrent.recurrent_attention(x.unsqueeze(2), v.unsqueeze(1), rho_e, ft, 100 + t,
                                                      RotaryEmbedding.ROPE, want_rows=True)
        out_d, rows_d = recurrent.state_step_deferred(log, x, v, rho_t, ft, 100 + t, want_rows=True)
        err = ((out_d - out_e[:, :, 0]).abs().max() / out_e.abs().max()).item()
        worst = max(worst, err)
        assert err < (2e-5 if dtype == torch.float32 else tol), f"step {t}: {err}"
        assert torch.equal(rows_d, rows_e[:, :, 0])
    assert log.pending == steps - K
    log.flush(rho_t)
    torch.cuda.synchronize()
    assert torch.equal(rho_t, rho_e)
    print(f"worst readout difference to the eager step: {worst:.2e}", flush=True)
    log.close()
