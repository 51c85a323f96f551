"""Model-level entry points of this library that the reference reaches through ModelState: the state given layer by
layer (bdh_model_forward_layers; src/model/state.rs:5-15, src/model/bdh.rs:274,304) and the decode step with deferred
state updates (bdh_model_forward_deferred / bdh_model_flush), through the C ABI.

Bars: per-layer pointers against the one-allocation call: bit equality of logits and states.  Deferred decode: logits
of every step against the CPU oracle's forward_with_state (src/model/bdh.rs:309-450) within 1e-3 (f32 state) / 2e-2
(bf16 state) and against the eager model call within 1e-4; the flushed state within 1e-5 of the eager one (the
activations downstream of a reassociated readout differ in the last bits, so not bit equality here -- the single-layer
test of the step itself holds that bar).
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import bdh_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def bda():
    if not torch.cuda.is_available():
        pytest.fail("no HIP device: the GPU tests must run on the MI355X box")
    import burn_dragon_amd

    return burn_dragon_amd


def rel_err(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def _model(bda, rotary, L, d, h, mult, V, seed, **kw):
    cfg = bda.BDHConfig(n_layer=L, n_embd=d, n_head=h, mlp_internal_dim_multiplier=mult, vocab_size=V)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding(rotary))
    shape = orc.BDHShape(n_layer=L, n_embd=d, n_head=h, mlp_internal_dim_multiplier=mult, vocab_size=V, rotary=rotary)
    w = orc.init_weights(shape, seed)
    return bda.BDH(cfg, DEV, weights=vars(w), **kw), shape, w


@pytest.mark.parametrize("rotary,lazy", [(orc.ROPE, False), (orc.ALIBI, True), (orc.POPE, False)])
def test_state_given_layer_by_layer_equals_the_single_allocation(bda, rotary, lazy):
    """A 6-token prompt and three decode steps: every layer's state in an allocation of its own (and, for the lazily
    decayed ALiBi state, its stamps too) against one [L,B,h,Nq,d] tensor."""
    from burn_dragon_amd import ffi

    L, d, h, mult, V, B = 3, 256, 2, 4, 64, 2
    model, shape, _ = _model(bda, rotary, L, d, h, mult, V, 5, alibi_lazy=lazy)
    N = model.latent
    Nq = model.latent_q
    rng = np.random.default_rng(1)
    calls = [rng.integers(0, V, size=(B, 6))] + [rng.integers(0, V, size=(B, 1)) for _ in range(3)]
    ctx, lib = model.ctx, model.ctx.lib

    def run(separate):
        whole = torch.zeros((L, B, h, Nq, d), device=DEV)
        stamps = torch.zeros((L, B, h, N), device=DEV, dtype=torch.int32) if lazy else None
        if separate:  # independent allocations, deliberately not adjacent
            rhos = [torch.zeros((B, h, Nq, d), device=DEV) for _ in range(L)]
            pad = [torch.zeros(1000 + 64 * i, device=DEV) for i in range(L)]  # noqa: F841
            sts = [torch.zeros((B, h, N), device=DEV, dtype=torch.int32) for _ in range(L)] if lazy else None
            rho_ptrs = (ctypes.c_void_p * L)(*[t.data_ptr() for t in rhos])
            st_ptrs = (ctypes.c_void_p * L)(*[t.data_ptr() for t in sts]) if lazy else None
        outs, pos = [], 0
        for toks in calls:
            tt = torch.from_numpy(toks).to(DEV)
            T = toks.shape[1]
            logits = torch.empty((B, T, V), device=DEV)
            nxt = torch.empty((B,), device=DEV, dtype=torch.int64)
            if separate:
                ctx.check(lib.bdh_model_forward_layers(model.handle, tt.data_ptr(), B, T, rho_ptrs, ffi.F32, st_ptrs, pos,
                                                       None, logits.data_ptr(), nxt.data_ptr(), None))
            else:
                ctx.check(lib.bdh_model_forward_lazy(model.handle, tt.data_ptr(), B, T, whole.data_ptr(), ffi.F32,
                                                     ffi.ptr(stamps), pos, None, logits.data_ptr(), nxt.data_ptr(), None))
            pos += T
            outs.append((logits, nxt))
        torch.cuda.synchronize()
        if separate:
            return outs, torch.stack(rhos), (torch.stack(sts) if lazy else None)
        return outs, whole, stamps

    model.ctx.set_option("model.one_launch", 0)  # the same kernel-by-kernel path on both sides
    try:
        outs_a, rho_a, st_a = run(False)
        outs_b, rho_b, st_b = run(True)
    finally:
        model.ctx.set_option("model.one_launch", 1)
    for (la, na), (lb, nb) in zip(outs_a, outs_b):
        assert torch.equal(la, lb) and torch.equal(na, nb)
    assert torch.equal(rho_a, rho_b)
    if lazy:
        assert torch.equal(st_a, st_b)
    # adjacent layers handed over one by one may take the fused decode forms: the values of the contiguous call
    whole = torch.zeros((L, B, h, Nq, d), device=DEV)
    stamps = torch.zeros((L, B, h, N), device=DEV, dtype=torch.int32) if lazy else None
    rho_ptrs = (ctypes.c_void_p * L)(*[whole[l].data_ptr() for l in range(L)])
    st_ptrs = (ctypes.c_void_p * L)(*[stamps[l].data_ptr() for l in range(L)]) if lazy else None
    pos = 0
    for toks in calls:
        tt = torch.from_numpy(toks).to(DEV)
        T = toks.shape[1]
        logits = torch.empty((B, T, V), device=DEV)
        ctx.check(lib.bdh_model_forward_layers(model.handle, tt.data_ptr(), B, T, rho_ptrs, ffi.F32, st_ptrs, pos, None,
                                               logits.data_ptr(), None, None))
        pos += T
    torch.cuda.synchronize()
    assert rel_err(whole.cpu().numpy(), rho_a.cpu().numpy()) < 1e-5
    with pytest.raises(ffi.BdhError):
        bad = (ctypes.c_void_p * L)(*([whole[0].data_ptr()] + [None] * (L - 1)))
        ctx.check(lib.bdh_model_forward_layers(model.handle, tt.data_ptr(), B, 1, bad, ffi.F32, None, pos, None,
                                               logits.data_ptr(), None, None))


@pytest.mark.parametrize("state,tol", [("f32", 1e-3), ("bf16", 2e-2)])
@pytest.mark.parametrize("capacity", [4, 32])
def test_model_decode_with_deferred_updates(bda, corc, state, tol, capacity):
    """L=3, d=256, h=4, N=1024: an 8-token prompt (eager call), 40 greedy steps with the updates deferred (the logs
    flush themselves every `capacity` steps), then a second prompt call, which must find the state flushed."""
    from burn_dragon_amd import ffi

    L, d, h, mult, V, B, T0, steps = 3, 256, 4, 16, 256, 2, 8, 40
    dt = ffi.F32 if state == "f32" else ffi.BF16
    model, shape, w = _model(bda, orc.ROPE, L, d, h, mult, V, 9, rho_dtype=dt, defer_updates=capacity)
    eager, _, _ = _model(bda, orc.ROPE, L, d, h, mult, V, 9, rho_dtype=dt)
    N = model.latent
    prompt = np.random.default_rng(2).integers(0, V, size=(B, T0))
    st, st_e = model.init_state(), eager.init_state()
    logits = model.forward_with_state(torch.from_numpy(prompt), st)
    logits_e = eager.forward_with_state(torch.from_numpy(prompt), st_e)
    assert torch.equal(logits, logits_e)
    rho_ref = np.zeros((L, B, h, N, d), np.float32)
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, prompt, rho_ref, 0)
    print(f"deferred model decode, {state} state, capacity {capacity}", flush=True)
    for step in range(steps):
        tok = np.array([[corc.greedy_token(logits_ref[b, -1])] for b in range(B)])
        logits = model.forward_with_state(torch.from_numpy(tok), st)
        logits_e = eager.forward_with_state(torch.from_numpy(tok), st_e)
        logits_ref, pos, _, _ = corc.forward_with_state(shape, w, tok, rho_ref, pos)
        assert rel_err(logits.cpu().numpy(), logits_ref) < tol, f"step {step}"
        assert rel_err(logits.cpu().numpy(), logits_e.cpu().numpy()) < (1e-4 if state == "f32" else tol), f"step {step}"
        assert st.logs is not None and 1 <= st.logs.pending <= capacity
    assert st.position == T0 + steps == pos
    tail = np.random.default_rng(3).integers(0, V, size=(B, 5))  # a prompt call flushes what is pending
    logits = model.forward_with_state(torch.from_numpy(tail), st)
    logits_e = eager.forward_with_state(torch.from_numpy(tail), st_e)
    assert st.logs.pending == 0
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, tail, rho_ref, pos)
    assert rel_err(logits.cpu().numpy(), logits_ref) < tol
    assert rel_err(st.storage.float().cpu().numpy(), st_e.storage.float().cpu().numpy()) < (1e-5 if state == "f32" else tol)
    assert rel_err(st.storage.float().cpu().numpy(), rho_ref) < tol
    # materialize_state is the explicit flush
    model.forward_with_state(torch.from_numpy(tail[:, :1]), st)
    assert st.logs.pending == 1
    model.materialize_state(st)
    assert st.logs.pending == 0


@pytest.mark.parametrize("state,tol", [("f32", 1e-3), ("bf16", 2e-2)])
def test_config4_architecture_with_deferred_updates(bda, corc, state, tol):
    """BASELINE config 4's layer shape (d=512, h=8, N=16384, V=256, RoPE) at L=2, B=2: an 8-token prompt, then 6
    greedy steps fed with the oracle's tokens through the deferred decode step with a log of 4 steps (one flush by the
    step itself, one by materialize_state): logits and final state against the oracle."""
    from burn_dragon_amd import ffi

    L, d, h, mult, V, B, T0 = 2, 512, 8, 256, 256, 2, 8
    dt = ffi.F32 if state == "f32" else ffi.BF16
    model, shape, w = _model(bda, orc.ROPE, L, d, h, mult, V, 44, rho_dtype=dt, defer_updates=4)
    N = model.latent
    assert N == 16384
    prompt = np.random.default_rng(4).integers(0, V, size=(B, T0))
    st = model.init_state()
    print(f"config-4 architecture with deferred updates, {state} state", flush=True)
    logits = model.forward_with_state(torch.from_numpy(prompt), st)
    rho_ref = np.zeros((L, B, h, N, d), np.float32)
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, prompt, rho_ref, 0)
    assert rel_err(logits.cpu().numpy(), logits_ref) < tol
    worst = 0.0
    for step in range(6):
        tok = np.array([[corc.greedy_token(logits_ref[b, -1])] for b in range(B)])
        logits = model.forward_with_state(torch.from_numpy(tok), st)
        logits_ref, pos, _, _ = corc.forward_with_state(shape, w, tok, rho_ref, pos)
        worst = max(worst, rel_err(logits.cpu().numpy(), logits_ref))
        assert worst < tol, f"step {step}: {worst}"
    assert st.logs.pending == 2
    model.materialize_state(st)
    e_state = rel_err(st.storage.float().cpu().numpy(), rho_ref)
    print(f"worst decode logits rel err {worst:.2e}, state rel err {e_state:.2e}", flush=True)
    assert e_state < tol


def test_deferred_decode_with_the_state_given_layer_by_layer(bda):
    """bdh_model_forward_deferred_layers / bdh_model_flush_layers on per-layer allocations against
    bdh_model_forward_deferred / bdh_model_flush on one tensor: the same launches on the same bytes, so logits and
    flushed states are equal bit for bit; 11 steps with a log capacity of 4 (two flushes by the steps themselves)."""
    from burn_dragon_amd import ffi

    L, d, h, mult, V, B, cap = 3, 256, 2, 8, 64, 2, 4
    model, _, _ = _model(bda, orc.ROPE, L, d, h, mult, V, 7)
    N = model.latent
    ctx, lib = model.ctx, model.ctx.lib
    rng = np.random.default_rng(4)
    prompt = torch.from_numpy(rng.integers(0, V, size=(B, 5))).to(DEV)
    steps = [torch.from_numpy(rng.integers(0, V, size=(B, 1))).to(DEV) for _ in range(11)]

    def run(separate):
        whole = torch.zeros((L, B, h, N, d), device=DEV)
        rhos = [torch.zeros((B, h, N, d), device=DEV) for _ in range(L)] if separate else [whole[l] for l in range(L)]
        ptrs = (ctypes.c_void_p * L)(*[t.data_ptr() for t in rhos])
        logs = ctypes.c_void_p()
        ctx.check(lib.bdh_model_logs_create(model.handle, B, ffi.F32, cap, ctypes.byref(logs)))
        try:
            logits = torch.empty((B, 5, V), device=DEV)
            ctx.check(lib.bdh_model_forward_layers(model.handle, prompt.data_ptr(), B, 5, ptrs, ffi.F32, None, 0, None,
                                                   logits.data_ptr(), None, None))
            outs, pos = [], 5
            for tok in steps:
                lg = torch.empty((B, 1, V), device=DEV)
                if separate:
                    ctx.check(lib.bdh_model_forward_deferred_layers(model.handle, logs, tok.data_ptr(), B, ptrs, ffi.F32,
                                                                    pos, None, lg.data_ptr(), None))
                else:
                    ctx.check(lib.bdh_model_forward_deferred(model.handle, logs, tok.data_ptr(), B, whole.data_ptr(),
                                                             ffi.F32, pos, None, lg.data_ptr(), None))
                pos += 1
                outs.append(lg)
            assert lib.bdh_model_logs_pending(logs) == 11 % cap
            if separate:
                ctx.check(lib.bdh_model_flush_layers(model.handle, logs, ptrs))
            else:
                ctx.check(lib.bdh_model_flush(model.handle, logs, whole.data_ptr()))
            assert lib.bdh_model_logs_pending(logs) == 0
            torch.cuda.synchronize()
            return outs, torch.stack(list(rhos)).clone()
        finally:
            lib.bdh_model_logs_destroy(model.handle, logs)

    model.ctx.set_option("model.one_launch", 0)  # the prompt call kernel by kernel on both sides
    try:
        outs_a, rho_a = run(False)
        outs_b, rho_b = run(True)
    finally:
        model.ctx.set_option("model.one_launch", 1)
    for la, lb in zip(outs_a, outs_b):
        assert torch.equal(la, lb)
    assert torch.equal(rho_a, rho_b)
    assert rho_a.abs().max() > 0
