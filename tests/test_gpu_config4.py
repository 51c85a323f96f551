"""BASELINE configs 4 and 5 on the GPU, through the C ABI.

Config 4 = the larger model (V=256, d=512, h=8, N=16384 per head, L=12, B=32, RoPE; the path of
src/model/bdh.rs:309-450 at that shape).  The C oracle walks a dense 67 M-parameter projection three times
per token and layer, so oracle parity runs the true layer shape with a reduced stack (L=2, B=2, a short
prompt and a few greedy steps); the full specification (L=12, B=32, 96 GiB of f32 state) is covered by
properties that need no oracle: decode == prefill, rows of never-active lane pairs keep their zero bits,
and the touched-row count of the step at the full layer shape equals the pair-closed count of its input.

Config 5 = the single-layer step at the config-4 layer shape over densities {1,2,5,10,20} % in f32 and
bf16 state, B in {1, 8, 64}: B=1 and B=8 against the oracle, B=64 (16 GiB f32) against an f32 torch
statement of the same step plus the index invariants.

Tolerances: 1e-3 relative (f32 state), 2e-2 (bf16 state) on the max-norm; index artefacts bit-exact.
"""
import numpy as np
import pytest
import torch

from oracle import bdh_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
MU = {0.01: -2.3263, 0.02: -2.0537, 0.05: -1.6449, 0.10: -1.2816, 0.20: -0.8416}  # Phi^-1(density)


@pytest.fixture(scope="module")
def bda():
    if not torch.cuda.is_available():
        pytest.fail("no HIP device: the GPU tests must run on the MI355X box")
    import burn_dragon_amd

    return burn_dragon_amd


def rel_err(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def _config4(bda, n_layer):
    cfg = bda.BDHConfig(n_layer=n_layer, n_embd=512, n_head=8, mlp_internal_dim_multiplier=256, vocab_size=256)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    shape = orc.BDHShape(n_layer=n_layer, n_embd=512, n_head=8, mlp_internal_dim_multiplier=256, vocab_size=256,
                         rotary=orc.ROPE)
    assert cfg.latent_per_head() == 16384 == shape.latent_per_head
    return cfg, shape


@pytest.fixture(scope="module")
def config4_weights():
    shape = orc.BDHShape(n_layer=2, n_embd=512, n_head=8, mlp_internal_dim_multiplier=256, vocab_size=256, rotary=orc.ROPE)
    return orc.init_weights(shape, 44)  # weights are shared by all layers: the same set serves L=2 and L=12


@pytest.mark.parametrize("state", ["f32", "bf16"])
def test_config4_architecture_against_oracle(bda, corc, config4_weights, state):
    """d=512, h=8, N=16384, V=256, RoPE at L=2, B=2: an 8-token prompt in one call, then 4 greedy steps fed
    with the oracle's tokens.  f32 state: logits 1e-3, layer-0 activations and active set bit-exact, deeper
    layers' sets equal away from zero pre-activations, final state 1e-3.  bf16 state: logits and state 2e-2."""
    from burn_dragon_amd import ffi

    cfg, shape = _config4(bda, 2)
    w = config4_weights
    tol = 1e-3 if state == "f32" else 2e-2
    model = bda.BDH(cfg, DEV, weights=vars(w), rho_dtype=ffi.F32 if state == "f32" else ffi.BF16)
    L, B, h, N, d, T0 = 2, 2, 8, 16384, 512, 8
    prompt = np.random.default_rng(4).integers(0, 256, size=(B, T0))
    st = model.init_state()
    x_tap = torch.zeros((L, B, h, T0, N), device=DEV)
    print(f"config-4 architecture L={L} B={B} state {state}: prompt of {T0}", flush=True)
    logits, nxt = model.forward_with_state(torch.from_numpy(prompt), st, want_next=True, x_tap=x_tap)
    torch.cuda.synchronize()
    rho_ref = np.zeros((L, B, h, N, d), np.float32)
    logits_ref, pos, x_ref, _ = corc.forward_with_state(shape, w, prompt, rho_ref, 0, taps=True)
    assert rel_err(logits.cpu().numpy(), logits_ref) < tol
    x_gpu = x_tap.cpu().numpy()
    assert np.array_equal(x_gpu[0], x_ref[0])  # layer 0 sees no state: values and active set bit-exact
    flips = (x_gpu[1] > 0) != (x_ref[1] > 0)
    if state == "f32":
        assert flips.mean() < 1e-3
        assert np.maximum(x_gpu[1], x_ref[1])[flips].max(initial=0.0) < 1e-4
    worst = 0.0
    for step in range(4):
        tok_ref = np.array([[corc.greedy_token(logits_ref[b, -1])] for b in range(B)])
        if state == "f32":
            for b in range(B):
                if int(nxt[b]) != tok_ref[b, 0]:
                    top = np.sort(logits_ref[b, -1])[-2:]
                    assert top[1] - top[0] < 1e-3 * np.abs(logits_ref).max(), f"step {step}: argmax differs on a clear lead"
        logits, nxt = model.forward_with_state(torch.from_numpy(tok_ref), st, want_next=True)
        logits_ref, pos, _, _ = corc.forward_with_state(shape, w, tok_ref, rho_ref, pos)
        worst = max(worst, rel_err(logits.cpu().numpy(), logits_ref))
        assert worst < tol, f"step {step}: {worst}"
    assert st.position == T0 + 4 == pos
    e_state = rel_err(st.storage.float().cpu().numpy(), rho_ref)
    print(f"config-4 architecture, {state} state: worst decode logits rel err {worst:.2e}, state rel err {e_state:.2e}, "
          f"layer-1 active-set flips {int(flips.sum())} of {flips.size}")
    assert e_state < tol


def test_config4_full_size_properties(bda, corc, config4_weights):
    """The full specification: L=12, B=32, f32 state [12,32,8,16384,512] = 96 GiB (two of them live here).
    (1) decode == prefill: a 3-token prompt in one call against three single-token calls — logits and
    states agree to f32 reassociation (the projections of a 96-row call and of a 32-row call take different
    tilings); (2) rows of lane pairs that were never active keep their zero bits; (3) the step at the full
    layer shape [32,8,16384,512] reports rows_touched == the pair-closed count of its x and the bitmask of
    x > 0, and leaves every other row's bits alone; (4) one batch entry of layer 0 against the oracle."""
    from burn_dragon_amd.positional import RotaryEmbedding
    from burn_dragon_amd.recurrent import recurrent_attention

    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info(0)
    if free < 210 * (1 << 30):
        pytest.skip(f"needs two 96 GiB states; {free >> 30} GiB free")
    cfg, shape = _config4(bda, 12)
    w = config4_weights
    model = bda.BDH(cfg, DEV, weights=vars(w))
    L, B, h, N, d, T = 12, 32, 8, 16384, 512, 3
    tokens = np.random.default_rng(6).integers(0, 256, size=(B, T))
    tt = torch.from_numpy(tokens)
    print("config 4 full size: prompt call", flush=True)
    st_a = model.init_state()
    x_tap = torch.zeros((L, B, h, T, N), device=DEV)
    logits_a = model.forward_with_state(tt, st_a, x_tap=x_tap)
    torch.cuda.synchronize()
    print("config 4 full size: token-by-token calls", flush=True)
    st_b = model.init_state()
    logits_b = torch.cat([model.forward_with_state(tt[:, t:t + 1], st_b) for t in range(T)], dim=1)
    torch.cuda.synchronize()
    assert st_a.position == st_b.position == T
    assert rel_err(logits_a.cpu().numpy(), logits_b.cpu().numpy()) < 1e-4
    for l in range(L):  # (1) states, layer by layer (8 GiB each)
        a, b = st_a.storage[l], st_b.storage[l]
        scale = float(a.abs().max())
        assert float((a - b).abs().max()) <= 1e-4 * scale, l
        # (2) a pair that was inactive for all T tokens was never written: still +0.0 in every bit
        never = ~(x_tap[l] > 0).view(B, h, T, N // 2, 2).any(-1).any(2)  # [B,h,N/2]
        rows = a.view(B, h, N // 2, 2 * d)[never]
        assert int(rows.view(torch.int32).count_nonzero()) == 0, l
        assert 0.003 < float(never.float().mean()) < 0.5
    del st_b, logits_b
    # (4) layer 0, batch entry 0 against the oracle: x of layer 0 comes from the embedding alone, so the
    # sequential state recurrence over the T tokens can be restated from the taps
    from burn_dragon_amd import ffi

    cur0 = corc.layer_norm(w.embed[tokens[0]])  # [T,d]  (src/model/bdh.rs:319-322)
    q0 = corc.rotate(x_tap[0, :1].cpu().numpy(), corc.build_freqs(N), orc.ROPE, 0)
    _, rho0_ref = corc.recurrent_attention(q0, cur0[None], np.zeros((1, h, N, d), np.float32), sparse=True)
    assert rel_err(st_a.storage[0, 0].cpu().numpy(), rho0_ref[0]) < 1e-3
    # (3) one more step on layer 5's state at the full layer shape, with its by-products
    g = torch.Generator(device=DEV).manual_seed(9)
    x = torch.relu(torch.randn((B, h, 1, N), device=DEV, generator=g) - 0.2)  # dense like random-init activations
    v = torch.randn((B, 1, d), device=DEV, generator=g)
    rho = st_a.storage[5]
    before = rho.clone()
    freqs = torch.from_numpy(corc.build_freqs(N)).to(DEV)
    print("config 4 full size: layer-shape step with by-products", flush=True)
    out, bm, rows = recurrent_attention(x, v, rho, freqs, 4095, RotaryEmbedding.ROPE, want_bitmask=True, want_rows=True)
    torch.cuda.synchronize()
    x_np = x.cpu().numpy()[:, :, 0]
    assert np.array_equal(rows.cpu().numpy()[:, :, 0], orc.pair_closed_rows(x_np))
    assert np.array_equal(bm.cpu().numpy().view(np.uint64)[:, :, 0], orc.active_bitmask(x_np))
    active = (x[:, :, 0] > 0).view(B, h, N // 2, 2).any(-1)
    assert torch.equal(rho.view(B, h, N // 2, 2 * d)[~active], before.view(B, h, N // 2, 2 * d)[~active])
    q = torch.from_numpy(corc.rotate(x.cpu().numpy(), freqs.cpu().numpy(), orc.ROPE, 4095)).to(DEV)[:, :, 0]
    out_t = torch.einsum("bhnd,bhn->bhd", before, q)
    assert rel_err(out[:, :, 0].cpu().numpy(), out_t.cpu().numpy()) < 1e-3
    before += q[..., None] * v[:, None, 0, None, :]
    assert float((rho - before).abs().max()) <= 1e-5 * float(before.abs().max())


def _sweep_inputs(seed, B, h, N, d, density):
    rng = np.random.default_rng(seed)
    x = np.maximum(rng.standard_normal((B, h, 1, N), dtype=np.float32) + np.float32(MU[density]), 0)
    v = rng.standard_normal((B, 1, d), dtype=np.float32)
    rho = np.float32(0.01) * rng.standard_normal((B, h, N, d), dtype=np.float32)
    return x, v, rho


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.bfloat16, 2e-2)], ids=["f32", "bf16"])
@pytest.mark.parametrize("density", [0.01, 0.02, 0.05, 0.10, 0.20])
@pytest.mark.parametrize("B", [1, 8])
def test_config5_step_against_oracle(bda, corc, B, density, dtype, tol):
    """The config-4 layer shape (h=8, N=16384, d=512), every density of the sweep, f32 and bf16 state, B=1 and
    B=8, against the oracle's step from the same (bf16-rounded, where it applies) state."""
    from burn_dragon_amd.positional import RotaryEmbedding
    from burn_dragon_amd.recurrent import recurrent_attention

    h, N, d = 8, 16384, 512
    x, v, rho = _sweep_inputs(int(density * 100) + B, B, h, N, d, density)
    rt = torch.from_numpy(rho).to(DEV).to(dtype)
    rho = rt.float().cpu().numpy()
    freqs = corc.build_freqs(N)
    print(f"config-5 step B={B} density {density} {dtype}", flush=True)
    out, bm, rows = recurrent_attention(torch.from_numpy(x).to(DEV), torch.from_numpy(v).to(DEV), rt,
                                        torch.from_numpy(freqs).to(DEV), 4000, RotaryEmbedding.ROPE,
                                        want_bitmask=True, want_rows=True)
    torch.cuda.synchronize()
    out_ref, rho_ref = corc.recurrent_attention(corc.rotate(x, freqs, orc.ROPE, 4000), v, rho, sparse=True)
    e_out, e_rho = rel_err(out.cpu().numpy(), out_ref), rel_err(rt.float().cpu().numpy(), rho_ref)
    print(f"config-5 shape B={B} density {density:.0%} {dtype}: readout rel err {e_out:.2e}, state rel err {e_rho:.2e}")
    assert e_out < tol and e_rho < tol
    assert np.array_equal(rows.cpu().numpy(), orc.pair_closed_rows(x))
    assert np.array_equal(bm.cpu().numpy().view(np.uint64), orc.active_bitmask(x))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.bfloat16, 2e-2)], ids=["f32", "bf16"])
@pytest.mark.parametrize("density", [0.01, 0.02, 0.05, 0.10, 0.20])
def test_config5_step_at_batch_64_properties(bda, corc, density, dtype, tol):
    """B=64 of the sweep (f32 state: 16 GiB): the step against an f32 torch statement of the same sums with q
    from the oracle's rotate, the index by-products against their definitions, and untouched rows bit-identical."""
    from burn_dragon_amd.positional import RotaryEmbedding
    from burn_dragon_amd.recurrent import recurrent_attention

    B, h, N, d = 64, 8, 16384, 512
    g = torch.Generator(device=DEV).manual_seed(int(density * 100))
    rho = (0.01 * torch.randn((B, h, N, d), device=DEV, generator=g)).to(dtype)
    x = torch.relu(torch.randn((B, h, 1, N), device=DEV, generator=g) + MU[density])
    v = torch.randn((B, 1, d), device=DEV, generator=g)
    freqs_np = corc.build_freqs(N)
    before = rho.clone()
    print(f"config-5 step B=64 density {density} {dtype}", flush=True)
    out, bm, rows = recurrent_attention(x, v, rho, torch.from_numpy(freqs_np).to(DEV), 2047, RotaryEmbedding.ROPE,
                                        want_bitmask=True, want_rows=True)
    torch.cuda.synchronize()
    x_np = x.cpu().numpy()
    assert np.array_equal(rows.cpu().numpy(), orc.pair_closed_rows(x_np))
    assert np.array_equal(bm.cpu().numpy().view(np.uint64), orc.active_bitmask(x_np))
    active = (x[:, :, 0] > 0).view(B, h, N // 2, 2).any(-1)
    assert torch.equal(rho.view(B, h, N // 2, 2 * d)[~active], before.view(B, h, N // 2, 2 * d)[~active])
    q = torch.from_numpy(corc.rotate(x_np, freqs_np, orc.ROPE, 2047)).to(DEV)[:, :, 0]
    out_t = torch.zeros((B, h, d), device=DEV)
    worst = 0.0
    for b in range(0, B, 8):  # in slabs, so the f32 copy of a bf16 state stays small
        old = before[b:b + 8].float()
        out_t[b:b + 8] = torch.einsum("bhnd,bhn->bhd", old, q[b:b + 8])
        new = old + q[b:b + 8, :, :, None] * v[b:b + 8, None, 0, None, :]
        worst = max(worst, float((rho[b:b + 8].float() - new).abs().max()) / float(new.abs().max()))
    assert rel_err(out[:, :, 0].cpu().numpy(), out_t.cpu().numpy()) < tol
    assert worst < tol
