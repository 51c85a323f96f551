"""GPU parity of bdh_prefill_chunked_ex: the bf16 matrix-core prefill for PoPE and ALiBi (recurrent semantics,
src/model/bdh.rs:288-302) and the row-normalised form of kernel::linear_attention::fused_state_aligned
(src/kernel/linear_attention.rs:11-115), through the C ABI, against the CPU oracle on the bf16-rounded inputs.
Tolerance class of the bf16 forms: 2e-2 of the output's max-norm (Q, the scores and the state copy that enters a
product are rounded to bf16 once; accumulation is f32)."""
import numpy as np
import pytest
import torch

from oracle import bdh_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-2


@pytest.fixture(scope="module")
def bda():
    if not torch.cuda.is_available():
        pytest.fail("no HIP device: the GPU tests must run on the MI355X box")
    import burn_dragon_amd

    return burn_dragon_amd


def rel_err(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def _case(seed, B, h, T, N, d, nq, rho0_scale, relu=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((B, h, T, N), generator=g)
    if relu:
        x = torch.relu(x - 0.5)
    x = x.to(torch.bfloat16)
    v = torch.randn((B, T, d), generator=g).to(torch.bfloat16)
    rho0 = (rho0_scale * torch.randn((B, h, nq, d), generator=g)).float()
    return x, v, rho0


ROT = {"rope": orc.ROPE, "alibi": orc.ALIBI, "pope": orc.POPE}


@pytest.mark.parametrize("rotary", ["pope", "alibi"])
@pytest.mark.parametrize("T,N,d,rho0_scale,position,chunk", [
    (70, 24, 40, 0.05, 5, 0),        # ragged against every tile
    (300, 264, 72, 0.0, 0, 0),       # fresh state, two score tiles
    (512, 256, 256, 0.05, 33, 0),    # full tiles: operands straight from global memory into LDS
    (600, 128, 64, 0.05, 9, 256),    # three passes: the state (and its decay) carried between them
])
def test_recurrent_prefill_pope_and_alibi(bda, corc, rotary, T, N, d, rho0_scale, position, chunk):
    """Oracle = the sequential loop of src/model/bdh.rs:288-302 (PoPE rotation of attention.rs:323-330; ALiBi decay of
    :299-301 with the reference's default slopes)."""
    from burn_dragon_amd.recurrent import prefill_chunked_ex

    B, h = 2, 3
    rot = ROT[rotary]
    nq = 2 * N if rotary == "pope" else N
    x, v, rho0 = _case(T + N, B, h, T, N, d, nq, rho0_scale)
    freqs = corc.build_freqs(N, rotary=rot)
    slopes = corc.default_alibi_slopes(h) if rotary == "alibi" else None
    q = corc.rotate(x.float().numpy(), freqs, rot, position)
    decay = None if slopes is None else corc.alibi_decay(slopes)
    out_ref, rho_ref = corc.recurrent_attention(q, v.float().numpy(), rho0.numpy(), decay=decay)
    rho = rho0.clone().to(DEV)
    out = prefill_chunked_ex(x.to(DEV), v.to(DEV), rho, torch.from_numpy(freqs).to(DEV), position,
                             rotary=bda.RotaryEmbedding.parse(rotary), alibi_slopes=slopes,
                             state_is_zero=(rho0_scale == 0.0), chunk=chunk)
    torch.cuda.synchronize()
    assert rel_err(out.cpu().numpy(), out_ref) < TOL
    assert rel_err(rho.cpu().numpy(), rho_ref) < TOL
    if rho0_scale == 0.0:
        assert not out[:, :, 0].any()  # token 0 reads only the initial state


def test_alibi_prefill_custom_slopes_then_decode_steps(bda, corc):
    """Caller-given slopes; and the state the call leaves continues under the eager ALiBi decode step
    (bdh_recurrent_attention) like the oracle's token loop over prompt + steps."""
    from burn_dragon_amd.recurrent import prefill_chunked_ex, recurrent_attention

    B, h, T, N, d, steps = 2, 4, 200, 64, 48, 6
    x, v, rho0 = _case(11, B, h, T + steps, N, d, N, 0.0)
    slopes = np.array([0.9, 0.3, 0.05, 0.0], np.float32)
    zeros = np.zeros(N, np.float32)
    out_ref, rho_ref = corc.recurrent_attention(x.float().numpy(), v.float().numpy(), rho0.numpy(),
                                                decay=corc.alibi_decay(slopes))
    rho = rho0.clone().to(DEV)
    out_p = prefill_chunked_ex(x[:, :, :T].contiguous().to(DEV), v[:, :T].contiguous().to(DEV), rho, None, 0,
                               rotary=bda.RotaryEmbedding.ALIBI, alibi_slopes=slopes, state_is_zero=True)
    out_d = recurrent_attention(x[:, :, T:].float().contiguous().to(DEV), v[:, T:].float().contiguous().to(DEV), rho,
                                torch.from_numpy(zeros).to(DEV), T, bda.RotaryEmbedding.ALIBI, alibi_slopes=slopes)
    torch.cuda.synchronize()
    assert rel_err(out_p.cpu().numpy(), out_ref[:, :, :T]) < TOL
    assert rel_err(out_d.cpu().numpy(), out_ref[:, :, T:]) < TOL
    assert rel_err(rho.cpu().numpy(), rho_ref) < TOL


def test_rope_through_the_extended_entry_point_is_the_plain_call(bda, corc):
    """rotary = RoPE without row normalisation is bdh_prefill_chunked, bit for bit (chunk-recurrent form included)."""
    from burn_dragon_amd.recurrent import prefill_chunked, prefill_chunked_ex

    B, h, T, N, d = 2, 2, 520, 256, 256
    x, v, rho0 = _case(3, B, h, T, N, d, N, 0.05)
    ft = torch.from_numpy(corc.build_freqs(N)).to(DEV)
    rho_a, rho_b = rho0.clone().to(DEV), rho0.clone().to(DEV)
    out_a = prefill_chunked(x.to(DEV), v.to(DEV), rho_a, ft, 7)
    out_b = prefill_chunked_ex(x.to(DEV), v.to(DEV), rho_b, ft, 7, rotary=bda.RotaryEmbedding.ROPE)
    torch.cuda.synchronize()
    assert torch.equal(out_a, out_b) and torch.equal(rho_a, rho_b)


@pytest.mark.parametrize("rotary,seed", [("rope", 1337), ("pope", 2024)])
def test_row_normalised_reference_recipes(bda, corc, rotary, seed):
    """tests/fused_kernel_tests.rs:70-170 on the bf16 path: B=1, h=2, T=6, N=8, dv=6, BlockPattern2d::dense(3);
    fused == dense tril(-1) + row-normalise.  The reference compares f32 paths at 1e-4; this path rounds Q and the
    scores to bf16: 2e-2."""
    from burn_dragon_amd.recurrent import prefill_chunked_ex

    rot = ROT[rotary]
    g = torch.Generator().manual_seed(seed)
    query = torch.randn((1, 2, 6, 8), generator=g).to(torch.bfloat16)
    value = torch.randn((1, 6, 6), generator=g).to(torch.bfloat16)
    freqs = corc.build_freqs(8, rotary=rot)
    got = prefill_chunked_ex(query.to(DEV), value.to(DEV), None, torch.from_numpy(freqs).to(DEV), 0,
                             rotary=bda.RotaryEmbedding.parse(rotary), row_normalize=True, block_size=3)
    torch.cuda.synchronize()
    q = orc.rotate(query.double().numpy(), freqs.astype(np.float64), rot, 0)
    scores = np.tril(q @ np.swapaxes(q, 2, 3), -1)
    scores = scores / (np.abs(scores).sum(3, keepdims=True) + 1e-6)
    reference = scores @ value.double().numpy()[:, None]
    assert rel_err(got.cpu().numpy(), reference) < TOL
    ref_c = corc.fused_state_aligned(query.float().numpy(), value.float().numpy(), freqs, None, 3, rot)
    assert rel_err(got.cpu().numpy(), ref_c) < TOL


@pytest.mark.parametrize("rotary", ["rope", "alibi", "pope"])
@pytest.mark.parametrize("T,N,dv,bs", [(300, 200, 70, 48),    # time blocks straddle the 256-wide score tiles
                                       (520, 64, 40, 64),     # time blocks aligned with them
                                       (512, 256, 256, 128)]) # full tiles
def test_row_normalised_medium_shapes(bda, corc, rotary, T, N, dv, bs):
    """Against the oracle's blocked form (src/kernel/linear_attention.rs:54-112): ALiBi adds slope * (s - t) to whole
    time blocks, the diagonal one included."""
    from burn_dragon_amd.recurrent import prefill_chunked_ex

    B, h = 2, 3
    rot = ROT[rotary]
    x, v, _ = _case(T + bs, B, h, T, N, dv, N, 0.0)
    slopes = corc.default_alibi_slopes(h) if rotary == "alibi" else None
    freqs = corc.build_freqs(N, rotary=rot)
    got = prefill_chunked_ex(x.to(DEV), v.to(DEV), None, torch.from_numpy(freqs).to(DEV), 0,
                             rotary=bda.RotaryEmbedding.parse(rotary), alibi_slopes=slopes, row_normalize=True,
                             block_size=bs)
    torch.cuda.synchronize()
    ref = corc.fused_state_aligned(x.float().numpy(), v.float().numpy(), freqs, slopes, bs, rot)
    assert rel_err(got.cpu().numpy(), ref) < TOL


def test_row_normalised_matches_the_f32_entry_point_at_a_long_sequence(bda, corc):
    """T = 1100 with 16 slices, ragged against the tiles and the time block of 100: the bf16 form against
    bdh_fused_state_aligned (f32 on the same bf16-rounded inputs), RoPE and ALiBi."""
    from burn_dragon_amd.kernel import linear_attention
    from burn_dragon_amd.recurrent import prefill_chunked_ex

    B, h, T, N, dv, bs = 4, 4, 1100, 64, 40, 100
    x, v, _ = _case(9, B, h, T, N, dv, N, 0.0)
    for rotary, rot in (("rope", orc.ROPE), ("alibi", orc.ALIBI)):
        slopes = corc.default_alibi_slopes(h) if rotary == "alibi" else None
        freqs = torch.from_numpy(corc.build_freqs(N, rotary=rot))
        want = linear_attention.fused_state_aligned(x.float().to(DEV), v.float()[:, None].to(DEV), freqs,
                                                    None if slopes is None else torch.from_numpy(slopes),
                                                    bda.BlockPattern2d.dense(bs), bda.RotaryEmbedding.parse(rotary))
        got = prefill_chunked_ex(x.to(DEV), v.to(DEV), None, freqs.to(DEV), 0, rotary=bda.RotaryEmbedding.parse(rotary),
                                 alibi_slopes=slopes, row_normalize=True, block_size=bs)
        torch.cuda.synchronize()
        assert rel_err(got.cpu().numpy(), want.cpu().numpy()) < TOL


def test_extended_prefill_contract_errors(bda):
    from burn_dragon_amd import ffi
    from burn_dragon_amd.recurrent import prefill_chunked_ex

    x = torch.zeros((1, 2, 8, 16), dtype=torch.bfloat16, device=DEV)
    v = torch.zeros((1, 8, 8), dtype=torch.bfloat16, device=DEV)
    ft = torch.zeros(16, device=DEV)
    ctx = ffi.default_context(0)
    out = torch.empty((1, 2, 8, 8), device=DEV)
    call = lambda rotary, flags, rho, h=2: ctx.lib.bdh_prefill_chunked_ex(
        ctx.handle, 1, h, 8, 16, 8, rotary, ffi.ptr(x), ffi.ptr(v), ffi.ptr(ft), None, 0, 0, flags, 1, rho, ffi.ptr(out))
    assert call(7, 0, None) == -1                       # unknown rotary mode
    assert call(0, 16, None) == -1                      # unknown flag bit
    assert call(1, 0, None) == -1                       # a recurrent call needs rho
    assert call(1, ffi.PREFILL_ROW_NORMALIZE, None) == 0  # the row-normalised form does not
    with pytest.raises(AssertionError):                 # PoPE state has 2N rows
        prefill_chunked_ex(x, v, torch.zeros((1, 2, 16, 8), device=DEV), ft, 0, rotary=bda.RotaryEmbedding.POPE)


# ------------------------------------------------- the option that routes prompt calls to the bf16 form
@pytest.fixture
def prompt_bf16(bda):
    from burn_dragon_amd import ffi

    ctx = ffi.default_context(0)
    ctx.set_option("state_step.prompt_bf16", 64)
    yield ctx
    ctx.set_option("state_step.prompt_bf16", 0)


@pytest.mark.parametrize("rotary", ["rope", "alibi", "pope"])
def test_recurrent_attention_takes_the_bf16_form_when_asked(bda, corc, prompt_bf16, rotary):
    """bdh_recurrent_attention with "state_step.prompt_bf16": f32 inputs, rounded to bf16 inside; against the oracle's
    token loop on the f32 inputs at the bf16 tolerance, and different from the default f32 path (so the option took)."""
    from burn_dragon_amd.recurrent import recurrent_attention

    B, h, T, N, d = 2, 3, 200, 128, 72
    rot = ROT[rotary]
    nq = 2 * N if rotary == "pope" else N
    g = torch.Generator().manual_seed(21)
    x = torch.relu(torch.randn((B, h, T, N), generator=g) - 0.5)
    v = torch.randn((B, T, d), generator=g)
    rho0 = 0.05 * torch.randn((B, h, nq, d), generator=g)
    freqs = corc.build_freqs(N, rotary=rot)
    slopes = corc.default_alibi_slopes(h) if rotary == "alibi" else None
    decay = None if slopes is None else corc.alibi_decay(slopes)
    out_ref, rho_ref = corc.recurrent_attention(corc.rotate(x.numpy(), freqs, rot, 40), v.numpy(), rho0.numpy(),
                                                decay=decay)
    ft = torch.from_numpy(freqs).to(DEV)
    rho = rho0.clone().to(DEV)
    out = recurrent_attention(x.to(DEV), v.to(DEV), rho, ft, 40, bda.RotaryEmbedding.parse(rotary), alibi_slopes=slopes)
    prompt_bf16.set_option("state_step.prompt_bf16", 0)
    rho32 = rho0.clone().to(DEV)
    out32 = recurrent_attention(x.to(DEV), v.to(DEV), rho32, ft, 40, bda.RotaryEmbedding.parse(rotary),
                                alibi_slopes=slopes)
    torch.cuda.synchronize()
    assert rel_err(out.cpu().numpy(), out_ref) < TOL and rel_err(rho.cpu().numpy(), rho_ref) < TOL
    assert rel_err(out32.cpu().numpy(), out_ref) < 1e-3
    assert not torch.equal(out, out32)


@pytest.mark.parametrize("lazy", [False, True], ids=["eager-decay", "lazy-decay"])
def test_trained_checkpoint_prompt_on_the_bf16_form(bda, corc, prompt_bf16, lazy):
    """The reference's trained ALiBi checkpoint (tests/golden/tiny_shakespeare): a 160-character prompt through
    forward_with_state with the state path of every layer on the bf16 matrix cores, then greedy decode steps on the
    state it left.  Logits against the oracle at the bf16 tolerance; the model still predicts the text."""
    import os

    from burn_dragon_amd import record

    ckpt = os.path.join(os.path.dirname(__file__), "golden", "tiny_shakespeare")
    text = ("First Citizen:\nBefore we proceed any further, hear me speak.\n\nAll:\nSpeak, speak.\n\n"
            "First Citizen:\nYou are all resolved rather to die than to famish?\n\nAll:\nResolved. resolved.\n")
    model, tok, _ = bda.BDH.from_checkpoint_dir(ckpt, DEV, alibi_lazy=lazy)
    _, weights, _, _ = record.load_checkpoint_dir(ckpt)
    shape = orc.BDHShape(n_layer=4, n_embd=128, n_head=4, mlp_internal_dim_multiplier=4, vocab_size=69, rotary=orc.ALIBI)
    w = orc.BDHWeights(**weights)
    ids = np.array([tok.encode(text)])
    n_prompt = 160
    assert ids.shape[1] > n_prompt + 4
    state = model.init_state()
    logits = model.forward_with_state(torch.from_numpy(ids[:, :n_prompt]), state).cpu().numpy()
    rho_ref = np.zeros((4, 1, 4, 128, 128), np.float32)
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, ids[:, :n_prompt], rho_ref, 0, sparse_state=False)
    assert rel_err(logits, logits_ref) < TOL
    z = logits[0].astype(np.float64)
    logp = z - z.max(-1, keepdims=True)
    logp -= np.log(np.exp(logp).sum(-1, keepdims=True))
    loss = float(-logp[np.arange(n_prompt - 1), ids[0, 1:n_prompt]].mean())
    assert loss < 1.4, loss  # uniform would be ln 69 = 4.23
    # decode steps (single tokens: the f32 step kernels) continue from the state the bf16 prompt left
    for t in range(n_prompt, n_prompt + 4):
        step = model.forward_with_state(torch.from_numpy(ids[:, t:t + 1]), state).cpu().numpy()
        step_ref, pos, _, _ = corc.forward_with_state(shape, w, ids[:, t:t + 1], rho_ref, pos, sparse_state=False)
        assert rel_err(step, step_ref) < TOL
    model.materialize_state(state)
    assert rel_err(state.storage.cpu().numpy(), rho_ref) < TOL and state.position == pos


@pytest.mark.parametrize("mode", ["alibi-recurrent", "rope-rownorm", "alibi-rownorm"])
def test_extended_prefill_at_the_config3_size(bda, corc, mode):
    """BASELINE config 3's shape (B=8, h=4, T=2048, N=8192, d=256, 5 % density) through bdh_prefill_chunked_ex, checked
    without the oracle's loops (too slow at this size):
      ALiBi, recurrent: token 0 reads a zero state; the final state is sum_s g^(T-s) q_s (x) v_s (src/model/bdh.rs:298-301
        summed over the tokens) by a device einsum per batch entry; out of one slice against the closed causal form with
        the decay powers; slices (b=0, h=0..1) hold the bits of a B=1, h=2 call with those heads' slopes.
      row-normalised: |out[t]| <= max|v| (a quotient of sum s_i v_i by sum |s_i|); one slice against the closed form
        on the device; slices hold the bits of the reduced call."""
    from burn_dragon_amd.recurrent import prefill_chunked_ex

    B, h, T, N, d, bs = 8, 4, 2048, 8192, 256, 64
    g = torch.Generator().manual_seed(17)
    x = torch.empty((B, h, T, N), dtype=torch.bfloat16)
    for b in range(B):
        x[b] = torch.relu(torch.randn((h, T, N), generator=g) - 1.6449).to(torch.bfloat16)
    v = torch.randn((B, T, d), generator=g).to(torch.bfloat16)
    xt, vt = x.to(DEV), v.to(DEV)
    slopes = corc.default_alibi_slopes(h)
    pos = torch.arange(T, device=DEV, dtype=torch.float32)
    print(f"extended prefill at the config-3 size: {mode}", flush=True)
    if mode == "alibi-recurrent":
        rho = torch.zeros((B, h, N, d), device=DEV)
        out = prefill_chunked_ex(xt, vt, rho, None, 0, rotary=bda.RotaryEmbedding.ALIBI, alibi_slopes=slopes,
                                 state_is_zero=True)
        torch.cuda.synchronize()
        assert not out[:, :, 0].any()
        logd = torch.log(torch.exp(-torch.from_numpy(slopes))).to(DEV)  # log of the rounded per-token factor
        for b in range(B):
            q = xt[b].float()  # [h,T,N]; ALiBi does not rotate
            w = torch.exp((T - pos)[None, :] * logd[:, None])  # [h,T]: g^(T-s)
            ref = torch.einsum("htn,ht,td->hnd", q, w, vt[b].float())
            err = float((rho[b] - ref).abs().max()) / float(ref.abs().max())
            assert err < TOL, f"batch entry {b}: {err}"
        q0 = xt[0, 1].float()
        dec = torch.exp((pos[:, None] - pos[None, :]).clamp(min=0) * logd[1])
        o = (torch.tril(q0 @ q0.T, -1) * dec) @ vt[0].float()
        assert float((out[0, 1] - o).abs().max()) / float(o.abs().max()) < TOL
        rho2 = torch.zeros((1, 2, N, d), device=DEV)
        out2 = prefill_chunked_ex(xt[:1, :2].contiguous(), vt[:1].contiguous(), rho2, None, 0,
                                  rotary=bda.RotaryEmbedding.ALIBI, alibi_slopes=slopes[:2], state_is_zero=True)
        torch.cuda.synchronize()
        assert torch.equal(out2[0], out[0, :2]) and torch.equal(rho2[0], rho[0, :2])
        return
    rot = bda.RotaryEmbedding.ROPE if mode == "rope-rownorm" else bda.RotaryEmbedding.ALIBI
    freqs = corc.build_freqs(N, rotary=orc.ROPE if mode == "rope-rownorm" else orc.ALIBI)
    ft = torch.from_numpy(freqs).to(DEV)
    sl = slopes if mode == "alibi-rownorm" else None
    out = prefill_chunked_ex(xt, vt, None, ft, 0, rotary=rot, alibi_slopes=sl, row_normalize=True, block_size=bs)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    assert float(out.abs().max()) <= float(vt.float().abs().max()) * (1 + 1e-3)
    hh = 2
    if mode == "rope-rownorm":
        q0 = torch.from_numpy(corc.rotate(x[0:1, hh:hh + 1].float().numpy(), freqs, orc.ROPE, 0)).to(DEV)[0, 0]
        q0 = q0.to(torch.bfloat16).float()
    else:
        q0 = xt[0, hh].float()
    s = torch.tril(q0 @ q0.T, -1)
    if sl is not None:  # the additive term on whole causal time blocks (the diagonal block included)
        blk = (torch.arange(T, device=DEV) // bs)
        s = s + float(sl[hh]) * (pos[None, :] - pos[:, None]) * (blk[None, :] <= blk[:, None])
    s = s.to(torch.bfloat16).float()
    o = (s @ vt[0].float()) / (s.abs().sum(1, keepdim=True) + 1e-6)
    assert float((out[0, hh] - o).abs().max()) / float(o.abs().max()) < TOL
    out2 = prefill_chunked_ex(xt[:1, :2].contiguous(), vt[:1].contiguous(), None, ft, 0, rotary=rot,
                              alibi_slopes=None if sl is None else sl[:2], row_normalize=True, block_size=bs)
    torch.cuda.synchronize()
    assert torch.equal(out2[0], out[0, :2])


def test_extended_prefill_edge_shapes(bda, corc):
    """One token, an empty batch, a latent that is not a multiple of 8, more heads than slopes can travel with."""
    from burn_dragon_amd import ffi
    from burn_dragon_amd.recurrent import prefill_chunked_ex

    ctx = ffi.default_context(0)
    # T = 1: the readout of the carried state alone, then one decayed update
    B, h, N, d = 2, 2, 16, 24
    g = torch.Generator().manual_seed(5)
    x = torch.relu(torch.randn((B, h, 1, N), generator=g)).to(torch.bfloat16)
    v = torch.randn((B, 1, d), generator=g).to(torch.bfloat16)
    rho0 = (0.1 * torch.randn((B, h, N, d), generator=g)).float()
    slopes = np.array([0.7, 0.2], np.float32)
    out_ref, rho_ref = corc.recurrent_attention(x.float().numpy(), v.float().numpy(), rho0.numpy(),
                                                decay=corc.alibi_decay(slopes))
    rho = rho0.clone().to(DEV)
    out = prefill_chunked_ex(x.to(DEV), v.to(DEV), rho, None, 3, rotary=bda.RotaryEmbedding.ALIBI, alibi_slopes=slopes)
    torch.cuda.synchronize()
    assert rel_err(out.cpu().numpy(), out_ref) < TOL and rel_err(rho.cpu().numpy(), rho_ref) < TOL
    # an empty batch is a no-op
    e = torch.zeros((0, h, 4, N), dtype=torch.bfloat16, device=DEV)
    assert prefill_chunked_ex(e, torch.zeros((0, 4, d), dtype=torch.bfloat16, device=DEV),
                              torch.zeros((0, h, N, d), device=DEV), None, 0, rotary=bda.RotaryEmbedding.ALIBI).shape == (0, h, 4, d)
    # N must be a multiple of 8 (x is read in 16-byte pieces)
    xb = torch.zeros((1, 1, 4, 12), dtype=torch.bfloat16, device=DEV)
    vb = torch.zeros((1, 4, 8), dtype=torch.bfloat16, device=DEV)
    ob = torch.empty((1, 1, 4, 8), device=DEV)
    rb = torch.zeros((1, 1, 12, 8), device=DEV)
    rc = ctx.lib.bdh_prefill_chunked_ex(ctx.handle, 1, 1, 4, 12, 8, int(bda.RotaryEmbedding.ALIBI), ffi.ptr(xb), ffi.ptr(vb),
                                        None, None, 0, 0, 0, 1, ffi.ptr(rb), ffi.ptr(ob))
    assert rc == ffi.E_SHAPE
    # more than 64 heads cannot carry per-head slopes in the kernel arguments
    xh = torch.zeros((1, 65, 2, 8), dtype=torch.bfloat16, device=DEV)
    vh = torch.zeros((1, 2, 8), dtype=torch.bfloat16, device=DEV)
    oh = torch.empty((1, 65, 2, 8), device=DEV)
    rh = torch.zeros((1, 65, 8, 8), device=DEV)
    rc = ctx.lib.bdh_prefill_chunked_ex(ctx.handle, 1, 65, 2, 8, 8, int(bda.RotaryEmbedding.ALIBI), ffi.ptr(xh), ffi.ptr(vh),
                                        None, None, 0, 0, 0, 1, ffi.ptr(rh), ffi.ptr(oh))
    assert rc == ffi.E_SHAPE
    # PoPE and RoPE with that many heads are fine (no per-head parameters)
    fq = torch.from_numpy(corc.build_freqs(8, rotary=orc.POPE)).to(DEV)
    rp = torch.zeros((1, 65, 16, 8), device=DEV)
    rc = ctx.lib.bdh_prefill_chunked_ex(ctx.handle, 1, 65, 2, 8, 8, int(bda.RotaryEmbedding.POPE), ffi.ptr(xh), ffi.ptr(vh),
                                        ffi.ptr(fq), None, 0, 0, 0, 1, ffi.ptr(rp), ffi.ptr(oh))
    assert rc == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("rotary", ["rope", "alibi", "pope"])
def test_fused_state_aligned_takes_the_bf16_form_when_asked(bda, corc, rotary):
    """bdh_fused_state_aligned with "fused_state_aligned.path" = 2 (dense pattern, row-normalised): against the oracle's
    blocked form at the bf16 tolerance, and a sparse pattern under the same option still takes the f32 path (1e-3)."""
    from burn_dragon_amd import ffi
    from burn_dragon_amd.kernel import linear_attention

    B, h, T, N, dv, bs = 2, 3, 300, 200, 72, 64
    rot = ROT[rotary]
    rng = np.random.default_rng(8)
    query = np.maximum(rng.standard_normal((B, h, T, N)) - 0.5, 0).astype(np.float32)
    value = rng.standard_normal((B, T, dv)).astype(np.float32)
    slopes = corc.default_alibi_slopes(h) if rotary == "alibi" else None
    freqs = corc.build_freqs(N, rotary=rot)
    qt, vt = torch.from_numpy(query).to(DEV), torch.from_numpy(value[:, None]).to(DEV)
    st = None if slopes is None else torch.from_numpy(slopes)
    ctx = ffi.default_context(0)
    ctx.set_option("fused_state_aligned.path", 2)
    try:
        got = linear_attention.fused_state_aligned(qt, vt, torch.from_numpy(freqs), st, bda.BlockPattern2d.dense(bs),
                                                   bda.RotaryEmbedding.parse(rotary))
        tb = (T + bs - 1) // bs
        pairs = {(r, c) for r in range(tb) for c in range(r + 1) if (r + c) % 2 == 0}
        got_sparse = linear_attention.fused_state_aligned(qt, vt, torch.from_numpy(freqs), st,
                                                          bda.BlockPattern2d.from_pairs(bs, pairs),
                                                          bda.RotaryEmbedding.parse(rotary))
    finally:
        ctx.set_option("fused_state_aligned.path", -1)
    exact = linear_attention.fused_state_aligned(qt, vt, torch.from_numpy(freqs), st, bda.BlockPattern2d.dense(bs),
                                                 bda.RotaryEmbedding.parse(rotary))
    torch.cuda.synchronize()
    ref = corc.fused_state_aligned(query, value, freqs, slopes, bs, rot)
    assert rel_err(got.cpu().numpy(), ref) < TOL
    assert rel_err(exact.cpu().numpy(), ref) < 1e-3
    assert not torch.equal(got, exact)  # the option took
    ref_sparse = corc.fused_state_aligned(query, value, freqs, slopes, bs, rot, pairs=pairs)
    assert rel_err(got_sparse.cpu().numpy(), ref_sparse) < 1e-3
