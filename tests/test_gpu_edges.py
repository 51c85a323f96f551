"""Edge cases of the C ABI on the GPU: empty and ragged shapes, the size limits, positions beyond the
exact-integer range of f32, a bf16-state model, degenerate rows.  Values against the CPU oracle
(f32 state 1e-3, bf16 state 2e-2, index artefacts bit-exact)."""
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


def test_empty_shapes_are_no_ops(bda):
    from burn_dragon_amd import ffi
    from burn_dragon_amd.kernel import BlockPattern1d
    from burn_dragon_amd.kernel.relu_lowrank import fused_forward
    from burn_dragon_amd.recurrent import layer_norm, recurrent_attention

    z = lambda *s: torch.zeros(s, device=DEV)
    out = recurrent_attention(z(0, 2, 1, 64), z(0, 1, 32), z(0, 2, 64, 32), z(64), 0)
    assert tuple(out.shape) == (0, 2, 1, 32)
    out = recurrent_attention(z(2, 2, 0, 64), z(2, 0, 32), z(2, 2, 64, 32), z(64), 0)
    assert tuple(out.shape) == (2, 2, 0, 32)
    assert tuple(fused_forward(z(0, 1, 3, 8), z(2, 8, 16), None, 0.0, BlockPattern1d.dense(4)).shape) == (0, 2, 3, 16)
    assert tuple(layer_norm(z(0, 16)).shape) == (0, 16)
    cfg = bda.BDHConfig(n_layer=1, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=8)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    model = bda.BDH(cfg, DEV, seed=1)
    st = model.init_state()
    assert tuple(model.forward_with_state(torch.zeros((2, 0), dtype=torch.int64), st).shape) == (2, 0, 8)
    assert st.position == 0
    ctx = ffi.default_context(0)
    assert ctx.lib.bdh_sample_top_k(ctx.handle, 0, 8, None, 8, 1.0, 0, None, None) == ffi.OK
    assert ctx.lib.bdh_alibi_materialize(ctx.handle, 0, 2, 8, 4, 0, None, None, None, ffi.F32, None) == ffi.OK
    torch.cuda.synchronize()


def test_zero_latent_gives_a_zero_readout(bda):
    from burn_dragon_amd.recurrent import recurrent_attention

    out = recurrent_attention(torch.zeros((2, 2, 1, 0), device=DEV), torch.ones((2, 1, 8), device=DEV),
                              torch.zeros((2, 2, 0, 8), device=DEV), torch.zeros(0, device=DEV), 3)
    torch.cuda.synchronize()
    assert tuple(out.shape) == (2, 2, 1, 8) and float(out.abs().max()) == 0.0


def test_size_limits(bda, corc):
    from burn_dragon_amd import ffi
    from burn_dragon_amd.recurrent import recurrent_attention

    rng = np.random.default_rng(0)
    # d = 1024 is the widest state row; h = 64 the most heads
    for B, h, N, d in [(1, 1, 64, 1024), (1, 64, 16, 8)]:
        x = np.maximum(rng.standard_normal((B, h, 1, N)), 0).astype(np.float32)
        v = rng.standard_normal((B, 1, d)).astype(np.float32)
        rho = (0.1 * rng.standard_normal((B, h, N, d))).astype(np.float32)
        freqs = corc.build_freqs(N)
        rt = torch.from_numpy(rho).to(DEV)
        out = recurrent_attention(torch.from_numpy(x).to(DEV), torch.from_numpy(v).to(DEV), rt,
                                  torch.from_numpy(freqs).to(DEV), 5)
        o_ref, r_ref = corc.recurrent_attention(corc.rotate(x, freqs, orc.ROPE, 5), v, rho)
        assert rel_err(out.cpu().numpy(), o_ref) < 1e-3 and rel_err(rt.cpu().numpy(), r_ref) < 1e-3
    ctx = ffi.default_context(0)
    t = torch.zeros(1 << 16, device=DEV)
    p = t.data_ptr()
    assert ctx.lib.bdh_state_step(ctx.handle, 1, 1, 4, 1028, ffi.ROPE, p, p, p, 0, None, None, p, ffi.F32, p, None,
                                  None) == ffi.E_SHAPE
    assert ctx.lib.bdh_state_step(ctx.handle, 1, 65, 4, 4, ffi.ROPE, p, p, p, 0, None, None, p, ffi.F32, p, None,
                                  None) == ffi.E_SHAPE
    assert b"n_head" in ctx.lib.bdh_last_error(ctx.handle)


@pytest.mark.parametrize("position", [(1 << 24) + 1, (1 << 31) + 12345, (1 << 40) + 7])
def test_positions_beyond_the_exact_range_of_f32(bda, corc, position):
    """The reference converts the position to f32 before multiplying by the frequency
    (src/model/attention.rs:337-343): beyond 2^24 that rounds, and the device must round the same way."""
    from burn_dragon_amd.recurrent import recurrent_attention

    rng = np.random.default_rng(7)
    B, h, N, d = 2, 2, 256, 256
    x = np.maximum(rng.standard_normal((B, h, 1, N)) - 1.0, 0).astype(np.float32)
    v = rng.standard_normal((B, 1, d)).astype(np.float32)
    rho = (0.1 * rng.standard_normal((B, h, N, d))).astype(np.float32)
    freqs = corc.build_freqs(N)
    rt = torch.from_numpy(rho).to(DEV)
    out = recurrent_attention(torch.from_numpy(x).to(DEV), torch.from_numpy(v).to(DEV), rt,
                              torch.from_numpy(freqs).to(DEV), position)
    o_ref, r_ref = corc.recurrent_attention(corc.rotate(x, freqs, orc.ROPE, position), v, rho)
    assert rel_err(out.cpu().numpy(), o_ref) < 1e-3 and rel_err(rt.cpu().numpy(), r_ref) < 1e-3


@pytest.mark.parametrize("B,h_in,T,d,h,N", [(1, 1, 1, 4, 1, 1), (2, 3, 17, 20, 3, 77), (3, 1, 9, 256, 2, 130)])
def test_relu_lowrank_ragged_shapes_bias_mask_and_gate(bda, corc, B, h_in, T, d, h, N):
    from burn_dragon_amd.kernel import BlockPattern1d
    from burn_dragon_amd.kernel.relu_lowrank import fused_forward

    rng = np.random.default_rng(B * 100 + N)
    inp = rng.standard_normal((B, h_in, T, d)).astype(np.float32)
    w = rng.standard_normal((h, d, N)).astype(np.float32)
    bias = rng.standard_normal((h, 1, N)).astype(np.float32)
    bs = 5
    nblk = (N + bs - 1) // bs
    active = sorted(set(rng.integers(0, nblk, size=max(nblk // 2, 1)).tolist()))
    layout = BlockPattern1d.from_blocks(bs, active)
    out = fused_forward(torch.from_numpy(inp).to(DEV), torch.from_numpy(w).to(DEV), torch.from_numpy(bias).to(DEV),
                        0.3, layout)
    ref = corc.relu_lowrank(inp, w, bias, 0.3, bs, active)
    assert np.array_equal(out.cpu().numpy(), ref)  # one k-sequential chain per output: bit-exact
    gate = np.maximum(rng.standard_normal((B, h, T, N)), 0).astype(np.float32)
    gated = fused_forward(torch.from_numpy(inp).to(DEV), torch.from_numpy(w).to(DEV), None, 0.0,
                          BlockPattern1d.dense(4), gate=torch.from_numpy(gate).to(DEV))
    assert np.array_equal(gated.cpu().numpy(), corc.relu_lowrank(inp, w, None, 0.0) * gate)


def test_layer_norm_degenerate_rows(bda, corc):
    from burn_dragon_amd.recurrent import layer_norm

    x = np.zeros((4, 33), np.float32)
    x[1] = 7.5  # constant row: variance 0 -> (x - mean) / sqrt(eps) = 0
    x[2, 5] = 1e20
    x[3] = np.linspace(-1, 1, 33)
    out = layer_norm(torch.from_numpy(x).to(DEV)).cpu().numpy()
    assert np.array_equal(out[:2], np.zeros((2, 33), np.float32))
    ref = corc.layer_norm(x)
    assert np.array_equal(np.isfinite(out), np.isfinite(ref))
    assert np.array_equal(out[3], ref[3])
    one = layer_norm(torch.full((3, 1), 2.0, device=DEV)).cpu().numpy()
    assert np.array_equal(one, np.zeros((3, 1), np.float32))  # d = 1: every row is constant


def test_smallest_model_and_argmax_ties(bda, corc):
    cfg = bda.BDHConfig(n_layer=1, n_embd=4, n_head=1, mlp_internal_dim_multiplier=1, vocab_size=1)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    model = bda.BDH(cfg, DEV, seed=3)
    logits, nxt = model.forward_with_state(torch.zeros((1, 1), dtype=torch.int64), model.init_state(), want_next=True)
    assert tuple(logits.shape) == (1, 1, 1) and int(nxt[0]) == 0
    # identical lm_head columns give identical logits: the argmax is the lowest index, as the oracle's
    cfg = bda.BDHConfig(n_layer=1, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=12)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    shape = orc.BDHShape(n_layer=1, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=12, rotary=orc.ROPE)
    w = orc.init_weights(shape, 4)
    w.lm_head[:, :] = w.lm_head[:, :1]
    model = bda.BDH(cfg, DEV, weights=vars(w))
    tokens = np.array([[3, 1, 4]])
    logits, nxt = model.forward_with_state(torch.from_numpy(tokens), model.init_state(), want_next=True)
    assert int(nxt[0]) == 0 == corc.greedy_token(logits[0, -1].cpu().numpy())


@pytest.mark.parametrize("rotary", ["rope", "alibi", "pope"])
def test_model_with_bf16_state(bda, corc, rotary):
    """bf16 storage of rho, f32 accumulate: logits within 2e-2 of the f32 oracle over a prompt and a few
    decode steps (north_star's tolerance for a bf16 state)."""
    from burn_dragon_amd import ffi

    cfg = bda.BDHConfig(n_layer=3, n_embd=256, n_head=4, mlp_internal_dim_multiplier=8, vocab_size=64)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.parse(rotary))
    rot = {"rope": orc.ROPE, "alibi": orc.ALIBI, "pope": orc.POPE}[rotary]
    shape = orc.BDHShape(n_layer=3, n_embd=256, n_head=4, mlp_internal_dim_multiplier=8, vocab_size=64, rotary=rot)
    w = orc.init_weights(shape, 13)
    model = bda.BDH(cfg, DEV, weights=vars(w), rho_dtype=ffi.BF16)
    tokens = np.random.default_rng(2).integers(0, 64, size=(2, 12))
    state = model.init_state()
    logits = model.forward_with_state(torch.from_numpy(tokens[:, :8]), state)
    assert state.storage.dtype == torch.bfloat16
    Nq = 512 * (2 if rotary == "pope" else 1)
    rho = np.zeros((3, 2, 4, Nq, 256), np.float32)
    ref, pos, _, _ = corc.forward_with_state(shape, w, tokens[:, :8], rho, 0, sparse_state=False)
    assert rel_err(logits.cpu().numpy(), ref) < 2e-2
    for t in range(8, 12):
        lg = model.forward_with_state(torch.from_numpy(tokens[:, t:t + 1]), state)
        ref, pos, _, _ = corc.forward_with_state(shape, w, tokens[:, t:t + 1], rho, pos, sparse_state=False)
        assert rel_err(lg.cpu().numpy(), ref) < 2e-2
    assert rel_err(state.storage.float().cpu().numpy(), rho) < 2e-2


def test_pope_step_at_the_config1_layer_shape(bda, corc):
    from burn_dragon_amd.recurrent import recurrent_attention

    rng = np.random.default_rng(11)
    B, h, N, d = 1, 4, 8192, 256
    x = rng.standard_normal((B, h, 1, N)).astype(np.float32)  # PoPE takes softplus(x): every row is active
    v = rng.standard_normal((B, 1, d)).astype(np.float32)
    rho = (0.01 * rng.standard_normal((B, h, 2 * N, d))).astype(np.float32)
    freqs = corc.build_freqs(N, rotary=orc.POPE)
    rt = torch.from_numpy(rho).to(DEV)
    out, rows = recurrent_attention(torch.from_numpy(x).to(DEV), torch.from_numpy(v).to(DEV), rt,
                                    torch.from_numpy(freqs).to(DEV), 777, bda.RotaryEmbedding.POPE, want_rows=True)
    o_ref, r_ref = corc.recurrent_attention(corc.rotate(x, freqs, orc.POPE, 777), v, rho)
    assert rel_err(out.cpu().numpy(), o_ref) < 1e-3 and rel_err(rt.cpu().numpy(), r_ref) < 1e-3
    assert (rows.cpu().numpy() == 2 * N).all()


def test_context_follows_torchs_current_stream(bda, corc):
    """The wrappers launch on whatever stream torch considers current: work queued on a side stream before the
    call (a large fill of the state) must be seen by the kernels, and the result must be ready for torch ops that
    follow on that stream, with no device-wide synchronisation in between."""
    from burn_dragon_amd import ffi
    from burn_dragon_amd.recurrent import recurrent_attention

    rng = np.random.default_rng(5)
    B, h, N, d = 8, 4, 2048, 256
    x = np.maximum(rng.standard_normal((B, h, 1, N)) - 1.0, 0).astype(np.float32)
    v = rng.standard_normal((B, 1, d)).astype(np.float32)
    freqs = corc.build_freqs(N)
    xt, vt, ft = (torch.from_numpy(a).to(DEV) for a in (x, v, freqs))
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=DEV)
    ctx = ffi.default_context(0)
    with torch.cuda.stream(side):
        junk = torch.empty((1 << 28,), device=DEV)
        for _ in range(4):  # a few milliseconds of fills queued ahead of the state's own fill
            junk.fill_(1.0)
        rho = torch.empty((B, h, N, d), device=DEV)
        rho.fill_(0.25)  # queued on the side stream, certainly not finished when the call below returns to the host
        out = recurrent_attention(xt, vt, rho, ft, 99, bda.RotaryEmbedding.ROPE)
        total = out.sum()  # torch op on the same stream, right behind the kernels
    assert ctx._stream == side.cuda_stream
    side.synchronize()
    q = corc.rotate(x, freqs, orc.ROPE, 99)
    out_ref, rho_ref = corc.recurrent_attention(q, v, np.full((B, h, N, d), 0.25, np.float32))
    assert rel_err(out.cpu().numpy(), out_ref) < 1e-3
    assert rel_err(rho.cpu().numpy(), rho_ref) < 1e-3
    assert abs(float(total) - float(out_ref.sum())) <= 1e-3 * np.abs(out_ref).sum()
    # back on the default stream the context follows again
    out2 = recurrent_attention(xt, vt, rho, ft, 100, bda.RotaryEmbedding.ROPE)
    torch.cuda.synchronize()
    assert ctx._stream == torch.cuda.current_stream(0).cuda_stream
    assert np.isfinite(out2.cpu().numpy()).all()


def test_context_rebind_orders_the_shared_workspace_between_streams(bda, corc):
    """Two calls through the default context on two different streams with no synchronisation in between: both use the
    context's one workspace (the prefill's rotated activations, state copies and value layouts), so the second stream
    must wait for the first stream's kernels at the re-bind.  Each call against the same call run alone."""
    from burn_dragon_amd import ffi
    from burn_dragon_amd.recurrent import prefill_chunked

    B, h, T, N, d = 2, 4, 1024, 2048, 256
    g = torch.Generator().manual_seed(3)
    cases = []
    for _ in range(2):
        x = torch.relu(torch.randn((B, h, T, N), generator=g) - 1.3).to(torch.bfloat16).to(DEV)
        v = torch.randn((B, T, d), generator=g).to(torch.bfloat16).to(DEV)
        cases.append((x, v))
    ft = torch.from_numpy(corc.build_freqs(N)).to(DEV)
    alone = []
    for x, v in cases:
        rho = torch.zeros((B, h, N, d), device=DEV)
        out = prefill_chunked(x, v, rho, ft, 0, state_is_zero=True)
        torch.cuda.synchronize()
        alone.append((out.clone(), rho.clone()))
    s1, s2 = torch.cuda.Stream(device=DEV), torch.cuda.Stream(device=DEV)
    rhos = [torch.zeros((B, h, N, d), device=DEV) for _ in range(2)]
    torch.cuda.synchronize()
    outs = []
    for _ in range(3):  # a few rounds: the calls of the two streams alternate back to back
        outs.clear()
        for rho in rhos:
            rho.zero_()
        torch.cuda.synchronize()
        for (x, v), rho, stream in zip(cases, rhos, (s1, s2)):
            with torch.cuda.stream(stream):
                outs.append(prefill_chunked(x, v, rho, ft, 0, state_is_zero=True))
        torch.cuda.synchronize()
        for (out, rho), (out_a, rho_a) in zip(zip(outs, rhos), alone):
            assert torch.equal(out, out_a) and torch.equal(rho, rho_a)
    assert ffi.default_context(0)._stream == s2.cuda_stream


def test_probe_chunks_moves_exactly_the_listed_chunks(bda):
    """bdh_probe_chunks (the decode step's memory traffic without its arithmetic): mode 0 reads the listed chunks,
    scales by 1 and writes them back -- the region is unchanged; mode 1 only reads; mode 2 writes zeros into the
    listed chunks and nowhere else; chunks outside the region are skipped; argument errors are reported."""
    from burn_dragon_amd import ffi

    ctx = ffi.default_context(0)
    lib = ctx.lib
    rng = np.random.default_rng(9)
    chunk_kib, n_region_chunks = 2, 4096  # an 8 MiB region
    region = torch.from_numpy(rng.standard_normal(n_region_chunks * chunk_kib * 256).astype(np.float32)).to(DEV)
    before = region.clone()
    listed = rng.choice(n_region_chunks, 400, replace=False).astype(np.int32)
    outside = np.array([n_region_chunks, n_region_chunks + 7, -1], np.int32)  # skipped
    index = torch.from_numpy(np.concatenate([listed, outside])).to(DEV)
    nbytes = region.numel() * 4
    for mode in (0, 1):
        ctx.check(lib.bdh_probe_chunks(ctx.handle, region.data_ptr(), nbytes, index.data_ptr(), index.numel(), chunk_kib,
                                       mode, 64))
        torch.cuda.synchronize()
        assert torch.equal(region, before)
    ctx.check(lib.bdh_probe_chunks(ctx.handle, region.data_ptr(), nbytes, index.data_ptr(), index.numel(), chunk_kib, 2, 64))
    torch.cuda.synchronize()
    got = region.view(n_region_chunks, -1)
    mask = torch.zeros(n_region_chunks, dtype=torch.bool, device=DEV)
    mask[torch.from_numpy(listed.astype(np.int64)).to(DEV)] = True
    assert not got[mask].any()
    assert torch.equal(got[~mask], before.view(n_region_chunks, -1)[~mask])
    # nothing listed: a no-op; bad arguments: an error code and a message, no launch
    assert lib.bdh_probe_chunks(ctx.handle, region.data_ptr(), nbytes, index.data_ptr(), 0, chunk_kib, 0, 64) == ffi.OK
    for bad in (dict(mode=3), dict(chunk_kib=0), dict(workgroups=0), dict(n=-1)):
        rc = lib.bdh_probe_chunks(ctx.handle, region.data_ptr(), nbytes, index.data_ptr(), bad.get("n", 4),
                                  bad.get("chunk_kib", chunk_kib), bad.get("mode", 0), bad.get("workgroups", 64))
        assert rc == ffi.E_INVAL, bad
    assert lib.bdh_probe_chunks(ctx.handle, region.data_ptr() + 4, nbytes - 4, index.data_ptr(), 4, chunk_kib, 0,
                                64) == ffi.E_ALIGN
