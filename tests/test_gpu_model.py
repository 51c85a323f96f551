"""GPU parity of the projections (relu_lowrank, layer_norm) and of the whole cached step
(BDH::forward_with_state) against the CPU oracle, through the C ABI.

Tolerance for logits: 1e-3 relative on the max-norm (north_star, f32 state).  Active-neuron
sets of the first layer are bit-exact against the oracle (both sides evaluate one k-sequential
f32 FMA chain per pre-activation); deeper layers inherit readout reassociation noise, so their
sets are compared away from zero pre-activations and the mismatch count is reported.
"""
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


def assert_close(lhs, rhs, atol, rtol):
    lhs, rhs = np.asarray(lhs, np.float64), np.asarray(rhs, np.float64)
    assert lhs.shape == rhs.shape
    assert not (np.abs(lhs - rhs) > atol + rtol * np.abs(rhs)).any(), f"max diff {np.abs(lhs - rhs).max()}"


def test_relu_lowrank_fused_matches_reference(bda):
    """tests/fused_kernel_tests.rs:35-68 on the device path: input [2,1,5,6], weight [1,3,6,8],
    bias [3,1,8], threshold 0.25, BlockPattern1d::from_blocks(3,[0,2]); atol = rtol = 1e-5."""
    from burn_dragon_amd.kernel import relu_lowrank

    g = torch.Generator().manual_seed(42)
    inp = torch.randn((2, 1, 5, 6), generator=g)
    weight = torch.randn((1, 3, 6, 8), generator=g)
    bias = 0.5 * torch.randn((3, 1, 8), generator=g)
    layout = bda.BlockPattern1d.from_blocks(3, [0, 2])
    fused = relu_lowrank.fused_forward(inp.to(DEV), weight.to(DEV), bias.to(DEV), 0.25, layout)
    reference = torch.relu(inp.double().matmul(weight.double()) + bias.double().reshape(1, 3, 1, 8) - 0.25)
    reference = reference * torch.tensor([1, 1, 1, 0, 0, 0, 1, 1], dtype=torch.float64)
    assert_close(fused.cpu().numpy(), reference.numpy(), 1e-5, 1e-5)


@pytest.mark.parametrize("d,N,h,h_in", [(128, 200, 4, 1), (192, 192, 4, 4), (256, 640, 4, 1), (320, 100, 2, 2), (512, 256, 8, 8)])
def test_relu_lowrank_single_row_small_matrix_bit_exact(bda, corc, d, N, h, h_in):
    """One input row against a matrix of a few MiB takes the kernel whose waves each fetch a 64-row span of k at once and
    hand the fmaf chain on in k order: same bits as the oracle's k-sequential chain and as the column-per-thread kernel,
    with bias, threshold and gate, for d that is and is not a multiple of the spans."""
    from burn_dragon_amd.kernel import relu_lowrank

    rng = np.random.default_rng(d + N)
    inp = rng.standard_normal((1, h_in, 1, d)).astype(np.float32)
    weight = (0.05 * rng.standard_normal((h, d, N))).astype(np.float32)
    bias = (0.1 * rng.standard_normal((h, 1, N))).astype(np.float32)
    gate = np.maximum(rng.standard_normal((1, h, 1, N)), 0).astype(np.float32)
    ref = corc.relu_lowrank(inp, weight, bias.reshape(h, N), 0.125)
    dense = bda.BlockPattern1d.dense(64)
    args = (torch.from_numpy(inp).to(DEV), torch.from_numpy(weight).to(DEV), torch.from_numpy(bias).to(DEV), 0.125, dense)
    got = relu_lowrank.fused_forward(*args)
    gated = relu_lowrank.fused_forward(*args, gate=torch.from_numpy(gate).to(DEV))
    ctx = bda.ffi.default_context(0)
    try:
        ctx.set_option("relu_lowrank.row", 0)
        plain = relu_lowrank.fused_forward(*args)
    finally:
        ctx.set_option("relu_lowrank.row", 1)
    assert np.array_equal(got.cpu().numpy(), ref)
    assert np.array_equal(plain.cpu().numpy(), ref)
    assert np.array_equal(gated.cpu().numpy(), gate * ref)
    assert 0.2 < (ref > 0).mean() < 0.8


@pytest.mark.parametrize("B,T,h_in", [(1, 1, 1), (3, 1, 1), (2, 5, 4), (8, 1, 1), (17, 1, 4), (32, 1, 1), (33, 1, 1), (1, 64, 4),
                                      (4, 16, 1), (2, 100, 1), (3, 43, 4)])
def test_relu_lowrank_bit_exact_against_oracle(bda, corc, B, T, h_in):
    """One k-sequential FMA chain per output on both sides: values, and therefore the active
    sets, are identical bit for bit whatever the launch tiling -- also on the f32 matrix cores, which calls
    of 8 to 64 rows take by default (a chain of v_mfma_f32_32x32x2_f32 over k is that same chain)."""
    from burn_dragon_amd.kernel import relu_lowrank

    h, d, N = 4, 256, 640
    rng = np.random.default_rng(B * 100 + T)
    inp = rng.standard_normal((B, h_in, T, d)).astype(np.float32)
    weight = (0.02 * rng.standard_normal((h, d, N))).astype(np.float32)
    gate = np.maximum(rng.standard_normal((B, h, T, N)), 0).astype(np.float32)
    ref = corc.relu_lowrank(inp, weight)
    args = (torch.from_numpy(inp).to(DEV), torch.from_numpy(weight).to(DEV), None, 0.0, bda.BlockPattern1d.dense(64))
    got = relu_lowrank.fused_forward(*args)
    assert np.array_equal(got.cpu().numpy(), ref)
    assert 0.4 < (ref > 0).mean() < 0.6
    ctx = bda.ffi.default_context(0)
    try:  # the matrix cores (8 to 64 rows; by default only for wide matrices), the scalar-input kernels (8 to 63
        # rows) and the LDS-staged ones all give the same bits
        ctx.set_option("relu_lowrank.mfma_rows", -8)
        mfma = relu_lowrank.fused_forward(*args)
        ctx.set_option("relu_lowrank.mfma_rows", 0)
        scalar = relu_lowrank.fused_forward(*args)
        ctx.set_option("relu_lowrank.scalar", 0)
        lds = relu_lowrank.fused_forward(*args)
    finally:
        ctx.set_option("relu_lowrank.scalar", 1)
        ctx.set_option("relu_lowrank.mfma_rows", 8)
    assert np.array_equal(mfma.cpu().numpy(), ref)
    assert np.array_equal(scalar.cpu().numpy(), ref)
    assert np.array_equal(lds.cpu().numpy(), ref)
    gated = relu_lowrank.fused_forward(*args, gate=torch.from_numpy(gate).to(DEV))
    assert np.array_equal(gated.cpu().numpy(), gate * ref)


@pytest.mark.parametrize("M,d,N,h_in", [(40, 512, 1024, 1), (64, 512, 520, 2), (9, 64, 132, 1), (32, 128, 4096, 2),
                                        (17, 64, 16384, 1)])
def test_relu_lowrank_on_the_matrix_cores_with_every_option(bda, corc, M, d, N, h_in):
    """The matrix-core projection (8 to 64 rows) with bias, threshold, block mask and gate, one and two row tiles,
    ragged column counts and wide value ranges (products from 1e-30 to 1e+6, results down to denormals): bit-exact
    against the oracle's fmaf chain and identical to the VALU kernels."""
    from burn_dragon_amd.kernel import relu_lowrank

    h = 2
    rng = np.random.default_rng(M + d + N)
    inp = (rng.standard_normal((M, h_in, 1, d)) * np.exp2(rng.integers(-40, 10, (M, h_in, 1, d)))).astype(np.float32)
    weight = (rng.standard_normal((h, d, N)) * np.exp2(rng.integers(-60, 10, (h, d, N)))).astype(np.float32)
    bias = (0.1 * rng.standard_normal((h, 1, N))).astype(np.float32)
    gate = np.maximum(rng.standard_normal((M, h, 1, N)), 0).astype(np.float32)
    blocks = [b for b in range(-(-N // 8)) if b % 3]
    layout = bda.BlockPattern1d.from_blocks(8, blocks)
    ref = corc.relu_lowrank(inp, weight, bias.reshape(h, N), 0.01, 8, blocks)
    args = (torch.from_numpy(inp).to(DEV), torch.from_numpy(weight).to(DEV), torch.from_numpy(bias).to(DEV), 0.01, layout)
    ctx = bda.ffi.default_context(0)
    try:
        ctx.set_option("relu_lowrank.mfma_rows", -8)  # whatever the width
        got = relu_lowrank.fused_forward(*args).cpu().numpy()
        gated = relu_lowrank.fused_forward(*args, gate=torch.from_numpy(gate).to(DEV)).cpu().numpy()
        ctx.set_option("relu_lowrank.mfma_rows", 0)
        valu = relu_lowrank.fused_forward(*args).cpu().numpy()
    finally:
        ctx.set_option("relu_lowrank.mfma_rows", 8)
    assert np.array_equal(got, ref)
    assert np.array_equal(valu, ref)
    assert np.array_equal(gated, gate * ref)
    assert 0.05 < (ref > 0).mean() < 0.6


@pytest.mark.parametrize("B,T,h_in,d,N", [(2, 100, 1, 256, 640), (1, 300, 3, 72, 203), (3, 64, 1, 512, 1024),
                                          (4, 130, 1, 64, 8192)])
def test_relu_lowrank_as_a_matrix_core_product_per_sequence(bda, corc, B, T, h_in, d, N):
    """Many tokens per sequence: one f32 matrix-core product per (sequence, head) whose k order is that of a scalar
    loop, so the outputs are again the bits of the oracle's fmaf chain -- with bias, threshold, block mask and gate,
    ragged tiles in rows, columns and k (K = 72 is not a multiple of the 16-wide stage), wide value ranges.  The last
    case (N a multiple of 256, 768 tiles of 128 x 256) takes the wide-tile instance that long prompts of a large
    model run on."""
    from burn_dragon_amd.kernel import relu_lowrank

    h = 3
    rng = np.random.default_rng(B + T + N)
    inp = (rng.standard_normal((B, h_in, T, d)) * np.exp2(rng.integers(-30, 8, (B, h_in, T, d)))).astype(np.float32)
    weight = (rng.standard_normal((h, d, N)) * np.exp2(rng.integers(-50, 8, (h, d, N)))).astype(np.float32)
    bias = (0.1 * rng.standard_normal((h, 1, N))).astype(np.float32)
    gate = np.maximum(rng.standard_normal((B, h, T, N)), 0).astype(np.float32)
    blocks = [b for b in range(-(-N // 8)) if b % 4]
    layout = bda.BlockPattern1d.from_blocks(8, blocks)
    ref = corc.relu_lowrank(inp, weight, bias.reshape(h, N), 0.01, 8, blocks)
    args = (torch.from_numpy(inp).to(DEV), torch.from_numpy(weight).to(DEV), torch.from_numpy(bias).to(DEV), 0.01, layout)
    ctx = bda.ffi.default_context(0)
    try:
        ctx.set_option("relu_lowrank.gemm_rows", -64)  # whatever the grid
        got = relu_lowrank.fused_forward(*args).cpu().numpy()
        gated = relu_lowrank.fused_forward(*args, gate=torch.from_numpy(gate).to(DEV)).cpu().numpy()
        ctx.set_option("relu_lowrank.gemm_rows", 0)
        tile = relu_lowrank.fused_forward(*args).cpu().numpy()
    finally:
        ctx.set_option("relu_lowrank.gemm_rows", 64)
    assert np.array_equal(tile, ref)
    assert np.array_equal(got, ref)
    assert np.array_equal(gated, gate * ref)
    assert 0.05 < (ref > 0).mean() < 0.6


def test_relu_lowrank_many_rows_with_bias_threshold_and_mask(bda, corc):
    """The 64-row tile kernel (B*T >= 64) with every optional input, bit-exact against the oracle, and
    identical to the 8-row kernel."""
    from burn_dragon_amd.kernel import relu_lowrank

    B, T, h, d, N = 2, 70, 3, 36, 200  # ragged in rows, columns and k
    rng = np.random.default_rng(8)
    inp = rng.standard_normal((B, 1, T, d)).astype(np.float32)
    weight = (0.2 * rng.standard_normal((h, d, N))).astype(np.float32)
    bias = (0.1 * rng.standard_normal((h, 1, N))).astype(np.float32)
    layout = bda.BlockPattern1d.from_blocks(8, [0, 3, 4, 17, 24])
    ref = corc.relu_lowrank(inp, weight, bias.reshape(h, N), 0.05, 8, [0, 3, 4, 17, 24])
    args = (torch.from_numpy(inp).to(DEV), torch.from_numpy(weight).to(DEV), torch.from_numpy(bias).to(DEV), 0.05, layout)
    ctx = bda.ffi.default_context(0)
    try:
        ctx.set_option("relu_lowrank.tile", 2)  # the default keeps the tile kernel for grids that cover the chip
        got = relu_lowrank.fused_forward(*args).cpu().numpy()
        ctx.set_option("relu_lowrank.tile", 0)
        small = relu_lowrank.fused_forward(*args).cpu().numpy()
    finally:
        ctx.set_option("relu_lowrank.tile", 1)
    assert np.array_equal(got, ref)
    assert 0.05 < (ref > 0).mean() < 0.2
    assert np.array_equal(got, small)
    # a shape whose tile grid covers the chip takes the tile kernel by default
    big_w = (0.05 * rng.standard_normal((4, 64, 8192))).astype(np.float32)
    big_in = rng.standard_normal((2, 1, 128, 64)).astype(np.float32)
    big = relu_lowrank.fused_forward(torch.from_numpy(big_in).to(DEV), torch.from_numpy(big_w).to(DEV), None, 0.0,
                                     bda.BlockPattern1d.dense(64)).cpu().numpy()
    assert np.array_equal(big, corc.relu_lowrank(big_in, big_w))


def test_layer_norm_matches_oracle_and_library(bda, corc):
    from burn_dragon_amd.recurrent import layer_norm

    rng = np.random.default_rng(3)
    for d in (16, 256, 512, 1000):
        x = (2.0 * rng.standard_normal((7, 3, d)) + 0.5).astype(np.float32)
        got = layer_norm(torch.from_numpy(x).to(DEV)).cpu().numpy()
        assert_close(got, corc.layer_norm(x), 2e-6, 1e-5)
        assert_close(got, torch.nn.functional.layer_norm(torch.from_numpy(x), (d,), eps=1e-5).numpy(), 2e-6, 1e-5)


def _shape_from_cfg(cfg):
    return orc.BDHShape(n_layer=cfg.n_layer, n_embd=cfg.n_embd, n_head=cfg.n_head,
                        mlp_internal_dim_multiplier=cfg.mlp_internal_dim_multiplier, vocab_size=cfg.vocab_size,
                        rotary=int(cfg.fused_kernels.rotary_embedding), rope_theta=cfg.fused_kernels.rope_theta,
                        relu_threshold=cfg.fused_kernels.relu_threshold, alibi_slopes=cfg.fused_kernels.alibi_slopes)


def _model_pair(bda, cfg, seed, **kw):
    shape = _shape_from_cfg(cfg)
    w = orc.init_weights(shape, seed)
    model = bda.BDH(cfg, DEV, weights={"embed": w.embed, "encoder": w.encoder, "encoder_v": w.encoder_v,
                                       "decoder": w.decoder, "lm_head": w.lm_head}, **kw)
    return shape, w, model


@pytest.mark.parametrize("rotary,fused", [("rope", False), ("pope", False), ("alibi", False), ("alibi", True)])
def test_inference_paths_run_across_configs(bda, corc, rotary, fused):
    """tests/model_paths.rs:66-91: L=2, d=16, h=2, mult=4, V=32, tokens [[0,1,2,3],[4,5,6,7]], the four
    (rotary, fused) configurations -> forward_fast logits [2,4,32]; forward_with_state logits [2,4,32],
    state.position == 4 — plus the values, against the oracle."""
    cfg = bda.BDHConfig(n_layer=2, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=32, dropout=0.0)
    cfg.fused_kernels.enabled = fused
    cfg.fused_kernels.set_block_sizes(4, 4)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.parse(rotary))
    shape, w, model = _model_pair(bda, cfg, seed=11)
    tokens = np.arange(8).reshape(2, 4)
    logits_fast = model.forward_fast(torch.from_numpy(tokens))
    assert tuple(logits_fast.shape) == (2, 4, 32)
    fast_ref = orc.forward_fast(shape, w, tokens, fused=fused, time_block=4)
    assert rel_err(logits_fast.cpu().numpy(), fast_ref) < 1e-3
    state = model.init_state()
    logits = model.forward_with_state(torch.from_numpy(tokens), state)
    torch.cuda.synchronize()
    assert tuple(logits.shape) == (2, 4, 32)
    assert state.position == 4
    Nq = model.latent_q
    rho_ref = np.zeros((2, 2, 2, Nq, 16), np.float32)
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, tokens, rho_ref, 0, sparse_state=False)
    assert pos == 4
    assert rel_err(logits.cpu().numpy(), logits_ref) < 1e-3
    assert rel_err(state.storage.cpu().numpy(), rho_ref) < 1e-3
    # a second call continues from the stored state and position
    more = np.array([[9], [10]])
    logits2 = model.forward_with_state(torch.from_numpy(more), state)
    logits2_ref, pos, _, _ = corc.forward_with_state(shape, w, more, rho_ref, 4, sparse_state=False)
    assert state.position == 5 == pos
    assert rel_err(logits2.cpu().numpy(), logits2_ref) < 1e-3


@pytest.mark.parametrize("rotary", ["rope", "pope"])
def test_long_prompt_takes_the_dense_chunk_form(bda, corc, rotary):
    """A prompt of 128+ tokens runs the state update as dense products on the f32 matrix cores; logits and
    state agree with the oracle's token loop, and decoding continues from that state."""
    cfg = bda.BDHConfig(n_layer=2, n_embd=32, n_head=2, mlp_internal_dim_multiplier=8, vocab_size=64, dropout=0.0)
    cfg.fused_kernels.set_block_sizes(4, 4)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.parse(rotary))
    shape, w, model = _model_pair(bda, cfg, seed=23)
    rng = np.random.default_rng(3)
    tokens = rng.integers(0, 64, (2, 150))
    state = model.init_state()
    logits = model.forward_with_state(torch.from_numpy(tokens), state)
    Nq = model.latent_q
    rho_ref = np.zeros((2, 2, 2, Nq, 32), np.float32)
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, tokens, rho_ref, 0, sparse_state=False)
    assert rel_err(logits.cpu().numpy(), logits_ref) < 1e-3
    assert rel_err(state.storage.cpu().numpy(), rho_ref) < 1e-3
    # the same prompt through the step kernels (dense form switched off) gives the same logits
    ctx = bda.ffi.default_context(0)
    try:
        ctx.set_option("state_step.dense_chunks", 0)
        state_s = model.init_state()
        logits_s = model.forward_with_state(torch.from_numpy(tokens), state_s)
    finally:
        ctx.set_option("state_step.dense_chunks", -1)
    assert rel_err(logits.cpu().numpy(), logits_s.cpu().numpy()) < 1e-4
    more = rng.integers(0, 64, (2, 1))
    logits2 = model.forward_with_state(torch.from_numpy(more), state)
    logits2_ref, pos, _, _ = corc.forward_with_state(shape, w, more, rho_ref, pos, sparse_state=False)
    assert state.position == 151 == pos
    assert rel_err(logits2.cpu().numpy(), logits2_ref) < 1e-3


def test_forward_fast_long_sequence_on_the_matrix_cores(bda):
    """T = 160 takes the f32 matrix-core form of fused_state_aligned inside forward_fast; both branches against
    the numpy composition."""
    cfg = bda.BDHConfig(n_layer=2, n_embd=32, n_head=2, mlp_internal_dim_multiplier=8, vocab_size=64, dropout=0.0)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.parse("rope"))
    tokens = np.random.default_rng(2).integers(0, 64, (2, 160))
    for fused in (False, True):
        cfg.fused_kernels.enabled = fused
        cfg.fused_kernels.set_block_sizes(32, 32)
        shape, w, model = _model_pair(bda, cfg, seed=31)
        got = model.forward_fast(torch.from_numpy(tokens)).cpu().numpy()
        want = orc.forward_fast(shape, w, tokens, fused=fused, time_block=32)
        assert rel_err(got, want) < 1e-3


@pytest.mark.parametrize("T", [12, 160])
def test_forward_fast_with_sparse_block_patterns(bda, T):
    """FusedKernelConfig.block_sparse with a sparse latent pattern (src/kernel/block_sparse.rs:25-36) and a sparse
    time-block pattern (:84-95) through forward_fast (src/model/bdh.rs:111-151): the latent mask reaches both
    projections, the pair list the attention, for the row kernel (T = 12) and the matrix-core form (T = 160).
    A pattern naming every causal pair and every latent block gives the dense result
    (tests/fused_kernel_tests.rs:108); with the fused kernels off the patterns are not consulted."""
    from burn_dragon_amd.kernel import BlockPattern1d, BlockPattern2d, BlockSparseConfig

    cfg = bda.BDHConfig(n_layer=2, n_embd=32, n_head=2, mlp_internal_dim_multiplier=8, vocab_size=64, dropout=0.0)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.parse("rope"))
    cfg.fused_kernels.enabled = True
    N = cfg.latent_per_head()  # 128
    lat_block, time_block = 16, 4 if T < 64 else 32
    tb = -(-T // time_block)
    tokens = np.random.default_rng(5).integers(0, 64, (2, T))
    latent_active = [0, 2, 3, 6]
    pairs = {(r, c) for r in range(tb) for c in range(r + 1) if (r + c) % 3 != 1} | {(0, 0)}
    cfg.fused_kernels.block_sparse = BlockSparseConfig(BlockPattern1d.from_blocks(lat_block, latent_active),
                                                       BlockPattern2d.from_pairs(time_block, pairs))
    shape, w, model = _model_pair(bda, cfg, seed=41)
    got = model.forward_fast(torch.from_numpy(tokens)).cpu().numpy()
    want = orc.forward_fast(shape, w, tokens, fused=True, time_block=time_block, time_pairs=pairs,
                            latent_block=lat_block, latent_active=latent_active)
    assert rel_err(got, want) < 1e-3
    dense_ref = orc.forward_fast(shape, w, tokens, fused=True, time_block=time_block)
    assert rel_err(dense_ref, want) > 1e-2  # the patterns matter at this size
    # every causal pair and every latent block named explicitly: the dense result
    cfg.fused_kernels.block_sparse = BlockSparseConfig(
        BlockPattern1d.from_blocks(lat_block, range(N // lat_block)),
        BlockPattern2d.from_pairs(time_block, {(r, c) for r in range(tb) for c in range(r + 1)}))
    _, _, model_all = _model_pair(bda, cfg, seed=41)
    assert rel_err(model_all.forward_fast(torch.from_numpy(tokens)).cpu().numpy(), dense_ref) < 1e-3
    # the plain branch ignores the patterns
    cfg.fused_kernels.block_sparse = BlockSparseConfig(BlockPattern1d.from_blocks(lat_block, latent_active),
                                                       BlockPattern2d.from_pairs(time_block, pairs))
    cfg.fused_kernels.enabled = False
    shape_p, w_p, model_p = _model_pair(bda, cfg, seed=41)
    assert rel_err(model_p.forward_fast(torch.from_numpy(tokens)).cpu().numpy(),
                   orc.forward_fast(shape_p, w_p, tokens, fused=False)) < 1e-3


def test_batched_decode_step_takes_the_split_k_encoder(bda, corc):
    """24+ sequences decoding together: the encoder E runs as a split-K product on the f32 matrix cores (the
    weights are streamed once); logits against the oracle and against the VALU kernel."""
    cfg = bda.BDHConfig(n_layer=2, n_embd=64, n_head=4, mlp_internal_dim_multiplier=64, vocab_size=64)  # N = 1024
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.parse("rope"))
    shape, w, model = _model_pair(bda, cfg, seed=5)
    rng = np.random.default_rng(1)
    B = 26
    steps = [rng.integers(0, 64, (B, 1)) for _ in range(3)]
    ctx = bda.ffi.default_context(0)
    outs = {}
    for rows in (24, 1 << 30):
        ctx.set_option("decoder.splitk_rows", -rows if rows == 24 else rows)  # forced: by default only for a large grid
        try:
            state = model.init_state()
            outs[rows] = np.concatenate([model.forward_with_state(torch.from_numpy(t), state).cpu().numpy() for t in steps], 1)
        finally:
            ctx.set_option("decoder.splitk_rows", 24)
    rho_ref = np.zeros((2, B, 4, 1024, 64), np.float32)
    pos, refs = 0, []
    for t in steps:
        lg, pos, _, _ = corc.forward_with_state(shape, w, t, rho_ref, pos, sparse_state=True)
        refs.append(lg)
    ref = np.concatenate(refs, 1)
    assert rel_err(outs[24], ref) < 1e-3 and rel_err(outs[1 << 30], ref) < 1e-3
    assert rel_err(outs[24], outs[1 << 30]) < 1e-5 and not np.array_equal(outs[24], outs[1 << 30])


def test_config1_architecture_prefill_and_greedy_decode(bda, corc):
    """BASELINE config 1 architecture (V=256, d=256, h=4, N=8192, RoPE) with L=2 and a short
    run so the oracle finishes in seconds: 16-byte prompt, 8 greedy tokens, batch 1."""
    cfg = bda.BDHConfig(n_layer=2, n_embd=256, n_head=4, mlp_internal_dim_multiplier=128, vocab_size=256)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    shape, w, model = _model_pair(bda, cfg, seed=5)
    assert model.latent == 8192
    rng = np.random.default_rng(0)
    prompt = rng.integers(0, 256, size=(1, 16))
    L, h, N, d = 2, 4, 8192, 256
    state = model.init_state()
    x_tap = torch.zeros((L, 1, h, 16, N), device=DEV)
    logits, nxt = model.forward_with_state(torch.from_numpy(prompt), state, want_next=True, x_tap=x_tap)
    torch.cuda.synchronize()
    rho_ref = np.zeros((L, 1, h, N, d), np.float32)
    logits_ref, pos, x_ref, _ = corc.forward_with_state(shape, w, prompt, rho_ref, 0, taps=True)
    assert rel_err(logits.cpu().numpy(), logits_ref) < 1e-3
    # active sets: layer 0 bit-exact; deeper layers identical wherever |pre-activation| is not ~0
    x_gpu = x_tap.cpu().numpy()
    assert np.array_equal(x_gpu[0] > 0, x_ref[0] > 0)
    assert np.array_equal(x_gpu[0], x_ref[0])
    flips = ((x_gpu[1] > 0) != (x_ref[1] > 0))
    assert flips.mean() < 1e-3
    assert np.maximum(x_gpu[1], x_ref[1])[flips].max(initial=0.0) < 1e-4
    dens = (x_ref > 0).mean()
    assert 0.4 < dens < 0.6  # random-init weights: about half the neurons fire
    tokens_gpu, tokens_ref = [], []
    tok_ref = corc.greedy_token(logits_ref[0, -1])
    assert int(nxt[0]) == tok_ref
    position = pos
    for _ in range(8):
        tokens_ref.append(tok_ref)
        tokens_gpu.append(int(nxt[0]))
        lg, nxt = model.forward_with_state(nxt.reshape(1, 1), state, want_next=True)
        lr, position, _, _ = corc.forward_with_state(shape, w, np.array([[tok_ref]]), rho_ref, position)
        assert rel_err(lg.cpu().numpy(), lr) < 1e-3
        tok_ref = corc.greedy_token(lr[0, -1])
    assert tokens_gpu == tokens_ref
    assert state.position == 24 == position
    assert rel_err(state.storage.cpu().numpy(), rho_ref) < 1e-3


def test_config1_full_run_against_oracle(bda, corc):
    """BASELINE config 1 at its full size: L=6, d=256, h=4, N=8192, V=256, B=1, a 64-byte prompt in
    one call and 256 greedy decode steps.  Every step's logits are held to 1e-3 of their max-norm.
    Both sides are fed the oracle's token, so a near-tie in the argmax cannot fork the two runs; where
    the device's argmax differs, the oracle's two best logits must be closer than the tolerance."""
    cfg = bda.BDHConfig(n_layer=6, n_embd=256, n_head=4, mlp_internal_dim_multiplier=128, vocab_size=256)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    shape, w, model = _model_pair(bda, cfg, seed=7)
    L, h, N, d, T0, steps = 6, 4, 8192, 256, 64, 256
    prompt = np.random.default_rng(1).integers(0, 256, size=(1, T0))
    state = model.init_state()
    x_tap = torch.zeros((L, 1, h, T0, N), device=DEV)
    logits, nxt = model.forward_with_state(torch.from_numpy(prompt), state, want_next=True, x_tap=x_tap)
    torch.cuda.synchronize()
    rho_ref = np.zeros((L, 1, h, N, d), np.float32)
    logits_ref, pos, x_ref, _ = corc.forward_with_state(shape, w, prompt, rho_ref, 0, taps=True)
    assert rel_err(logits.cpu().numpy(), logits_ref) < 1e-3
    x_gpu = x_tap.cpu().numpy()
    assert np.array_equal(x_gpu[0], x_ref[0])  # layer 0: values and active set bit-exact
    for l in range(1, L):  # deeper layers: the sets differ only where the pre-activation is ~0
        flips = (x_gpu[l] > 0) != (x_ref[l] > 0)
        assert flips.mean() < 1e-3, (l, flips.mean())
        assert np.maximum(x_gpu[l], x_ref[l])[flips].max(initial=0.0) < 1e-4
    worst, disagreements = 0.0, 0
    for step in range(steps):
        tok_ref = corc.greedy_token(logits_ref[0, -1])
        if int(nxt[0]) != tok_ref:
            top = np.sort(logits_ref[0, -1])[-2:]
            assert top[1] - top[0] < 1e-3 * np.abs(logits_ref).max(), f"step {step}: argmax differs on a clear lead"
            disagreements += 1
        feed = torch.tensor([[tok_ref]])
        logits, nxt = model.forward_with_state(feed, state, want_next=True)
        logits_ref, pos, _, _ = corc.forward_with_state(shape, w, np.array([[tok_ref]]), rho_ref, pos)
        worst = max(worst, rel_err(logits.cpu().numpy(), logits_ref))
        assert worst < 1e-3, f"step {step}: {worst}"
    assert state.position == T0 + steps == pos
    assert rel_err(state.storage.cpu().numpy(), rho_ref) < 1e-3
    print(f"config 1 full run: worst logits rel err {worst:.2e}, argmax near-ties {disagreements}")


def test_decode_equals_prefill_on_device(bda):
    """T tokens in one call == T single-token calls carrying the state: bit for bit when the single-token calls
    run kernel by kernel, to a few ulp when they take the one-launch decode step this model is small enough for
    (its sums over state rows and over the decoder's k are taken in a tree of its own)."""
    cfg = bda.BDHConfig(n_layer=3, n_embd=256, n_head=4, mlp_internal_dim_multiplier=8, vocab_size=64)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    model = bda.BDH(cfg, DEV, seed=9)
    tokens = torch.randint(0, 64, (4, 6), generator=torch.Generator().manual_seed(1))
    sa, sb, sc = model.init_state(), model.init_state(), model.init_state()
    la = model.forward_with_state(tokens, sa)
    ctx = bda.ffi.default_context(0)
    try:
        ctx.set_option("model.one_launch", 0)
        rows = [model.forward_with_state(tokens[:, t : t + 1], sb) for t in range(6)]
    finally:
        ctx.set_option("model.one_launch", 1)
    torch.cuda.synchronize()
    assert torch.equal(torch.cat(rows, 1), la)
    assert torch.equal(sa.storage, sb.storage) and sa.position == sb.position == 6
    try:
        ctx.set_option("model.one_launch", 2)  # whatever the size and the batch
        one = torch.cat([model.forward_with_state(tokens[:, t : t + 1], sc) for t in range(6)], 1)
    finally:
        ctx.set_option("model.one_launch", 1)
    torch.cuda.synchronize()
    assert not torch.equal(one, torch.zeros_like(one))
    assert rel_err(one.cpu().numpy(), la.cpu().numpy()) < 1e-5
    assert rel_err(sc.storage.cpu().numpy(), sa.storage.cpu().numpy()) < 1e-5 and sc.position == 6


@pytest.mark.parametrize("rotary,lazy", [("rope", False), ("pope", False), ("alibi", False), ("alibi", True)])
@pytest.mark.parametrize("d,h,mult,L,V", [(64, 1, 4, 2, 40), (128, 4, 4, 3, 69), (256, 8, 8, 2, 256), (32, 16, 16, 2, 17)])
def test_one_launch_decode_step(bda, corc, rotary, lazy, d, h, mult, L, V):
    """A small model's decode step (one token per sequence, no by-products) runs as ONE launch, a workgroup per
    sequence.  Logits, state and greedy tokens against the C oracle (1e-3) and against the same steps run kernel by
    kernel (1e-5: only the summation trees differ), after a prompt that went through the many-token path."""
    cfg = bda.BDHConfig(n_layer=L, n_embd=d, n_head=h, mlp_internal_dim_multiplier=mult, vocab_size=V, dropout=0.0)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.parse(rotary))
    shape = _shape_from_cfg(cfg)
    w = orc.init_weights(shape, seed=d + h)
    weights = {"embed": w.embed, "encoder": w.encoder, "encoder_v": w.encoder_v, "decoder": w.decoder, "lm_head": w.lm_head}
    one = bda.BDH(cfg, DEV, weights=weights, alibi_lazy=lazy)
    ref = bda.BDH(cfg, DEV, weights=weights, alibi_lazy=lazy)
    B, T0, steps = 3, 5, 4
    rng = np.random.default_rng(7 * d + h)
    prompt = rng.integers(0, V, (B, T0))
    rho_ref = np.zeros((L, B, h, one.latent_q, d), np.float32)
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, prompt, rho_ref, 0, sparse_state=False)
    s_one, s_ref = one.init_state(), ref.init_state()
    ctx = bda.ffi.default_context(0)
    _, nxt = one.forward_with_state(torch.from_numpy(prompt), s_one, want_next=True)
    ref.forward_with_state(torch.from_numpy(prompt), s_ref)
    feed = logits_ref[:, -1].argmax(-1)
    for step in range(steps):
        tok = feed.reshape(B, 1)
        logits_ref, pos, _, _ = corc.forward_with_state(shape, w, tok, rho_ref, pos, sparse_state=False)
        try:
            ctx.set_option("model.one_launch", 2)  # whatever the size and the batch
            got, nxt = one.forward_with_state(torch.from_numpy(tok), s_one, want_next=True)
            ctx.set_option("model.one_launch", 0)
            kbk = ref.forward_with_state(torch.from_numpy(tok), s_ref)
        finally:
            ctx.set_option("model.one_launch", 1)
        torch.cuda.synchronize()
        got_np = got.cpu().numpy()
        assert rel_err(got_np, logits_ref) < 1e-3, f"step {step} against the oracle"
        assert rel_err(got_np, kbk.cpu().numpy()) < 1e-5, f"step {step} against the kernel-by-kernel step"
        assert np.array_equal(nxt.cpu().numpy(), got_np[:, 0].argmax(-1))
        feed = logits_ref[:, -1].argmax(-1)
    assert s_one.position == T0 + steps == pos
    one.materialize_state(s_one)
    ref.materialize_state(s_ref)
    torch.cuda.synchronize()
    assert rel_err(s_one.storage.cpu().numpy(), rho_ref) < 1e-3
    assert rel_err(s_one.storage.cpu().numpy(), s_ref.storage.cpu().numpy()) < 1e-5
    if lazy:
        assert torch.equal(s_one.stamps, s_ref.stamps)


@pytest.mark.parametrize("rotary,lazy", [("rope", False), ("pope", False), ("alibi", False), ("alibi", True)])
@pytest.mark.parametrize("d,h,mult,L,V", [(128, 4, 32, 2, 40), (192, 3, 4, 3, 69), (256, 4, 16, 2, 256), (512, 8, 4, 2, 17)])
def test_two_launch_layer_decode_step(bda, corc, rotary, lazy, d, h, mult, L, V):
    """A decode step of a mid-size model at a small batch runs two launches per layer (a workgroup per 64 neurons of a
    head of a sequence).  Logits, state and greedy tokens against the C oracle (1e-3) and against the same steps run
    kernel by kernel (1e-5: only the summation trees differ), after a prompt that went through the many-token path."""
    cfg = bda.BDHConfig(n_layer=L, n_embd=d, n_head=h, mlp_internal_dim_multiplier=mult, vocab_size=V, dropout=0.0)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.parse(rotary))
    shape = _shape_from_cfg(cfg)
    w = orc.init_weights(shape, seed=d + h)
    weights = {"embed": w.embed, "encoder": w.encoder, "encoder_v": w.encoder_v, "decoder": w.decoder, "lm_head": w.lm_head}
    fused = bda.BDH(cfg, DEV, weights=weights, alibi_lazy=lazy)
    ref = bda.BDH(cfg, DEV, weights=weights, alibi_lazy=lazy)
    assert fused.latent % 64 == 0
    B, T0, steps = 3, 5, 4
    rng = np.random.default_rng(7 * d + h)
    prompt = rng.integers(0, V, (B, T0))
    rho_ref = np.zeros((L, B, h, fused.latent_q, d), np.float32)
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, prompt, rho_ref, 0, sparse_state=False)
    s_fused, s_ref = fused.init_state(), ref.init_state()
    ctx = bda.ffi.default_context(0)
    fused.forward_with_state(torch.from_numpy(prompt), s_fused)
    ref.forward_with_state(torch.from_numpy(prompt), s_ref)
    feed = logits_ref[:, -1].argmax(-1)
    for step in range(steps):
        tok = feed.reshape(B, 1)
        logits_ref, pos, _, _ = corc.forward_with_state(shape, w, tok, rho_ref, pos, sparse_state=False)
        got, nxt = fused.forward_with_state(torch.from_numpy(tok), s_fused, want_next=True)  # B <= 8: two launches per layer
        try:
            ctx.set_option("model.one_launch", 0)
            kbk = ref.forward_with_state(torch.from_numpy(tok), s_ref)
        finally:
            ctx.set_option("model.one_launch", 1)
        torch.cuda.synchronize()
        got_np = got.cpu().numpy()
        assert rel_err(got_np, logits_ref) < 1e-3, f"step {step} against the oracle"
        assert rel_err(got_np, kbk.cpu().numpy()) < 1e-5, f"step {step} against the kernel-by-kernel step"
        assert not np.array_equal(got_np, kbk.cpu().numpy()), "the two-launch layer was not taken"
        assert np.array_equal(nxt.cpu().numpy(), got_np[:, 0].argmax(-1))
        feed = logits_ref[:, -1].argmax(-1)
    assert s_fused.position == T0 + steps == pos
    fused.materialize_state(s_fused)
    ref.materialize_state(s_ref)
    torch.cuda.synchronize()
    assert rel_err(s_fused.storage.cpu().numpy(), rho_ref) < 1e-3
    assert rel_err(s_fused.storage.cpu().numpy(), s_ref.storage.cpu().numpy()) < 1e-5
    if lazy:
        assert torch.equal(s_fused.stamps, s_ref.stamps)


@pytest.mark.parametrize("rotary,lazy", [("rope", False), ("pope", False), ("alibi", False), ("alibi", True)])
@pytest.mark.parametrize("form,d,h,mult,L,V", [("one-launch", 128, 4, 4, 3, 69), ("one-launch", 256, 8, 8, 2, 256),
                                              ("two-launch-layer", 256, 4, 16, 2, 256),
                                              ("two-launch-layer", 192, 3, 4, 3, 69)])
def test_fused_decode_forms_with_bf16_state(bda, corc, form, rotary, lazy, d, h, mult, L, V):
    """The one-launch step and the two-launch layer with the state stored in bf16 (f32 arithmetic, one rounding per
    stored element per token, like the kernel-by-kernel bf16 step): logits against the f32 oracle within the 2e-2
    allowed for a bf16 state, and against the kernel-by-kernel bf16 step, where only summation trees differ (the
    inputs of a rounding can differ in their last bits, so a few stored elements may land one bf16 step apart)."""
    from burn_dragon_amd import ffi

    cfg = bda.BDHConfig(n_layer=L, n_embd=d, n_head=h, mlp_internal_dim_multiplier=mult, vocab_size=V, dropout=0.0)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.parse(rotary))
    shape = _shape_from_cfg(cfg)
    w = orc.init_weights(shape, seed=d + h)
    weights = {"embed": w.embed, "encoder": w.encoder, "encoder_v": w.encoder_v, "decoder": w.decoder, "lm_head": w.lm_head}
    fused = bda.BDH(cfg, DEV, weights=weights, alibi_lazy=lazy, rho_dtype=ffi.BF16)
    ref = bda.BDH(cfg, DEV, weights=weights, alibi_lazy=lazy, rho_dtype=ffi.BF16)
    B, T0, steps = 3, 5, 4
    rng = np.random.default_rng(7 * d + h)
    prompt = rng.integers(0, V, (B, T0))
    rho_ref = np.zeros((L, B, h, fused.latent_q, d), np.float32)
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, prompt, rho_ref, 0, sparse_state=False)
    s_fused, s_ref = fused.init_state(), ref.init_state()
    ctx = bda.ffi.default_context(0)
    fused.forward_with_state(torch.from_numpy(prompt), s_fused)
    ref.forward_with_state(torch.from_numpy(prompt), s_ref)
    assert s_fused.storage.dtype == torch.bfloat16
    feed = logits_ref[:, -1].argmax(-1)
    for step in range(steps):
        tok = feed.reshape(B, 1)
        logits_ref, pos, _, _ = corc.forward_with_state(shape, w, tok, rho_ref, pos, sparse_state=False)
        try:
            ctx.set_option("model.one_launch", 2 if form == "one-launch" else 1)
            got, nxt = fused.forward_with_state(torch.from_numpy(tok), s_fused, want_next=True)
            ctx.set_option("model.one_launch", 0)
            kbk = ref.forward_with_state(torch.from_numpy(tok), s_ref)
        finally:
            ctx.set_option("model.one_launch", 1)
        torch.cuda.synchronize()
        got_np = got.cpu().numpy()
        assert rel_err(got_np, logits_ref) < 2e-2, f"step {step} against the oracle"
        assert rel_err(got_np, kbk.cpu().numpy()) < 2e-3, f"step {step} against the kernel-by-kernel step"
        assert not np.array_equal(got_np, kbk.cpu().numpy()), "the fused form was not taken"
        assert np.array_equal(nxt.cpu().numpy(), got_np[:, 0].argmax(-1))
        feed = logits_ref[:, -1].argmax(-1)
    fused.materialize_state(s_fused)
    ref.materialize_state(s_ref)
    torch.cuda.synchronize()
    assert rel_err(s_fused.storage.float().cpu().numpy(), rho_ref) < 2e-2
    # one bf16 step of the largest element is 2^-8 of it; an element that landed a step apart can drift by another
    # step at a later token, so the bound is one step per decode step, and few elements may differ at all
    err_forms = rel_err(s_fused.storage.float().cpu().numpy(), s_ref.storage.float().cpu().numpy())
    assert err_forms < steps * 2.0 ** -8, err_forms
    differing = (s_fused.storage != s_ref.storage).float().mean().item()
    assert differing < 0.02, f"{differing:.4f} of the stored elements differ between the forms"
    if lazy:
        assert torch.equal(s_fused.stamps, s_ref.stamps)


def test_bad_token_poisons_only_its_row(bda):
    cfg = bda.BDHConfig(n_layer=1, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=32)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    model = bda.BDH(cfg, DEV, seed=2)
    logits = model.forward_with_state(torch.tensor([[3], [99]]), model.init_state())
    torch.cuda.synchronize()
    assert torch.isfinite(logits[0]).all() and torch.isnan(logits[1]).all()


def test_model_create_rejects_bad_configs(bda):
    from burn_dragon_amd import ffi

    cfg = bda.BDHConfig(n_layer=1, n_embd=16, n_head=2, mlp_internal_dim_multiplier=1, vocab_size=8)  # N = 8
    cfg.n_head = 16  # latent_per_head = 1: odd, RoPE must refuse it (src/model/attention.rs:310)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    with pytest.raises(ffi.BdhError) as err:
        bda.BDH(cfg, DEV, seed=1)
    assert err.value.status == ffi.E_SHAPE


@pytest.mark.parametrize("d,mult,B", [(256, 16, 2), (256, 128, 2), (128, 4, 2), (256, 128, 1)],
                         ids=["two-launch-layer", "kernel-by-kernel", "one-launch", "four-launch-layer"])
def test_decode_graph_replays_match_eager_steps(bda, d, mult, B):
    """A captured decode step is replayed several times, with eager work and synchronisations of the
    same program between the replays, and every replay is checked against the eager path -- for each of
    the four forms a decode step can take."""
    cfg = bda.BDHConfig(n_layer=3, n_embd=d, n_head=4, mlp_internal_dim_multiplier=mult, vocab_size=64)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    model = bda.BDH(cfg, DEV, seed=21)
    prompt = torch.randint(0, 64, (B, 5), generator=torch.Generator().manual_seed(2))
    se, sg = model.init_state(), model.init_state()
    _, nxt_e = model.forward_with_state(prompt, se, want_next=True)
    _, nxt_g = model.forward_with_state(prompt, sg, want_next=True)
    graph = model.capture_decode_step(sg, nxt_g)
    assert torch.equal(sg.storage, se.storage)  # capture must not disturb the state
    for step in range(6):
        logits_e, new_e = model.forward_with_state(nxt_e.reshape(B, 1), se, want_next=True)
        torch.cuda.synchronize()
        junk = torch.randn(1 << 16, device=DEV).sum()  # unrelated eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(graph.logits, logits_e), f"replay {step}"
        assert torch.equal(graph.tokens, new_e)
        assert torch.equal(sg.storage, se.storage)
        assert sg.position == se.position == 6 + step
        assert int(graph.positions[0]) == sg.position
        nxt_e = new_e
        del junk


@pytest.mark.parametrize("d,mult,h,state", [(256, 32, 4, "f32"), (512, 16, 2, "f32"), (256, 32, 4, "bf16")])
def test_single_sequence_decode_folds_the_reductions_into_the_projections(bda, corc, d, mult, h, state):
    """A decode step of one sequence through a RoPE model with more than 64 blocks of 64 neurons takes four launches
    per layer ("model.fused_rows"): D_y sums the readout partials and applies their LayerNorm itself, the next layer's
    D_x the encoder partials with the two LayerNorms and the residual.  Against the kernel-by-kernel step (1e-5: other
    summation trees; a bf16 state: one rounding step) and the oracle (1e-3 / 2e-2), over a prompt and 12 greedy steps;
    the state both leave is compared too."""
    from burn_dragon_amd import ffi

    cfg = bda.BDHConfig(n_layer=3, n_embd=d, n_head=h, mlp_internal_dim_multiplier=mult, vocab_size=256)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    dt = ffi.BF16 if state == "bf16" else ffi.F32
    shape, w, model = _model_pair(bda, cfg, seed=13, rho_dtype=dt)
    N = model.latent
    assert h * N // 64 > 64  # too many blocks for the two-launch layer
    ctx = ffi.default_context(0)
    prompt = np.random.default_rng(3).integers(0, 256, size=(1, 9))
    runs = {}
    for fused in (1, 0):
        ctx.set_option("model.fused_rows", fused)
        try:
            st = model.init_state()
            lg, nxt = model.forward_with_state(torch.from_numpy(prompt), st, want_next=True)
            steps = []
            for _ in range(12):
                lg, nxt2 = model.forward_with_state(nxt.reshape(1, 1), st, want_next=True)
                steps.append((lg.cpu().numpy(), int(nxt[0])))
                nxt = nxt2
            torch.cuda.synchronize()
            runs[fused] = (steps, st.storage.float().cpu().numpy())
        finally:
            ctx.set_option("model.fused_rows", 1)
    tol_pair, tol_orc = (1e-5, 1e-3) if state == "f32" else (2e-2, 2e-2)
    rho_ref = np.zeros((3, 1, h, N, d), np.float32)
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, prompt, rho_ref, 0)
    for (lg1, tok1), (lg0, tok0) in zip(*[runs[k][0] for k in (1, 0)]):
        assert tok1 == tok0
        assert rel_err(lg1, lg0) < tol_pair
        logits_ref, pos, _, _ = corc.forward_with_state(shape, w, np.array([[tok1]]), rho_ref, pos)
        assert rel_err(lg1, logits_ref) < tol_orc
    assert rel_err(runs[1][1], runs[0][1]) < tol_pair
    assert rel_err(runs[1][1], rho_ref) < tol_orc
    # other summation trees: the two forms do not give the same bits, so the option did select another path
    assert any(not np.array_equal(a[0], b[0]) for a, b in zip(runs[1][0], runs[0][0]))
