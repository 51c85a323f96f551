"""GPU parity of the LayerVizState by-products of the cached step (the reference's "viz" feature,
src/model/state.rs:17-24, src/model/bdh.rs:386-434) against the CPU oracle, through the C ABI.

Tolerances: the maps are slices of activations of the pinned forward pass (1e-3 relative on the
max-norm, as the logits); the energy map is a sum of |rho|, compared at 1e-4 relative per entry
(f32 state) and 2e-2 (bf16 state).
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


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,h,N,d", [(3, 2, 10, 24), (2, 4, 130, 256), (1, 1, 7, 70), (5, 3, 64, 512)])
def test_rho_energy_matches_oracle(bda, corc, B, h, N, d, dtype):
    from burn_dragon_amd.recurrent import rho_energy

    rng = np.random.default_rng(B * 1000 + N)
    rho = torch.from_numpy(rng.standard_normal((B, h, N, d)).astype(np.float32)).to(dtype)
    got = rho_energy(rho.to(DEV).contiguous()).cpu().numpy()
    want = corc.rho_energy(rho.float().numpy())  # the oracle reads the same (rounded) values
    assert got.shape == (h, N)
    np.testing.assert_allclose(got, want, rtol=1e-5)


def test_rho_energy_of_an_empty_batch_is_zero(bda):
    from burn_dragon_amd.recurrent import rho_energy

    got = rho_energy(torch.zeros((0, 2, 8, 16), device=DEV))
    assert tuple(got.shape) == (2, 8) and not got.any()


def test_rho_energy_reads_a_lazy_alibi_state_through_its_pending_decay(bda, corc):
    """Energy of the lazily decayed state at clock == energy of the materialized state."""
    from burn_dragon_amd.recurrent import alibi_materialize, rho_energy

    rng = np.random.default_rng(77)
    B, h, N, d = 3, 4, 96, 256
    rho = torch.from_numpy(rng.standard_normal((B, h, N, d)).astype(np.float32)).to(DEV)
    stamps = torch.from_numpy(rng.integers(0, 40, (B, h, N)).astype(np.int32)).to(DEV)
    clock = 40
    lazy = rho_energy(rho, stamps, clock).cpu().numpy()
    clocks = torch.full((B,), clock, device=DEV, dtype=torch.int32)
    lazy_dev_clock = rho_energy(rho, stamps, 0, clocks=clocks).cpu().numpy()
    np.testing.assert_array_equal(lazy, lazy_dev_clock)
    eager = rho.clone()
    alibi_materialize(eager, stamps.clone(), clock)
    want = corc.rho_energy(eager.cpu().numpy())
    np.testing.assert_allclose(lazy, want, rtol=2e-5)
    # and it differs from the energy of the raw stored rows
    assert rel_err(rho_energy(rho).cpu().numpy(), want) > 0.05


@pytest.mark.parametrize("lazy", [False, True], ids=["eager", "lazy"])
@pytest.mark.parametrize("rotary", ["rope", "pope", "alibi"])
def test_forward_viz_taps_match_oracle(bda, corc, rotary, lazy):
    if lazy and rotary != "alibi":
        pytest.skip("lazy decay is an ALiBi state format")
    cfg = bda.BDHConfig(n_layer=2, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=32, dropout=0.0)
    cfg.fused_kernels.set_block_sizes(4, 4)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.parse(rotary))
    shape = orc.BDHShape(n_layer=2, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=32,
                         rotary=int(cfg.fused_kernels.rotary_embedding))
    w = orc.init_weights(shape, seed=21)
    model = bda.BDH(cfg, DEV, weights={"embed": w.embed, "encoder": w.encoder, "encoder_v": w.encoder_v,
                                       "decoder": w.decoder, "lm_head": w.lm_head}, alibi_lazy=lazy)
    N, Nq = model.latent, model.latent_q
    rho_ref = np.zeros((2, 2, 2, Nq, 16), np.float32)
    state = model.init_state()
    pos = 0
    for tokens in (np.array([[5, 1, 9, 30, 2], [0, 31, 7, 7, 12]]), np.array([[3], [4]])):  # prefill, then a decode step
        logits = model.forward_with_state(torch.from_numpy(tokens), state, viz=True)
        logits_ref, pos, viz_ref = corc.forward_with_state_viz(shape, w, tokens, rho_ref, pos, sparse_state=False)
        assert rel_err(logits.cpu().numpy(), logits_ref) < 1e-3
        maps = state.take_viz()
        assert len(maps) == 2 and all(m is not None for m in maps)
        assert state.take_viz() == [None, None]  # take_viz empties the slots (src/model/state.rs:59-65)
        for l, m in enumerate(maps):
            for k, name in enumerate(("x_last", "y_last", "xy_last", "rho_last")):
                got = getattr(m, name).cpu().numpy()
                assert got.shape == (2, N)
                assert rel_err(got, viz_ref[l, k]) < 1e-3 or not viz_ref[l, k].any(), (l, name)
            if rotary == "pope":
                assert not m.rho_last.any()
            else:
                np.testing.assert_allclose(m.rho_last.cpu().numpy(), viz_ref[l, 3], rtol=1e-3, atol=1e-9)
            # first-layer activations come from the same k-sequential sums on both sides
            if l == 0:
                np.testing.assert_array_equal(m.x_last.cpu().numpy() > 0, viz_ref[0, 0] > 0)
            np.testing.assert_array_equal((m.xy_last.cpu().numpy()), (m.x_last * m.y_last).cpu().numpy())
    # without viz nothing is stored
    model.forward_with_state(torch.from_numpy(np.array([[1], [2]])), state)
    assert state.take_viz() == [None, None]


def test_viz_taps_on_the_trained_checkpoint(bda, corc):
    """The shipped ALiBi checkpoint: sparse x, sparser xy, and an energy map that matches the oracle's."""
    import os

    from burn_dragon_amd.record import load_checkpoint_dir

    directory = os.path.join(os.path.dirname(__file__), "golden", "tiny_shakespeare")
    model, tok, _ = bda.BDH.from_checkpoint_dir(directory, DEV, alibi_lazy=True)
    _, weights, _, _ = load_checkpoint_dir(directory)
    shape = orc.BDHShape(n_layer=4, n_embd=128, n_head=4, mlp_internal_dim_multiplier=4, vocab_size=69,
                         rotary=orc.ALIBI)
    w = orc.BDHWeights(**weights)
    ids = np.array([tok.encode("To be, or not to be, that is the question:", False, False)])
    state = model.init_state()
    logits = model.forward_with_state(torch.from_numpy(ids), state, viz=True)
    rho_ref = np.zeros((shape.n_layer, 1, shape.n_head, shape.latent_per_head, shape.n_embd), np.float32)
    logits_ref, _, viz_ref = corc.forward_with_state_viz(shape, w, ids, rho_ref, 0, sparse_state=False)
    assert rel_err(logits.cpu().numpy(), logits_ref) < 1e-3
    for l, m in enumerate(state.take_viz()):
        np.testing.assert_allclose(m.rho_last.cpu().numpy(), viz_ref[l, 3], rtol=1e-3, atol=1e-9)
        assert rel_err(m.y_last.cpu().numpy(), viz_ref[l, 1]) < 1e-3
        frac_x = float((m.x_last > 0).float().mean())
        frac_xy = float((m.xy_last > 0).float().mean())
        assert frac_xy <= frac_x < 0.6


def test_viz_state_collects_last_token(bda):
    """src/viz/encoder.rs:314-348, the reference's own test of LayerVizState: L=2, d=8, h=2, mult=2, V=16,
    default (ALiBi) kernel config with fused kernels off, tokens [[1,2,3]] -> one LayerVizState per layer
    whose four maps are [n_head, latent_per_head]."""
    config = bda.BDHConfig()
    config.n_layer, config.n_embd, config.n_head = 2, 8, 2
    config.mlp_internal_dim_multiplier, config.vocab_size, config.dropout = 2, 16, 0.0
    config.fused_kernels.enabled = False
    model = bda.BDH(config, DEV)
    state = bda.ModelState.new(config.n_layer)
    model.forward_with_state(torch.tensor([[1, 2, 3]]), state, viz=True)
    layers = state.take_viz()
    assert len(layers) == config.n_layer
    for layer in layers:
        assert layer is not None, "expected viz state per layer"
        dims = tuple(layer.x_last.shape)
        assert dims == (config.n_head, config.latent_per_head())
        assert tuple(layer.y_last.shape) == dims and tuple(layer.xy_last.shape) == dims
        assert tuple(layer.rho_last.shape) == dims
