"""Golden vectors under tests/golden/ (written by tests/golden/make_fixtures.py from the pinned
oracle).  CPU: the oracle still reproduces them bit for bit.  GPU: the HIP path matches them."""
import os

import numpy as np
import pytest

from oracle import bdh_oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = ["rope_d256", "rope_small", "alibi_small", "pope_small"]


def load_case(name):
    z = np.load(os.path.join(GOLDEN, "state_step.npz"))
    return {k.split(".", 1)[1]: z[k] for k in z.files if k.startswith(name + ".")}


@pytest.mark.parametrize("name", CASES)
def test_oracle_reproduces_state_step_fixture(corc, name):
    c = load_case(name)
    rotary = int(c["rotary"])
    decay = corc.alibi_decay(c["slopes"]) if c["slopes"].size else None
    assert np.array_equal(corc.build_freqs(c["x"].shape[-1], 65536.0, rotary), c["freqs"])
    q = corc.rotate(c["x"], c["freqs"], rotary, int(c["position"]))
    out, rho1 = corc.recurrent_attention(q, c["v"], c["rho0"], decay)
    assert np.array_equal(out, c["out"]) and np.array_equal(rho1, c["rho1"])
    # the numpy restatement agrees with the frozen vectors to reassociation noise
    out_n, rho_n = orc.recurrent_attention(orc.rotate(c["x"], c["freqs"], rotary, int(c["position"])), c["v"], c["rho0"], decay)
    np.testing.assert_allclose(out_n, c["out"], atol=2e-5, rtol=1e-4)
    np.testing.assert_allclose(rho_n, c["rho1"], atol=2e-6, rtol=1e-5)


def test_oracle_reproduces_model_fixture(corc):
    z = np.load(os.path.join(GOLDEN, "model_paths_rope.npz"))
    shape = orc.BDHShape(n_layer=2, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=32, rotary=orc.ROPE)
    w = orc.init_weights(shape, seed=int(z["seed"]))
    rho = np.zeros_like(z["rho"])
    logits, pos, _, _ = corc.forward_with_state(shape, w, z["tokens"], rho, 0, sparse_state=False)
    assert pos == int(z["position"]) == 4
    assert np.array_equal(logits, z["logits"]) and np.array_equal(rho, z["rho"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", CASES)
def test_hip_state_step_matches_fixture(name):
    import torch

    assert torch.cuda.is_available(), "no HIP device"
    from burn_dragon_amd.positional import RotaryEmbedding
    from burn_dragon_amd.recurrent import recurrent_attention

    c = load_case(name)
    dev = "cuda:0"
    rho = torch.from_numpy(c["rho0"]).to(dev)
    slopes = c["slopes"] if c["slopes"].size else None
    out, bm, rows = recurrent_attention(torch.from_numpy(c["x"]).to(dev), torch.from_numpy(c["v"]).to(dev), rho,
                                        torch.from_numpy(c["freqs"]).to(dev), int(c["position"]),
                                        RotaryEmbedding(int(c["rotary"])), slopes, want_bitmask=True, want_rows=True)
    torch.cuda.synchronize()
    scale = np.abs(c["out"]).max()
    assert np.abs(out.cpu().numpy() - c["out"]).max() <= 1e-3 * scale  # north_star bound, f32 state
    assert np.abs(rho.cpu().numpy() - c["rho1"]).max() <= 1e-3 * np.abs(c["rho1"]).max()
    assert np.array_equal(bm.cpu().numpy().view(np.uint64), c["bitmask"])  # index sets: bit-exact
    if int(c["rotary"]) == orc.ROPE:
        assert np.array_equal(rows.cpu().numpy(), c["rows"])


@pytest.mark.gpu
def test_hip_model_matches_fixture():
    import torch

    assert torch.cuda.is_available(), "no HIP device"
    import burn_dragon_amd as bda

    z = np.load(os.path.join(GOLDEN, "model_paths_rope.npz"))
    cfg = bda.BDHConfig(n_layer=2, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=32)
    cfg.fused_kernels.set_rotary_embedding(bda.RotaryEmbedding.ROPE)
    shape = orc.BDHShape(n_layer=2, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=32, rotary=orc.ROPE)
    w = orc.init_weights(shape, seed=int(z["seed"]))
    model = bda.BDH(cfg, "cuda:0", weights=vars(w))
    state = model.init_state()
    logits = model.forward_with_state(torch.from_numpy(z["tokens"]), state)
    torch.cuda.synchronize()
    assert state.position == 4
    assert np.abs(logits.cpu().numpy() - z["logits"]).max() <= 1e-3 * np.abs(z["logits"]).max()
