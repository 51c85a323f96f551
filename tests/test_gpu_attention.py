"""GPU tests of the Attention mirror (src/model/attention.rs:102-349) through the C ABI: the reference's own
two known-answer tests (attention.rs:383-432), the rotation against the oracle, and forward against the
oracle's statements of both branches.

Tolerances: rotation 2e-6 relative (device sincos against libm); forward 1e-4 on the max-norm."""
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


def _kernel(bda, rotary, fused=False, block=64, slopes=None):
    k = bda.FusedKernelConfig()
    k.enabled = fused
    k.set_block_sizes(block, block)
    k.set_rotary_embedding(bda.RotaryEmbedding.parse(rotary))
    if slopes is not None:
        k.set_alibi_slopes(slopes)
    return k


def test_alibi_decay_matches_exp_neg_slope(bda):
    """src/model/attention.rs:383-402."""
    from burn_dragon_amd.model import Attention

    att = Attention(1, 2, DEV, _kernel(bda, "alibi", slopes=[0.5, 1.0]))
    decay = att.alibi_decay()
    assert np.abs(decay - np.exp(np.array([-0.5, -1.0], np.float32))).max() < 1e-6
    assert Attention(2, 2, DEV, _kernel(bda, "rope")).alibi_decay() is None


@pytest.mark.parametrize("fused", [False, True])
def test_alibi_bias_applies_in_forward(bda, fused):
    """src/model/attention.rs:404-432: q = [1,1], v = [1,3], slope 0.5 -> [0, 1] (plain branch); the
    fused branch adds the bias to the whole diagonal block, so with both tokens in one block row 0 sees
    the future token: scores [[0, 0.5], [0.5, 0]] -> [3, 1]."""
    from burn_dragon_amd.model import Attention

    att = Attention(1, 1, DEV, _kernel(bda, "alibi", fused=fused, slopes=[0.5]))
    query = torch.tensor([1.0, 1.0], device=DEV).reshape(1, 1, 2, 1)
    value = torch.tensor([1.0, 3.0], device=DEV).reshape(1, 1, 2, 1)
    out = att.forward(query, value).cpu().numpy().reshape(-1)
    if not fused:
        assert abs(out[0]) < 1e-6 and abs(out[1] - 1.0) < 1e-4
    else:
        assert abs(out[0] - 3.0) < 1e-4 and abs(out[1] - 1.0) < 1e-4


@pytest.mark.parametrize("rotary", ["rope", "pope", "alibi"])
def test_rotate_positions_matches_oracle(bda, corc, rotary):
    from burn_dragon_amd.model import Attention

    B, h, T, N = 2, 3, 5, 34
    rng = np.random.default_rng(4)
    x = np.maximum(rng.standard_normal((B, h, T, N)), 0).astype(np.float32)
    att = Attention(N, h, DEV, _kernel(bda, rotary))
    code = int(bda.RotaryEmbedding.parse(rotary))
    freqs = corc.build_freqs(N, rotary=code)
    np.testing.assert_array_equal(att.freqs.reshape(-1).cpu().numpy(), freqs)
    got = att.rotate_positions(torch.from_numpy(x).to(DEV), 1234).cpu().numpy()
    want = corc.rotate(x, freqs, code, 1234)
    assert got.shape == want.shape
    assert rel_err(got, want) < 2e-6
    if rotary == "alibi":
        np.testing.assert_array_equal(got, x)
    # per-sequence start positions
    pos = torch.tensor([7, 4000], device=DEV, dtype=torch.int32)
    got = att.rotate_positions(torch.from_numpy(x).to(DEV), 0, pos).cpu().numpy()
    for b, p in enumerate([7, 4000]):
        assert rel_err(got[b : b + 1], corc.rotate(x[b : b + 1], freqs, code, p)) < 2e-6


@pytest.mark.parametrize("rotary", ["rope", "alibi"])
@pytest.mark.parametrize("fused", [False, True])
def test_forward_matches_oracle(bda, corc, rotary, fused):
    """Plain branch == the oracle's Attention::forward; fused branch == its fused_state_aligned with the
    model's time-block size (src/model/attention.rs:142-175)."""
    from burn_dragon_amd.model import Attention

    B, h, T, N, dv, block = 2, 2, 13, 16, 6, 4
    rng = np.random.default_rng(9)
    q = np.maximum(rng.standard_normal((B, h, T, N)), 0).astype(np.float32)
    v = rng.standard_normal((B, 1, T, dv)).astype(np.float32)
    att = Attention(N, h, DEV, _kernel(bda, rotary, fused=fused, block=block))
    out = att.forward(torch.from_numpy(q).to(DEV), torch.from_numpy(v).to(DEV)).cpu().numpy()
    code = int(bda.RotaryEmbedding.parse(rotary))
    freqs = corc.build_freqs(N, rotary=code)
    slopes = att.alibi_slopes.numpy() if rotary == "alibi" else None
    if fused:
        want = corc.fused_state_aligned(q, v, freqs, slopes, block, code)
    else:
        want = corc.attention_forward(q, v, freqs, slopes, code, True)
    assert rel_err(out, want) < 1e-4
    if rotary == "rope":  # without the bias the two branches are the same function
        other = Attention(N, h, DEV, _kernel(bda, rotary, fused=not fused, block=block))
        out2 = other.forward(torch.from_numpy(q).to(DEV), torch.from_numpy(v).to(DEV)).cpu().numpy()
        assert rel_err(out, out2) < 1e-5
