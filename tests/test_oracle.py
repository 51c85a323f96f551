"""Pins the CPU oracle (oracle/bdh_oracle.c and oracle/bdh_oracle.py) before it is
trusted as the checker for the HIP path.

Sources of truth used here, none of which is the oracle's own formula retyped:
  * the recipes, shapes and tolerances of the reference's own tests
    (tests/fused_kernel_tests.rs, tests/model_paths.rs, src/model/attention.rs:384-432);
  * library routines (torch layer_norm, numpy float64 matmul);
  * closed forms and invariants of the mathematics (brute-force causal sums in
    float64, chunk consistency, rotation invariants).
CPU only; the whole file runs in well under a minute.
"""
import math

import numpy as np
import pytest

from oracle import bdh_oracle as orc
from oracle.bdh_oracle import ALIBI, POPE, ROPE


def assert_close(lhs, rhs, atol, rtol):
    """tests/fused_kernel_tests.rs:13-33."""
    lhs, rhs = np.asarray(lhs, np.float64), np.asarray(rhs, np.float64)
    assert lhs.shape == rhs.shape
    bad = np.abs(lhs - rhs) > atol + rtol * np.abs(rhs)
    assert not bad.any(), f"max diff {np.abs(lhs - rhs).max()}"


# ---------------------------------------------------------------- build_freqs
@pytest.mark.parametrize("latent", [8, 64, 8192])
def test_build_freqs_closed_form(corc, latent):
    # closed form in exact arithmetic: f_i = theta^(-2*floor(i/2)/N) / (2 pi)
    i = np.arange(latent)
    for rotary, expo in ((ROPE, 2 * (i // 2) / latent), (POPE, i / latent)):
        exact = 65536.0 ** (-expo) / (2 * math.pi)
        c = corc.build_freqs(latent, 65536.0, rotary)
        n = orc.build_freqs(latent, 65536.0, rotary)
        np.testing.assert_allclose(c, exact, rtol=3e-6)
        np.testing.assert_allclose(n, exact, rtol=3e-6)
        if rotary == ROPE:
            assert np.array_equal(c[0::2], c[1::2])  # one frequency per lane pair
    assert corc.build_freqs(latent, 65536.0, ROPE)[0] == np.float32(1.0 / np.float32(2.0 * np.float32(np.pi)))
    assert not corc.build_freqs(latent, 65536.0, ALIBI).any()  # src/model/attention.rs:368


# -------------------------------------------------------------------- rotate
def _rope_by_pairs(x, freqs, start):
    """Textbook 2-D rotation of each lane pair by angle 2*pi*frac(pos*f) in float64."""
    B, h, T, N = x.shape
    out = np.empty_like(x, dtype=np.float64)
    for t in range(T):
        raw = np.float32(start + t) * freqs.astype(np.float32)  # the f32 product IS the definition
        ang = (raw.astype(np.float64) - np.floor(raw.astype(np.float64))) * 2 * math.pi
        c, s = np.cos(ang[0::2]), np.sin(ang[0::2])
        e, o = x[:, :, t, 0::2].astype(np.float64), x[:, :, t, 1::2].astype(np.float64)
        out[:, :, t, 0::2] = e * c - o * s
        out[:, :, t, 1::2] = o * c + e * s
    return out


def test_rope_matches_pair_rotation_and_invariants(corc):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((2, 3, 5, 16)).astype(np.float32)
    freqs = corc.build_freqs(16)
    for start in (0, 3, 4095):
        qc = corc.rotate(x, freqs, ROPE, start)
        qn = orc.rotate(x, freqs, ROPE, start)
        ref = _rope_by_pairs(x, freqs, start)
        np.testing.assert_allclose(qc, ref, atol=2e-6)
        np.testing.assert_allclose(qn, ref, atol=2e-6)
        # rotation preserves the norm of every lane pair
        np.testing.assert_allclose(qc[..., 0::2] ** 2 + qc[..., 1::2] ** 2,
                                   x[..., 0::2] ** 2 + x[..., 1::2] ** 2, rtol=1e-5, atol=1e-6)
    # position 0 is the identity (phase 0: cos 1, sin 0)
    assert np.array_equal(corc.rotate(x[:, :, :1], freqs, ROPE, 0), x[:, :, :1])


def test_rope_scores_depend_on_relative_position_only():
    # float64 numpy statement: <rot_t(a), rot_s(b)> == <rot_{t+k}(a), rot_{s+k}(b)>
    rng = np.random.default_rng(8)
    N = 32
    a = rng.standard_normal((1, 1, 1, N))
    b = rng.standard_normal((1, 1, 1, N))
    # frequencies whose products with integer positions are exact in binary
    freqs = np.repeat(2.0 ** -np.arange(1, N // 2 + 1), 2)
    def score(t, s):
        return float((orc.rotate(a, freqs, ROPE, t) * orc.rotate(b, freqs, ROPE, s)).sum())
    assert abs(score(5, 2) - score(105, 102)) < 1e-9
    assert abs(score(5, 2) - score(6, 2)) > 1e-6  # and it does depend on t - s


def test_pope_magnitude_and_layout(corc):
    rng = np.random.default_rng(9)
    x = rng.standard_normal((1, 2, 4, 8)).astype(np.float32)
    freqs = corc.build_freqs(8, 65536.0, POPE)
    for q in (corc.rotate(x, freqs, POPE, 11), orc.rotate(x, freqs, POPE, 11)):
        assert q.shape == (1, 2, 4, 16)  # cat(real, imag) doubles the latent
        mag = np.log1p(np.exp(x.astype(np.float64)))  # softplus
        np.testing.assert_allclose(q[..., :8] ** 2 + q[..., 8:] ** 2, mag ** 2, rtol=2e-5)
        ang = np.arctan2(q[..., 8:], q[..., :8]) % (2 * math.pi)
        raw = np.float32(11 + np.arange(4)).reshape(4, 1) * freqs.reshape(1, 8)
        np.testing.assert_allclose(ang, np.broadcast_to((raw % 1.0) * 2 * math.pi, ang.shape), atol=1e-5)


def test_alibi_rotate_is_identity(corc):
    x = np.arange(24, dtype=np.float32).reshape(1, 2, 3, 4)
    assert np.array_equal(corc.rotate(x, np.zeros(4, np.float32), ALIBI, 5), x)
    assert orc.rotate(x, np.zeros(4, np.float32), ALIBI, 5) is x


# ---------------------------------------------------------------- layer_norm
def test_layer_norm_matches_library(corc):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(10)
    x = (3.0 * rng.standard_normal((6, 5, 256)) + 1.5).astype(np.float32)
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x), (256,), eps=1e-5).numpy()
    np.testing.assert_allclose(corc.layer_norm(x), ref, atol=2e-6, rtol=1e-5)
    np.testing.assert_allclose(orc.layer_norm(x), ref, atol=2e-6, rtol=1e-5)
    y = corc.layer_norm(x).astype(np.float64)
    assert np.abs(y.mean(-1)).max() < 1e-6 and np.abs(y.var(-1) - 1).max() < 1e-3


# -------------------------------------------------------------- relu_lowrank
def test_relu_lowrank_reference_recipe(corc):
    """tests/fused_kernel_tests.rs:35-68: input [2,1,5,6], weight [1,3,6,8], bias [3,1,8],
    threshold 0.25, BlockPattern1d::from_blocks(3, [0, 2]); tolerance 1e-5/1e-5."""
    rng = np.random.default_rng(42)
    inp = rng.standard_normal((2, 1, 5, 6)).astype(np.float32)
    weight = rng.standard_normal((3, 6, 8)).astype(np.float32)
    bias = (0.5 * rng.standard_normal((3, 1, 8))).astype(np.float32)
    ref = np.matmul(inp.astype(np.float64), weight.astype(np.float64)[None]) + bias.astype(np.float64).reshape(1, 3, 1, 8)
    ref = np.maximum(ref - 0.25, 0)
    mask = np.array([1, 1, 1, 0, 0, 0, 1, 1], np.float64)  # blocks {0,2} of size 3 over 8 lanes
    ref = ref * mask
    got_c = corc.relu_lowrank(inp, weight, bias.reshape(3, 8), 0.25, 3, [0, 2])
    got_n = orc.relu_lowrank(inp, weight, bias.reshape(3, 8), 0.25, 3, [0, 2])
    assert got_c.shape == (2, 3, 5, 8)
    assert_close(got_c, ref, 1e-5, 1e-5)
    assert_close(got_n, ref, 1e-5, 1e-5)
    assert (got_c[..., 3:6] == 0).all()
    # dense pattern, no bias, threshold 0 == plain relu(matmul)  (src/model/bdh.rs:346-350)
    plain = np.maximum(np.matmul(inp.astype(np.float64), weight.astype(np.float64)[None]), 0)
    assert_close(corc.relu_lowrank(inp, weight), plain, 1e-5, 1e-5)


def test_relu_lowrank_per_head_input(corc):
    rng = np.random.default_rng(43)
    inp = rng.standard_normal((2, 3, 4, 6)).astype(np.float32)  # the D_y call: one input per head
    weight = rng.standard_normal((3, 6, 8)).astype(np.float32)
    ref = np.maximum(np.einsum("bhtk,hkn->bhtn", inp.astype(np.float64), weight.astype(np.float64)), 0)
    assert_close(corc.relu_lowrank(inp, weight), ref, 1e-5, 1e-5)
    assert_close(orc.relu_lowrank(inp, weight), ref, 1e-5, 1e-5)


# ------------------------------------------------- fused_state_aligned / forward
@pytest.mark.parametrize("rotary,seed", [(ROPE, 1337), (POPE, 2024)])
def test_fused_attention_matches_dense_reference(corc, rotary, seed):
    """tests/fused_kernel_tests.rs:70-170: B=1, h=2, T=6, N=8, dv=6, block 3, tol 1e-4."""
    rng = np.random.default_rng(seed)
    query = rng.standard_normal((1, 2, 6, 8)).astype(np.float32)
    value = rng.standard_normal((1, 6, 6)).astype(np.float32)
    freqs = corc.build_freqs(8, 65536.0, rotary)
    # dense statement in float64, written as the test file does (scores.tril(-1), row normalise)
    q = orc.rotate(query.astype(np.float64), freqs.astype(np.float64), rotary, 0)
    scores = np.tril(q @ np.swapaxes(q, 2, 3), -1)
    scores = scores / (np.abs(scores).sum(3, keepdims=True) + 1e-6)
    reference = scores @ value.astype(np.float64)[:, None]
    for impl in (corc, orc):
        fused = impl.fused_state_aligned(query, value, freqs, None, 3, rotary)
        dense = impl.attention_forward(query, value, freqs, None, rotary, True)
        assert_close(fused, reference, 1e-4, 1e-4)
        assert_close(dense, reference, 1e-4, 1e-4)
    # block size must not matter for a dense pattern (incl. a ragged last block)
    for blk in (1, 2, 4, 6, 64):
        assert_close(corc.fused_state_aligned(query, value, freqs, None, blk, rotary), reference, 1e-4, 1e-4)


def test_alibi_decay_kat(corc):
    """src/model/attention.rs:384-403."""
    for dec in (corc.alibi_decay([0.5, 1.0]), orc.alibi_decay(np.array([0.5, 1.0], np.float32))):
        assert abs(dec[0] - math.exp(-0.5)) < 1e-6 and abs(dec[1] - math.exp(-1.0)) < 1e-6


def test_alibi_forward_kat(corc):
    """src/model/attention.rs:405-432: q=[1,1] (N=1,T=2), v=[1,3], slope 0.5 -> out[0]=0, out[1]~=1."""
    query = np.array([1.0, 1.0], np.float32).reshape(1, 1, 2, 1)
    value = np.array([1.0, 3.0], np.float32).reshape(1, 2, 1)
    freqs = np.zeros(1, np.float32)
    for impl in (corc, orc):
        out = impl.attention_forward(query, value, freqs, [0.5], ALIBI, True).reshape(-1)
        assert abs(out[0]) < 1e-6 and abs(out[1] - 1.0) < 1e-4


def test_default_alibi_slopes(corc):
    """src/kernel/linear_attention.rs:152-163: 2^(-i/h)."""
    np.testing.assert_allclose(corc.default_alibi_slopes(4), 2.0 ** (-np.arange(4) / 4), rtol=1e-6)
    np.testing.assert_allclose(orc.default_alibi_slopes(4), 2.0 ** (-np.arange(4) / 4), rtol=1e-6)
    assert corc.default_alibi_slopes(0).size == 0


def test_fused_alibi_block_form_c_equals_numpy(corc):
    # the ALiBi term of the blocked form is added to whole blocks (linear_attention.rs:97-100);
    # the two independent restatements must agree on that, and with the hand value below
    rng = np.random.default_rng(5)
    query = np.abs(rng.standard_normal((1, 2, 5, 4))).astype(np.float32)
    value = rng.standard_normal((1, 5, 3)).astype(np.float32)
    sl = [0.5, 0.25]
    a = corc.fused_state_aligned(query, value, np.zeros(4, np.float32), sl, 2, ALIBI)
    b = orc.fused_state_aligned(query, value, np.zeros(4, np.float32), sl, 2, ALIBI)
    assert_close(a, b, 1e-5, 1e-5)
    # hand value, first row of head 0, block size 2: scores row 0 = [0 (tril), 0 + 0.5*(1-0)]
    # -> normalised [0, 1] -> out = v[1]
    np.testing.assert_allclose(a[0, 0, 0], value[0, 1], atol=1e-4)


# ------------------------------------------------------- recurrent_attention
def _rand_qv(seed, B=2, h=2, T=7, N=12, d=5, density=0.4, dtype=np.float32):
    rng = np.random.default_rng(seed)
    x = np.maximum(rng.standard_normal((B, h, T, N)) - (0.0 if density > 0.45 else 0.3), 0).astype(dtype)
    v = rng.standard_normal((B, T, d)).astype(dtype)
    return x, v


def test_recurrent_equals_strictly_causal_sum_bruteforce(corc):
    """out_t = sum_{s<t} (q_t . q_s) v_s, checked term by term in float64."""
    x, v = _rand_qv(21)
    freqs = corc.build_freqs(x.shape[-1])
    q = corc.rotate(x, freqs, ROPE, 3)
    B, h, T, N = q.shape
    brute = np.zeros((B, h, T, v.shape[-1]))
    for b in range(B):
        for hh in range(h):
            for t in range(T):
                for s in range(t):
                    brute[b, hh, t] += float(np.dot(q[b, hh, t].astype(np.float64), q[b, hh, s].astype(np.float64))) * v[b, s].astype(np.float64)
    rho0 = np.zeros((B, h, N, v.shape[-1]), np.float32)
    out_c, rho_c = corc.recurrent_attention(q, v, rho0)
    out_n, rho_n = orc.recurrent_attention(q, v, rho0)
    np.testing.assert_allclose(out_c, brute, atol=2e-5, rtol=1e-5)
    np.testing.assert_allclose(out_n, brute, atol=2e-5, rtol=1e-5)
    np.testing.assert_allclose(orc.causal_unnormalised(q.astype(np.float64), v.astype(np.float64)), brute, atol=1e-10)
    # first token reads an all-zero state; final state is Q^T V
    assert not out_c[:, :, 0].any()
    qtv = np.einsum("bhtn,btd->bhnd", q.astype(np.float64), v.astype(np.float64))
    np.testing.assert_allclose(rho_c, qtv, atol=2e-5, rtol=1e-5)
    np.testing.assert_allclose(rho_n, qtv, atol=2e-5, rtol=1e-5)
    # after exactly one token the state is q0 (x) v0 with a single rounding per element
    _, rho1 = corc.recurrent_attention(q[:, :, :1], v[:, :1], rho0)
    assert np.array_equal(rho1, q[:, :, 0, :, None] * v[:, None, 0, None, :])


def test_recurrent_chunk_consistency_and_sparse_form(corc):
    x, v = _rand_qv(22, T=9)
    freqs = corc.build_freqs(x.shape[-1])
    B, h, T, N = x.shape
    rho0 = (0.01 * np.random.default_rng(1).standard_normal((B, h, N, v.shape[-1]))).astype(np.float32)
    q_all = corc.rotate(x, freqs, ROPE, 10)
    out_all, rho_all = corc.recurrent_attention(q_all, v, rho0)
    # [0,a) then [a,T) with the rotation restarted at the right position == one call
    a = 4
    q1 = corc.rotate(x[:, :, :a], freqs, ROPE, 10)
    q2 = corc.rotate(x[:, :, a:], freqs, ROPE, 10 + a)
    o1, r1 = corc.recurrent_attention(q1, v[:, :a], rho0)
    o2, r2 = corc.recurrent_attention(q2, v[:, a:], r1)
    assert np.array_equal(np.concatenate([o1, o2], 2), out_all)
    assert np.array_equal(r2, rho_all)
    # sparse-row form: values compare equal to the dense form
    out_s, rho_s = corc.recurrent_attention(q_all, v, rho0, sparse=True)
    assert np.array_equal(out_s, out_all) and np.array_equal(rho_s, rho_all)
    # numpy statement agrees to reassociation noise
    out_n, rho_n = orc.recurrent_attention(q_all, v, rho0)
    np.testing.assert_allclose(out_n, out_all, atol=1e-5, rtol=1e-5)
    np.testing.assert_allclose(rho_n, rho_all, atol=1e-6, rtol=1e-6)


def test_recurrent_alibi_decay(corc):
    """src/model/bdh.rs:299-301: the state is scaled by exp(-slope_h) AFTER each update, so
    out_t = sum_{s<t} exp(-slope (t-s)) (q_t.q_s) v_s."""
    x, v = _rand_qv(23, T=6)
    B, h, T, N = x.shape
    slopes = np.array([0.5, 0.125], np.float32)
    decay = corc.alibi_decay(slopes)
    out_c, rho_c = corc.recurrent_attention(x, v, np.zeros((B, h, N, v.shape[-1]), np.float32), decay)
    out_n, _ = orc.recurrent_attention(x, v, np.zeros((B, h, N, v.shape[-1]), np.float32), decay)
    brute = np.zeros(out_c.shape)
    for hh in range(h):
        for t in range(T):
            for s in range(t):
                w = math.exp(-float(slopes[hh]) * (t - s))
                brute[:, hh, t] += w * np.einsum("bn,bn->b", x[:, hh, t].astype(np.float64), x[:, hh, s].astype(np.float64))[:, None] * v[:, s].astype(np.float64)
    np.testing.assert_allclose(out_c, brute, atol=2e-5, rtol=2e-5)
    np.testing.assert_allclose(out_n, brute, atol=2e-5, rtol=2e-5)


def test_state_step_dense_is_rotate_plus_recurrent(corc):
    rng = np.random.default_rng(24)
    B, h, N, d = 2, 2, 16, 8
    x = np.maximum(rng.standard_normal((B, h, N)) - 1.0, 0).astype(np.float32)
    v = rng.standard_normal((B, d)).astype(np.float32)
    rho = (0.01 * rng.standard_normal((B, h, N, d))).astype(np.float32)
    freqs = corc.build_freqs(N)
    q = corc.rotate(x[:, :, None], freqs, ROPE, 77)
    out_ref, rho_ref = corc.recurrent_attention(q, v[:, None], rho)
    rho_step = rho.copy()
    out = corc.state_step_dense(x, v, freqs, 77, rho_step)
    assert np.array_equal(out, out_ref[:, :, 0]) and np.array_equal(rho_step, rho_ref)


# -------------------------------------------------------- forward_with_state
def _small_shape(rotary):
    """tests/model_paths.rs:12-24: L=2, d=16, h=2, mult=4, V=32."""
    return orc.BDHShape(n_layer=2, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=32, rotary=rotary)


@pytest.mark.parametrize("rotary", [ROPE, POPE, ALIBI])
def test_forward_with_state_shapes_and_position(corc, rotary):
    """tests/model_paths.rs:66-91: tokens [[0,1,2,3],[4,5,6,7]] -> logits [2,4,32], position 4."""
    shape = _small_shape(rotary)
    w = orc.init_weights(shape, seed=3)
    tokens = np.arange(8).reshape(2, 4)
    N = shape.latent_per_head
    assert N == 32
    Nq = 2 * N if rotary == POPE else N
    rho = np.zeros((2, 2, 2, Nq, 16), np.float32)
    logits_c, pos, _, _ = corc.forward_with_state(shape, w, tokens, rho, 0, sparse_state=False)
    st = orc.ModelState(2)
    logits_n = orc.forward_with_state(shape, w, tokens, st)
    assert logits_c.shape == (2, 4, 32) and logits_n.shape == (2, 4, 32)
    assert pos == 4 and st.position == 4
    # the two independent restatements agree (reassociation noise through 2 layers)
    np.testing.assert_allclose(logits_c, logits_n, atol=2e-4, rtol=2e-3)
    for l in range(2):
        np.testing.assert_allclose(rho[l], st.rho[l], atol=2e-5, rtol=1e-3)
    assert np.isfinite(logits_c).all()


@pytest.mark.parametrize("rotary", [ROPE, ALIBI])
def test_forward_decode_equals_prefill(corc, rotary):
    """T tokens in one call == T single-token calls carrying the state (same rho, same logits)."""
    shape = _small_shape(rotary)
    w = orc.init_weights(shape, seed=4)
    tokens = np.array([[5, 1, 9, 30, 2, 2], [0, 31, 7, 7, 12, 3]])
    N = shape.latent_per_head
    rho_a = np.zeros((2, 2, 2, N, 16), np.float32)
    logits_a, pos_a, xa, _ = corc.forward_with_state(shape, w, tokens, rho_a, 0, taps=True, sparse_state=False)
    rho_b = np.zeros_like(rho_a)
    pos_b = 0
    rows = []
    for t in range(tokens.shape[1]):
        lg, pos_b, _, _ = corc.forward_with_state(shape, w, tokens[:, t : t + 1], rho_b, pos_b, sparse_state=(rotary == ROPE))
        rows.append(lg)
    assert pos_a == pos_b == 6
    np.testing.assert_array_equal(np.concatenate(rows, 1), logits_a)  # same op order -> identical
    np.testing.assert_array_equal(rho_a, rho_b)
    # random-init weights give about half the neurons active (zero-mean pre-activations)
    frac = (xa > 0).mean()
    assert 0.35 < frac < 0.65


def test_rho_energy_is_the_batch_mean_of_row_mean_abs(corc):
    """src/model/bdh.rs:411-419 against a float64 library statement."""
    rng = np.random.default_rng(41)
    rho = rng.standard_normal((3, 2, 10, 24)).astype(np.float32)
    want = np.abs(rho.astype(np.float64)).mean(axis=3).mean(axis=0)
    np.testing.assert_allclose(corc.rho_energy(rho), want, rtol=2e-6)
    np.testing.assert_allclose(orc.rho_energy(rho), want, rtol=2e-6)
    # one hot row: energy = |value| / d / B at that neuron only
    one = np.zeros((2, 1, 4, 8), np.float32)
    one[1, 0, 2, 5] = -3.0
    e = corc.rho_energy(one)
    assert e[0, 2] == np.float32(3.0 / 8 / 2) and np.count_nonzero(e) == 1


@pytest.mark.parametrize("rotary", [ROPE, POPE, ALIBI])
def test_forward_viz_taps(corc, rotary):
    """LayerVizState (src/model/bdh.rs:386-434): last token of the first sequence, energy of the updated
    state; the C and numpy restatements agree and the taps are consistent with the plain forward."""
    shape = _small_shape(rotary)
    w = orc.init_weights(shape, seed=6)
    tokens = np.array([[5, 1, 9, 30, 2], [0, 31, 7, 7, 12]])
    N, h, d, L = shape.latent_per_head, 2, 16, 2
    Nq = 2 * N if rotary == POPE else N
    rho = np.zeros((L, 2, h, Nq, d), np.float32)
    logits, pos, viz = corc.forward_with_state_viz(shape, w, tokens, rho, 0, sparse_state=False)
    rho_plain = np.zeros_like(rho)
    logits_plain, _, x_tap, _ = corc.forward_with_state(shape, w, tokens, rho_plain, 0, taps=True, sparse_state=False)
    np.testing.assert_array_equal(logits, logits_plain)
    np.testing.assert_array_equal(rho, rho_plain)
    assert pos == 5 and viz.shape == (L, 4, h, N)
    st = orc.ModelState(L)
    taps = {}
    orc.forward_with_state(shape, w, tokens, st, taps)
    for l in range(L):
        np.testing.assert_array_equal(viz[l, 0], x_tap[l, 0, :, -1])  # x_last = x[b=0, :, T-1]
        np.testing.assert_array_equal(viz[l, 2], viz[l, 0] * viz[l, 1])  # xy = x * y
        assert (viz[l, 1] >= 0).all() and (viz[l, 1] > 0).any()
        nv = taps["viz"][l]
        np.testing.assert_allclose(viz[l, 0], nv["x_last"], atol=2e-5, rtol=1e-3)
        np.testing.assert_allclose(viz[l, 1], nv["y_last"], atol=2e-5, rtol=1e-3)
        np.testing.assert_allclose(viz[l, 2], nv["xy_last"], atol=2e-6, rtol=1e-3)
        np.testing.assert_allclose(viz[l, 3], nv["rho_last"], atol=1e-7, rtol=1e-3)
        if rotary == POPE:
            assert not viz[l, 3].any()  # state rows 2N != N: the reference stores zeros
        else:
            np.testing.assert_allclose(viz[l, 3], np.abs(rho[l].astype(np.float64)).mean(3).mean(0), rtol=1e-5)


@pytest.mark.parametrize("rotary,fused", [(ROPE, False), (POPE, False), (ALIBI, False), (ALIBI, True)])
def test_forward_fast_shapes_and_relation_to_the_parts(rotary, fused):
    """tests/model_paths.rs:44-50,77-83: tokens [[0,1,2,3],[4,5,6,7]] -> logits [2,4,32] for the four
    configurations; the first token's attention row is empty, so its logits are those of a model whose
    attention output is zero (LN(0) = 0 -> y = relu(0) = 0 -> the layer is the identity on LN(embed))."""
    shape = _small_shape(rotary)
    w = orc.init_weights(shape, seed=3)
    tokens = np.arange(8).reshape(2, 4)
    logits = orc.forward_fast(shape, w, tokens, fused=fused, time_block=4)
    assert logits.shape == (2, 4, 32) and np.isfinite(logits).all()
    if not (fused and rotary == ALIBI):  # the fused ALiBi branch lets row 0 see its block through the bias
        cur0 = orc.layer_norm(w.embed[tokens[:, 0]])
        for _ in range(shape.n_layer):
            cur0 = orc.layer_norm(cur0 + orc.layer_norm(np.zeros_like(cur0)))
        np.testing.assert_allclose(logits[:, 0], cur0 @ w.lm_head, atol=1e-5)
    # causal: changing the last token leaves the earlier positions alone
    tokens2 = tokens.copy()
    tokens2[:, -1] = [9, 10]
    logits2 = orc.forward_fast(shape, w, tokens2, fused=fused, time_block=4)
    if not (fused and rotary == ALIBI):
        np.testing.assert_array_equal(logits2[:, :-1], logits[:, :-1])
    assert not np.array_equal(logits2[:, -1], logits[:, -1])


def test_forward_rejects_bad_token(corc):
    shape = _small_shape(ROPE)
    w = orc.init_weights(shape, seed=4)
    rho = np.zeros((2, 1, 2, 32, 16), np.float32)
    with pytest.raises(ValueError):
        corc.forward_with_state(shape, w, np.array([[32]]), rho, 0)


def test_greedy_is_argmax(corc):
    rng = np.random.default_rng(6)
    for _ in range(5):
        row = rng.standard_normal(256).astype(np.float32)
        assert corc.greedy_token(row) == int(np.argmax(row)) == orc.greedy_token(row)


def test_latent_per_head_matches_config_rule():
    """src/model/config.rs:141-155."""
    assert orc.BDHShape().latent_per_head == 256  # defaults: mult 4, d 256, h 4
    assert orc.BDHShape(mlp_internal_dim_multiplier=128).latent_per_head == 8192
    with pytest.raises(AssertionError):
        _ = orc.BDHShape(n_embd=10, n_head=3, mlp_internal_dim_multiplier=1).latent_per_head


def test_bitmask_and_pair_rows_helpers():
    x = np.zeros((2, 128), np.float32)
    x[0, 0] = 1
    x[0, 65] = 2
    x[1, 127] = 3
    bm = orc.active_bitmask(x)
    assert bm.shape == (2, 2)
    assert bm[0, 0] == 1 and bm[0, 1] == 2 and bm[1, 0] == 0 and bm[1, 1] == np.uint64(1) << np.uint64(63)
    assert orc.pair_closed_rows(x).tolist() == [4, 2]


# ---- sampling (src/generation.rs:26-72): pinned by the softmax of a library, an inverse CDF in
# float64, the argmax special case and the draw frequencies ----
def test_sampler_probabilities_are_the_softmax_of_the_scaled_logits(corc):
    from scipy.special import softmax

    rng = np.random.default_rng(0)
    logits = (3 * rng.standard_normal(69)).astype(np.float32)
    for temperature in (0.5, 1.0, 1.7):
        _, p = corc.sample_from_logits(logits, temperature, None, 0.3)
        assert np.allclose(p, softmax(logits.astype(np.float64) / temperature), rtol=1e-5, atol=1e-9)
        _, p_np = orc.sample_from_logits(logits, temperature, None, 0.3)
        assert np.allclose(p, p_np, rtol=1e-6, atol=1e-9)


def test_sampler_index_is_the_inverse_cdf(corc):
    rng = np.random.default_rng(1)
    logits = rng.standard_normal(50).astype(np.float32)
    _, p = corc.sample_from_logits(logits, 1.0, None, 0.0)
    cdf = np.cumsum(p.astype(np.float64))
    for u in rng.random(300):
        if np.abs(cdf - u * cdf[-1]).min() < 1e-5:  # too close to a boundary for f32 vs f64 to agree
            continue
        want = int(np.searchsorted(cdf[:-1], u * cdf[-1], side="right"))
        assert corc.sample_from_logits(logits, 1.0, None, float(u))[0] == want
        assert orc.sample_from_logits(logits, 1.0, None, float(u))[0] == want
    assert corc.sample_from_logits(logits, 1.0, None, 0.0)[0] == 0
    assert corc.sample_from_logits(logits, 1.0, None, 1.0)[0] == 49  # clamped below 1: the last index


def test_sampler_top_k(corc):
    rng = np.random.default_rng(2)
    logits = rng.standard_normal(256).astype(np.float32)
    for u in (0.0, 0.37, 0.999):  # top_k = 1 is greedy whatever the draw
        assert corc.sample_from_logits(logits, 0.8, 1, u)[0] == int(np.argmax(logits)) == corc.greedy_token(logits)
    _, p = corc.sample_from_logits(logits, 1.0, 5, 0.5)
    assert (p > 0).sum() == 5 and set(np.nonzero(p)[0]) == set(np.argsort(logits)[-5:])
    tied = logits.copy()
    tied[[3, 77]] = np.sort(logits)[-5]  # two more entries equal to the 5th largest: all survive (:43-45)
    _, p = corc.sample_from_logits(tied, 1.0, 5, 0.5)
    assert (p > 0).sum() == 7
    for k in (0, 256, 1000):  # no truncation
        assert (corc.sample_from_logits(logits, 1.0, k, 0.5)[1] > 0).all()


def test_sampler_degenerate_rows_fall_back_to_uniform(corc):
    row = np.full(8, np.nan, np.float32)
    idx, p = corc.sample_from_logits(row, 1.0, None, 0.51)
    assert np.allclose(p, 1 / 8) and idx == 4
    idx, p = corc.sample_from_logits(np.full(8, -np.inf, np.float32), 1.0, None, 0.26)
    assert np.allclose(p, 1 / 8) and idx == 2


def test_sampler_draw_frequencies_follow_the_distribution(corc):
    from scipy.stats import chisquare

    logits = np.array([0.0, 1.0, 2.0, -1.0, 0.5], np.float32)
    _, p = corc.sample_from_logits(logits, 1.0, None, 0.0)
    us = (np.arange(20000) + 0.5) / 20000  # stratified uniforms: frequencies must match p to 1/n
    counts = np.bincount([corc.sample_from_logits(logits, 1.0, None, float(u))[0] for u in us], minlength=5)
    assert np.abs(counts / 20000 - p).max() < 2e-4
    draws = np.random.default_rng(5).random(5000)
    counts = np.bincount([orc.sample_from_logits(logits, 1.0, None, float(u))[0] for u in draws], minlength=5)
    p64 = p.astype(np.float64)
    assert chisquare(counts, p64 / p64.sum() * 5000).pvalue > 1e-3
