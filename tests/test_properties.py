"""Property tests (hypothesis, CPU) of the host logic and of the oracle: invariants the domain offers,
on generated inputs — tokenizer round trips, record framing, linearity and chunk consistency of the
recurrence, monotonicity of the sampler."""
import numpy as np
import pytest
from hypothesis import HealthCheck, given, settings
from hypothesis import strategies as st

from burn_dragon_amd import record
from burn_dragon_amd.tokenizer import ByteTokenizer, CharVocab
from oracle import bdh_oracle as orc

FAST = settings(max_examples=40, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
text_no_specials = st.text(alphabet=st.characters(min_codepoint=4, blacklist_categories=("Cs",)), max_size=60)


@FAST
@given(text=st.text(alphabet=st.characters(blacklist_categories=("Cs",)), max_size=80), bos=st.booleans(),
       eos=st.booleans())
def test_byte_tokenizer_round_trip(text, bos, eos):
    t = ByteTokenizer(True)
    ids = t.encode(text, bos, eos)
    assert len(ids) == len(text.encode("utf-8")) + bos + eos and max(ids, default=0) < len(t)
    assert t.decode(ids) == text


@FAST
@given(texts=st.lists(text_no_specials, min_size=1, max_size=4), probe=text_no_specials)
def test_char_vocab_round_trip_and_unknowns(texts, probe):
    v = CharVocab.fit(texts, True)
    assert CharVocab.from_json_str(__import__("json").dumps(v.to_record())) == v
    for t in texts:
        assert v.decode(v.encode(t, True, True)) == t
    known = set("".join(texts))
    assert v.decode(v.encode(probe)) == "".join(c if c in known else "?" for c in probe)
    assert len(v) == len(known) + 4


@FAST
@given(h=st.integers(1, 3), d=st.integers(1, 6), mult=st.integers(1, 3), V=st.integers(1, 300), half=st.booleans(),
       seed=st.integers(0, 10), cut=st.floats(0.0, 0.999))
def test_record_framing_round_trip_and_truncation(h, d, mult, V, half, seed, cut):
    N = mult * d  # latent_per_head * h must be a multiple of d
    rng = np.random.default_rng(seed)
    w = {"embed": rng.standard_normal((V, d)), "encoder": rng.standard_normal((h, d, N)),
         "encoder_v": rng.standard_normal((h, d, N)), "decoder": rng.standard_normal((h * N, d)),
         "lm_head": rng.standard_normal((d, V))}
    w = {k: a.astype(np.float32) for k, a in w.items()}
    buf = record.serialize_record(w, half=half)
    meta, params = record.parse_record(buf)
    back = record.weights_from_params(params)
    for k in w:
        want = w[k].astype(np.float16).astype(np.float32) if half else w[k]
        assert np.array_equal(back[k], want)
    assert record.infer_dimensions(back)["vocab_size"] == V
    # any proper prefix either fails cleanly or holds fewer than five complete parameters
    prefix = buf[: int(len(buf) * cut)]
    try:
        _, ps = record.parse_record(prefix)
        assert len(ps) < 5
    except record.RecordError:
        pass


@FAST
@given(seed=st.integers(0, 1000), T=st.integers(1, 6), split=st.integers(0, 6), alpha=st.floats(-2, 2))
def test_recurrence_is_linear_in_the_values_and_chunk_consistent(corc, seed, T, split, alpha):
    rng = np.random.default_rng(seed)
    B, h, N, d = 2, 2, 8, 5
    q = rng.standard_normal((B, h, T, N)).astype(np.float32)
    v1, v2 = (rng.standard_normal((B, T, d)).astype(np.float32) for _ in range(2))
    zero = np.zeros((B, h, N, d), np.float32)
    o1, r1 = corc.recurrent_attention(q, v1, zero)
    o2, r2 = corc.recurrent_attention(q, v2, zero)
    o3, r3 = corc.recurrent_attention(q, (v1 + np.float32(alpha) * v2).astype(np.float32), zero)
    assert np.allclose(o3, o1 + alpha * o2, atol=1e-4) and np.allclose(r3, r1 + alpha * r2, atol=1e-4)
    a = min(split, T)
    oa, ra = corc.recurrent_attention(q[:, :, :a], v1[:, :a], zero)
    ob, rb = corc.recurrent_attention(q[:, :, a:], v1[:, a:], ra)
    assert np.allclose(np.concatenate([oa, ob], 2), o1, atol=1e-5) and np.allclose(rb, r1, atol=1e-5)
    assert not o1[:, :, 0].any()  # the first token reads the zero state


@FAST
@given(seed=st.integers(0, 1000), V=st.integers(1, 40), k=st.integers(0, 45), temperature=st.floats(0.2, 3.0),
       us=st.lists(st.floats(0, 1), min_size=2, max_size=6))
def test_sampler_index_is_in_range_and_monotone_in_the_variate(corc, seed, V, k, temperature, us):
    logits = (2 * np.random.default_rng(seed).standard_normal(V)).astype(np.float32)
    us = sorted(us)
    idx = [corc.sample_from_logits(logits, temperature, k, float(u))[0] for u in us]
    assert all(0 <= i < V for i in idx) and idx == sorted(idx)
    _, p = corc.sample_from_logits(logits, temperature, k, 0.5)
    assert abs(float(p.sum()) - 1) < 1e-4 and all(p[i] > 0 for i in idx)
    if 0 < k < V:
        assert (p > 0).sum() >= k  # ties with the k-th largest survive


@FAST
@given(data=st.data())
def test_damaged_record_framing_fails_cleanly(data):
    """Random byte edits in the framing of a small record: the reader returns or raises RecordError,
    never another exception (no index errors, no huge allocations)."""
    rng = np.random.default_rng(0)
    w = {"embed": rng.standard_normal((5, 4)), "encoder": rng.standard_normal((2, 4, 6)),
         "encoder_v": rng.standard_normal((2, 4, 6)), "decoder": rng.standard_normal((12, 4)),
         "lm_head": rng.standard_normal((4, 5))}
    buf = bytearray(record.serialize_record({k: a.astype(np.float32) for k, a in w.items()}))
    n_edits = data.draw(st.integers(1, 4))
    for _ in range(n_edits):
        pos = data.draw(st.integers(0, len(buf) - 1))
        buf[pos] = data.draw(st.integers(0, 255))
    if data.draw(st.booleans()):
        del buf[data.draw(st.integers(0, len(buf) - 1)):]
    try:
        _, params = record.parse_record(bytes(buf))
        record.weights_from_params(params)
    except record.RecordError:
        pass


def _bf16_rne(a):
    u = np.asarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def _split3_bf16(a):
    """The three-term split the dense f32 products use on the GPU (csrc/attention_parallel.hip, fsa_split3):
    each term is the remainder so far rounded to bf16 (= an f32 with a zero lower half), nearest even."""
    a = np.asarray(a, np.float32)
    h = _bf16_rne(a)
    r1 = a - h
    m = _bf16_rne(r1)
    r2 = r1 - m
    return h, m, _bf16_rne(r2), r1, r2


@FAST
@given(seed=st.integers(0, 2**31 - 1), spread=st.integers(0, 60))
def test_three_bf16_terms_add_up_to_the_float_and_six_products_keep_f32_accuracy(seed, spread):
    """h + m + l == a exactly (both remainders are exact in f32, the third term holds what is left), and
    |a b - (hh + hm + mh + hl + lh + mm)| <= 2^-22 |a b|: the three dropped products."""
    rng = np.random.default_rng(seed)
    n = 4096
    a = (rng.standard_normal(n) * np.exp2(rng.integers(-spread, spread + 1, n))).astype(np.float32)
    b = (rng.standard_normal(n) * np.exp2(rng.integers(-spread, spread + 1, n))).astype(np.float32)
    f = lambda t: t.astype(np.float64)
    ha, ma, la, r1, r2 = _split3_bf16(a)
    assert np.array_equal(f(r1), f(a) - f(ha)) and np.array_equal(f(r2), f(r1) - f(ma))  # exact remainders
    assert np.array_equal(f(ha) + f(ma) + f(la), f(a))
    hb, mb, lb, _, _ = _split3_bf16(b)
    six = f(la) * f(hb) + f(ha) * f(lb) + f(ma) * f(mb) + f(ma) * f(hb) + f(ha) * f(mb) + f(ha) * f(hb)
    exact = f(a) * f(b)
    assert np.all(np.abs(exact - six) <= np.abs(exact) * 2.0**-22)
