"""GPU tests of the generation side: the on-device sampler against the oracle's restatement of
sample_from_logits_values, the trained checkpoint of the reference (tests/golden/tiny_shakespeare,
ALiBi) through the HIP model step against the oracle, and the generation loop.

Tolerances: logits 1e-3 of their max-norm (f32 state); sampled indices bit-exact for every draw that is
not within 1e-5 of a boundary of the cumulative distribution (the device expf and libm's differ in the
last bits)."""
import os

import numpy as np
import pytest
import torch

from oracle import bdh_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
CKPT = os.path.join(os.path.dirname(__file__), "golden", "tiny_shakespeare")
TEXT = ("First Citizen:\nBefore we proceed any further, hear me speak.\n\nAll:\nSpeak, speak.\n\n"
        "First Citizen:\nYou are all resolved rather to die than to famish?\n\nAll:\nResolved. resolved.\n")


@pytest.fixture(scope="module")
def trained():
    if not torch.cuda.is_available():
        pytest.fail("no HIP device: the GPU tests must run on the MI355X box")
    import burn_dragon_amd as bda
    from burn_dragon_amd import record

    model, tok, block_size = bda.BDH.from_checkpoint_dir(CKPT, DEV)
    _, weights, _, _ = record.load_checkpoint_dir(CKPT)
    shape = orc.BDHShape(n_layer=4, n_embd=128, n_head=4, mlp_internal_dim_multiplier=4, vocab_size=69,
                         rotary=orc.ALIBI)
    return model, tok, block_size, shape, orc.BDHWeights(**weights)


def rel_err(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


@pytest.mark.parametrize("V", [5, 69, 256, 259, 1000, 8192])
def test_device_sampler_matches_oracle(trained, corc, V):
    from burn_dragon_amd.generation import sample_from_logits

    model = trained[0]
    rng = np.random.default_rng(V)
    B = 48
    logits = (2.5 * rng.standard_normal((B, V))).astype(np.float32)
    logits[1, : V // 2] = logits[1, 0]  # ties
    us = rng.random(B).astype(np.float32)
    us[0], us[2] = 0.0, 0.99999994
    lt = torch.from_numpy(logits).to(DEV)
    checked = 0
    for temperature, top_k in [(1.0, None), (0.7, 1), (1.3, 4), (0.9, V - 1), (1.0, V + 3), (2.0, 40)]:
        got = sample_from_logits(model, lt, temperature, top_k, torch.from_numpy(us).to(DEV)).cpu().numpy()
        for b in range(B):
            want, p = corc.sample_from_logits(logits[b], temperature, top_k, float(us[b]))
            cdf = np.cumsum(p.astype(np.float64))
            if np.abs(cdf - np.float64(us[b]) * cdf[-1]).min() < 1e-5 and 0 < us[b] < 0.9999:
                continue
            assert got[b] == want, (temperature, top_k, b)
            checked += 1
            if top_k == 1 and b != 1:
                assert got[b] == int(np.argmax(logits[b]))
    assert checked > 5 * B


def test_device_sampler_strided_rows_and_degenerate_input(trained, corc):
    from burn_dragon_amd.generation import sample_from_logits

    model = trained[0]
    full = torch.randn((6, 3, 69), device=DEV, generator=torch.Generator(device=DEV).manual_seed(3))
    last = full[:, -1]  # rows strided by T*V, as the last-token logits of a [B,T,V] tensor are
    u = torch.full((6,), 0.5, device=DEV)
    got = sample_from_logits(model, last, 1.0, 10, u).cpu().numpy()
    for b in range(6):
        assert got[b] == corc.sample_from_logits(last[b].cpu().numpy(), 1.0, 10, 0.5)[0]
    nan_rows = torch.full((2, 8), float("nan"), device=DEV)
    assert sample_from_logits(model, nan_rows, 1.0, None, torch.tensor([0.51, 0.26], device=DEV)).tolist() == [4, 2]
    from burn_dragon_amd import ffi

    with pytest.raises(ffi.BdhError) as err:
        sample_from_logits(model, torch.zeros((1, 9000), device=DEV), 1.0, None, torch.zeros(1, device=DEV))
    assert err.value.status == ffi.E_SHAPE


def test_trained_checkpoint_matches_oracle_and_predicts_the_text(trained, corc):
    model, tok, _, shape, w = trained
    ids = np.array([tok.encode(TEXT)])
    state = model.init_state()
    logits = model.forward_with_state(torch.from_numpy(ids), state).cpu().numpy()
    rho_ref = np.zeros((4, 1, 4, 128, 128), np.float32)
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, ids, rho_ref, 0, sparse_state=False)
    assert rel_err(logits, logits_ref) < 1e-3
    assert rel_err(state.storage.cpu().numpy(), rho_ref) < 1e-3 and state.position == pos == ids.shape[1]
    z = logits[0].astype(np.float64)
    logp = z - z.max(-1, keepdims=True)
    logp -= np.log(np.exp(logp).sum(-1, keepdims=True))
    loss = float(-logp[np.arange(ids.shape[1] - 1), ids[0, 1:]].mean())
    assert loss < 1.35, loss  # uniform would be ln 69 = 4.23


def test_greedy_generation_from_the_checkpoint_follows_the_oracle(trained, corc):
    from burn_dragon_amd.generation import GenerationSettings, generate_tokens

    model, tok, _, shape, w = trained
    prompt = tok.encode("First Citizen:\n")
    n_new = 48
    tokens = generate_tokens(model, prompt, GenerationSettings(max_new_tokens=n_new, temperature=1.0, top_k=1))
    assert tokens[: len(prompt)] == prompt and len(tokens) == len(prompt) + n_new
    # oracle: greedy with the same rule; a step whose two best logits are closer than the tolerance may differ
    rho = np.zeros((4, 1, 4, 128, 128), np.float32)
    logits, pos, _, _ = corc.forward_with_state(shape, w, np.array([prompt]), rho, 0, sparse_state=False)
    for i in range(n_new):
        best = corc.greedy_token(logits[0, -1])
        got = tokens[len(prompt) + i]
        if got != best:
            top = np.sort(logits[0, -1])[-2:]
            assert top[1] - top[0] < 1e-3 * np.abs(logits[0, -1]).max(), f"token {i}"
        logits, pos, _, _ = corc.forward_with_state(shape, w, np.array([[got]]), rho, pos, sparse_state=False)
    text = tok.decode(tokens)
    assert text.startswith("First Citizen:\n") and len(text) == len(prompt) + n_new
    print(repr(text))


def test_sampled_generation_streams_and_is_reproducible(trained):
    from burn_dragon_amd.generation import (ContextStrategy, GenerationConfig, GenerationSettings, generate_text,
                                            generate_tokens)

    model, tok, block_size, _, _ = trained
    cfg = GenerationConfig(prompt="ROMEO:", max_tokens=64, temperature=0.8, top_k=20,
                           context_strategy=ContextStrategy.sliding(0))
    a = generate_text(model, tok, block_size, cfg, torch.Generator(device=DEV).manual_seed(11))
    b = generate_text(model, tok, block_size, cfg, torch.Generator(device=DEV).manual_seed(11))
    c = generate_text(model, tok, block_size, cfg, torch.Generator(device=DEV).manual_seed(12))
    assert a == b and a != c and a.startswith("ROMEO:") and len(a) <= 6 + 64
    seen = []
    streamed = generate_tokens(model, tok.encode("ROMEO:"), GenerationSettings(64, 0.8, 20), seen.append,
                               torch.Generator(device=DEV).manual_seed(11))
    assert tok.decode(streamed) == a and seen == streamed[6:]

    def stop_after_five(t):  # an unbounded run ends when the callback says so
        seen.append(t)
        if len(seen) >= 5:
            raise StopIteration

    seen.clear()
    out = generate_tokens(model, tok.encode("A"), GenerationSettings(None, 1.0, None), stop_after_five)
    assert len(out) == 1 + 5
    with pytest.raises(ValueError):
        generate_tokens(model, [], GenerationSettings(1, 1.0, None))
    print(repr(a))


def test_sampled_token_frequencies_follow_the_softmax(trained):
    from burn_dragon_amd.generation import sample_from_logits

    model = trained[0]
    logits = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5]], device=DEV).repeat(20000, 1)
    u = torch.rand(20000, device=DEV, generator=torch.Generator(device=DEV).manual_seed(0))
    counts = torch.bincount(sample_from_logits(model, logits, 1.0, None, u), minlength=5).cpu().numpy()
    p = torch.softmax(logits[0].double(), 0).cpu().numpy()
    from scipy.stats import chisquare

    assert chisquare(counts, p * 20000).pvalue > 1e-3


def test_trained_checkpoint_with_lazily_decayed_state(trained, corc):
    """The ALiBi checkpoint with the state kept lazily decayed: same logits as the oracle's eager decay
    for a prompt and the following greedy steps (eager launches and a replayed HIP graph), and the
    materialised state equals the oracle's."""
    import burn_dragon_amd as bda

    _, tok, _, shape, w = trained
    model, _, _ = bda.BDH.from_checkpoint_dir(CKPT, DEV, alibi_lazy=True)
    ids = np.array([tok.encode(TEXT[:90])])
    state = model.init_state()
    logits, nxt = model.forward_with_state(torch.from_numpy(ids), state, want_next=True)
    assert state.stamps is not None and tuple(state.stamps.shape) == (4, 1, 4, 128)
    rho_ref = np.zeros((4, 1, 4, 128, 128), np.float32)
    logits_ref, pos, _, _ = corc.forward_with_state(shape, w, ids, rho_ref, 0, sparse_state=False)
    assert rel_err(logits.cpu().numpy(), logits_ref) < 1e-3
    graph = None
    for step in range(12):
        tok_ref = corc.greedy_token(logits_ref[0, -1])
        if step == 6:
            graph = model.capture_decode_step(state, torch.tensor([tok_ref]))
        if graph is None:
            logits, nxt = model.forward_with_state(torch.tensor([[tok_ref]]), state, want_next=True)
        else:
            graph.tokens.fill_(tok_ref)
            graph.replay()
            logits = graph.logits
        logits_ref, pos, _, _ = corc.forward_with_state(shape, w, np.array([[tok_ref]]), rho_ref, pos, sparse_state=False)
        assert rel_err(logits.cpu().numpy(), logits_ref) < 1e-3, step
    assert state.position == pos
    lazy_rows = float((state.stamps < state.position).float().mean())
    assert lazy_rows > 0.3  # most rows were NOT touched by the last token: that is the saving
    model.materialize_state(state)
    torch.cuda.synchronize()
    assert (state.stamps == state.position).all()
    assert rel_err(state.storage.cpu().numpy(), rho_ref) < 1e-3


def test_model_generate_has_the_reference_signature(trained):
    """BDH::generate (src/model/bdh.rs:170-252): indices [1,T] -> [1,T+n]; top_k = 1 equals the greedy
    generate_tokens run, a sampled run is reproducible from its generator and equals generate_tokens with
    the same variates."""
    from burn_dragon_amd.generation import GenerationSettings, generate_tokens

    model, tok, _, _, _ = trained
    prompt = tok.encode("JULIET:\n")
    idx = torch.tensor([prompt])
    greedy = model.generate(idx, 24, 1.0, 1)
    assert tuple(greedy.shape) == (1, len(prompt) + 24)
    assert greedy[0].tolist() == generate_tokens(model, prompt, GenerationSettings(24, 1.0, 1))
    a = model.generate(idx, 24, 0.9, 12, torch.Generator(device=DEV).manual_seed(3))[0].tolist()
    b = model.generate(idx, 24, 0.9, 12, torch.Generator(device=DEV).manual_seed(3))[0].tolist()
    c = generate_tokens(model, prompt, GenerationSettings(24, 0.9, 12), None, torch.Generator(device=DEV).manual_seed(3))
    assert a == b == c and a != greedy[0].tolist()
    with pytest.raises(AssertionError):
        model.generate(torch.tensor([prompt, prompt]), 1)  # batch size 1 only, as in the reference
