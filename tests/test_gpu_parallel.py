"""GPU parity of the all-tokens-at-once forms: the f32 block-tiled normalised attention
(bdh_fused_state_aligned, the reference's training-path kernel) and the bf16 matrix-core
chunked prefill (bdh_prefill_chunked), through the C ABI, against the CPU oracle."""
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


def assert_close(lhs, rhs, atol, rtol):
    """tests/fused_kernel_tests.rs:13-33."""
    lhs, rhs = np.asarray(lhs, np.float64), np.asarray(rhs, np.float64)
    assert lhs.shape == rhs.shape
    assert not (np.abs(lhs - rhs) > atol + rtol * np.abs(rhs)).any(), f"max diff {np.abs(lhs - rhs).max()}"


def rel_err(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


# ------------------------------------------------------------ fused_state_aligned
@pytest.fixture(params=[0, 1], ids=["row-kernel", "matrix-cores"])
def fsa_path(request, bda):
    """Runs a test once per implementation of fused_state_aligned (the default picks by T)."""
    from burn_dragon_amd import ffi

    ctx = ffi.default_context(0)
    ctx.set_option("fused_state_aligned.path", request.param)
    yield request.param
    ctx.set_option("fused_state_aligned.path", -1)


@pytest.mark.parametrize("rotary,seed", [("rope", 1337), ("pope", 2024)])
def test_fused_attention_matches_reference(bda, corc, fsa_path, rotary, seed):
    """tests/fused_kernel_tests.rs:70-170 on the device path: B=1, h=2, T=6, N=8, dv=6,
    BlockPattern2d::dense(3); fused == dense tril(-1) + row-normalise, tolerance 1e-4."""
    from burn_dragon_amd.kernel import linear_attention

    rot = bda.RotaryEmbedding.parse(rotary)
    g = torch.Generator().manual_seed(seed)
    query = torch.randn((1, 2, 6, 8), generator=g)
    value = torch.randn((1, 1, 6, 6), generator=g)
    freqs = linear_attention.build_freqs(8, 65536.0, rot)
    fused = linear_attention.fused_state_aligned(query.to(DEV), value.to(DEV), freqs.to(DEV), None,
                                                 bda.BlockPattern2d.dense(3), rot)
    torch.cuda.synchronize()
    # dense reference in float64, as the reference test writes it
    q = orc.rotate(query.double().numpy(), freqs.double().numpy().reshape(-1), int(rot), 0)
    scores = np.tril(q @ np.swapaxes(q, 2, 3), -1)
    scores = scores / (np.abs(scores).sum(3, keepdims=True) + 1e-6)
    reference = scores @ value.double().numpy()
    assert_close(fused.cpu().numpy(), reference, 1e-4, 1e-4)
    # and the oracle's blocked form
    ref_c = corc.fused_state_aligned(query.numpy(), value.numpy()[:, 0], freqs.numpy().reshape(-1), None, 3, int(rot))
    assert_close(fused.cpu().numpy(), ref_c, 1e-4, 1e-4)


def test_fused_attention_alibi_sparse_pattern_and_unnormalised(bda, corc, fsa_path):
    from burn_dragon_amd.kernel import linear_attention

    rng = np.random.default_rng(3)
    B, h, T, N, dv = 2, 2, 11, 16, 5
    query = np.abs(rng.standard_normal((B, h, T, N))).astype(np.float32)
    value = rng.standard_normal((B, T, dv)).astype(np.float32)
    slopes = np.array([0.5, 0.25], np.float32)
    zeros = np.zeros(N, np.float32)
    qt, vt = torch.from_numpy(query).to(DEV), torch.from_numpy(value[:, None]).to(DEV)
    # ALiBi, dense pattern, ragged last block (the term is added to whole blocks: linear_attention.rs:97-100)
    got = linear_attention.fused_state_aligned(qt, vt, torch.from_numpy(zeros), torch.from_numpy(slopes),
                                               bda.BlockPattern2d.dense(4), bda.RotaryEmbedding.ALIBI)
    assert_close(got.cpu().numpy(), corc.fused_state_aligned(query, value, zeros, slopes, 4, orc.ALIBI), 1e-4, 1e-4)
    # sparse (row, col) block pairs; row block 1 has no active column -> zeros (linear_attention.rs:70-73)
    pairs = {(0, 0), (2, 0), (2, 2)}
    freqs = corc.build_freqs(N)
    got = linear_attention.fused_state_aligned(qt, vt, torch.from_numpy(freqs), None,
                                               bda.BlockPattern2d.from_pairs(4, pairs), bda.RotaryEmbedding.ROPE)
    ref = corc.fused_state_aligned(query, value, freqs, None, 4, orc.ROPE, pairs=pairs)
    assert_close(got.cpu().numpy(), ref, 1e-4, 1e-4)
    assert not got[:, :, 4:8].any()
    # row_normalize = 0 equals the recurrent path started from a zero state at position 0
    got = linear_attention.fused_state_aligned(qt, vt, torch.from_numpy(freqs), None, bda.BlockPattern2d.dense(4),
                                               bda.RotaryEmbedding.ROPE, row_normalize=False)
    out_rec, _ = corc.recurrent_attention(corc.rotate(query, freqs, orc.ROPE, 0), value, np.zeros((B, h, N, dv), np.float32))
    assert_close(got.cpu().numpy(), out_rec, 1e-4, 1e-4)


@pytest.mark.parametrize("rotary", ["rope", "alibi", "pope"])
def test_fused_attention_medium_shapes_on_the_matrix_cores(bda, corc, rotary):
    """T = 300 (default path: f32 matrix cores), ragged against the 128-wide tiles and the time block of
    48, N and dv not multiples of 4: against the oracle's blocked form, normalised and not, dense and
    with a sparse block pattern."""
    from burn_dragon_amd.kernel import linear_attention

    rng = np.random.default_rng(5)
    B, h, T, N, dv, bs = 2, 3, 300, 202, 70, 48
    query = np.maximum(rng.standard_normal((B, h, T, N)) - 0.5, 0).astype(np.float32)
    value = rng.standard_normal((B, T, dv)).astype(np.float32)
    rot = {"rope": orc.ROPE, "alibi": orc.ALIBI, "pope": orc.POPE}[rotary]
    slopes = corc.default_alibi_slopes(h) if rotary == "alibi" else None
    freqs = corc.build_freqs(N, rotary=rot)
    qt, vt = torch.from_numpy(query).to(DEV), torch.from_numpy(value[:, None]).to(DEV)
    st = None if slopes is None else torch.from_numpy(slopes)
    tb = (T + bs - 1) // bs
    pairs = {(r, c) for r in range(tb) for c in range(r + 1) if (r + 2 * c) % 3 != 1}
    for layout, kw in [(bda.BlockPattern2d.dense(bs), {}), (bda.BlockPattern2d.from_pairs(bs, pairs), {"pairs": pairs})]:
        got = linear_attention.fused_state_aligned(qt, vt, torch.from_numpy(freqs), st, layout,
                                                   bda.RotaryEmbedding.parse(rotary))
        ref = corc.fused_state_aligned(query, value, freqs, slopes, bs, rot, **kw)
        assert rel_err(got.cpu().numpy(), ref) < 1e-3
    got = linear_attention.fused_state_aligned(qt, vt, torch.from_numpy(freqs), st, bda.BlockPattern2d.dense(bs),
                                               bda.RotaryEmbedding.parse(rotary), row_normalize=False)
    if rotary != "alibi":  # the un-normalised dense form is the recurrent path from a zero state
        Nq = 2 * N if rotary == "pope" else N
        out_rec, _ = corc.recurrent_attention(corc.rotate(query, freqs, rot, 0), value,
                                              np.zeros((B, h, Nq, dv), np.float32))
        assert rel_err(got.cpu().numpy(), out_rec) < 1e-3


def test_fused_attention_long_sequences_take_the_large_tiles(bda, corc):
    """T = 1100 with 16 slices: the 256 x 256 tiles of the matrix-core path, ragged against them and
    against the time block of 100; ALiBi (the term lands on whole blocks) and RoPE."""
    from burn_dragon_amd.kernel import linear_attention

    rng = np.random.default_rng(9)
    B, h, T, N, dv, bs = 4, 4, 1100, 66, 40, 100
    query = np.maximum(rng.standard_normal((B, h, T, N)) - 0.5, 0).astype(np.float32)
    value = rng.standard_normal((B, T, dv)).astype(np.float32)
    qt, vt = torch.from_numpy(query).to(DEV), torch.from_numpy(value[:, None]).to(DEV)
    for rotary, rot in (("rope", orc.ROPE), ("alibi", orc.ALIBI)):
        slopes = corc.default_alibi_slopes(h) if rotary == "alibi" else None
        freqs = corc.build_freqs(N, rotary=rot)
        got = linear_attention.fused_state_aligned(qt, vt, torch.from_numpy(freqs),
                                                   None if slopes is None else torch.from_numpy(slopes),
                                                   bda.BlockPattern2d.dense(bs), bda.RotaryEmbedding.parse(rotary))
        ref = corc.fused_state_aligned(query, value, freqs, slopes, bs, rot)
        assert rel_err(got.cpu().numpy(), ref) < 1e-3


# ---------------------------------------------------------------- chunked prefill
def _prefill_case(seed, B, h, T, N, d, density, rho0_scale):
    from scipy.stats import norm

    g = torch.Generator().manual_seed(seed)
    x = torch.relu(torch.randn((B, h, T, N), generator=g) + float(norm.ppf(density))).to(torch.bfloat16)
    v = torch.randn((B, T, d), generator=g).to(torch.bfloat16)
    rho0 = (rho0_scale * torch.randn((B, h, N, d), generator=g)).float()
    return x, v, rho0


@pytest.mark.parametrize("T,N,d,rho0_scale,position", [(64, 256, 256, 0.0, 0), (200, 512, 256, 0.05, 77),
                                                       (300, 264, 72, 0.05, 5), (520, 128, 512, 0.0, 1000),
                                                       (512, 192, 256, 0.05, 33), (256, 64, 512, 0.0, 9)])
def test_prefill_chunked_equals_sequential_recurrence(bda, corc, T, N, d, rho0_scale, position):
    """Oracle = the sequential f32 loop of src/model/bdh.rs:288-302 on the bf16-rounded inputs.
    Tolerance 2e-2 relative on the max-norm (north_star, bf16 path); Q is rounded to bf16 once
    and the scores are kept in bf16."""
    from burn_dragon_amd.recurrent import prefill_chunked

    B, h = 2, 2
    x, v, rho0 = _prefill_case(T + N, B, h, T, N, d, 0.2, rho0_scale)
    freqs = corc.build_freqs(N)
    q = corc.rotate(x.float().numpy(), freqs, orc.ROPE, position)
    out_ref, rho_ref = corc.recurrent_attention(q, v.float().numpy(), rho0.numpy(), sparse=True)
    rho = rho0.clone().to(DEV)
    out = prefill_chunked(x.to(DEV), v.to(DEV), rho, torch.from_numpy(freqs).to(DEV), position,
                          state_is_zero=(rho0_scale == 0.0))
    torch.cuda.synchronize()
    assert rel_err(out.cpu().numpy(), out_ref) < 2e-2
    assert rel_err(rho.cpu().numpy(), rho_ref) < 2e-2
    assert not out[:, :, 0].any() or rho0_scale != 0.0  # token 0 reads only the initial state


@pytest.mark.parametrize("T,N,chunk,rho0_scale,position,hilo", [
    (256, 256, 0, 0.0, 0, False), (512, 512, 0, 0.05, 77, False), (1024, 256, 512, 0.0, 3000, False),
    (768, 512, 256, 0.05, 5, True), (600, 256, 512, 0.05, 9, False), (1280, 256, 0, 0.05, 1, True)])
def test_prefill_chunk_recurrent_form(bda, corc, T, N, chunk, rho0_scale, position, hilo):
    """Shapes that take the chunk-recurrent kernels (d = 256, N a multiple of 256, passes of 256+ tokens; a ragged tail
    of the last pass falls to the all-scores form): several 256-token chunks per pass, several passes per call, a
    carried-in state with and without the bf16 pair, against the sequential oracle (2e-2) and against the all-scores
    form of the same call."""
    from burn_dragon_amd.recurrent import prefill_chunked

    B, h, d = 2, 2, 256
    x, v, rho0 = _prefill_case(T + N + chunk, B, h, T, N, d, 0.2, rho0_scale)
    freqs = corc.build_freqs(N)
    q = corc.rotate(x.float().numpy(), freqs, orc.ROPE, position)
    out_ref, rho_ref = corc.recurrent_attention(q, v.float().numpy(), rho0.numpy(), sparse=True)
    ft = torch.from_numpy(freqs).to(DEV)
    rho = rho0.clone().to(DEV)
    print(f"chunk-recurrent prefill T={T} N={N} chunk={chunk} hilo={hilo}", flush=True)
    out = prefill_chunked(x.to(DEV), v.to(DEV), rho, ft, position, state_is_zero=(rho0_scale == 0.0), chunk=chunk,
                          hilo=hilo)
    torch.cuda.synchronize()
    e_out, e_rho = rel_err(out.cpu().numpy(), out_ref), rel_err(rho.cpu().numpy(), rho_ref)
    print(f"   out rel err {e_out:.2e}, state rel err {e_rho:.2e}")
    assert e_out < 2e-2 and e_rho < 2e-2
    rho_s = rho0.clone().to(DEV)
    out_s = prefill_chunked(x.to(DEV), v.to(DEV), rho_s, ft, position, state_is_zero=(rho0_scale == 0.0), chunk=chunk,
                            all_scores=True)
    d_out, d_rho = rel_err(out.cpu().numpy(), out_s.cpu().numpy()), rel_err(rho.cpu().numpy(), rho_s.cpu().numpy())
    # both accumulate Q^T V in f32; their Q differ by a bf16 rounding step here and there (inside a chunk the
    # chunk-recurrent kernel steps the rotation by angle addition from the chunk's exact phase)
    assert d_out < 2e-2 and d_rho < 5e-3, (d_out, d_rho)


@pytest.mark.parametrize("T,N,rho0_scale,position,hilo", [(768, 256, 0.0, 0, False), (1024, 512, 0.05, 41, True)])
def test_prefill_chunk_recurrent_form_with_unequal_pair_frequencies(bda, corc, T, N, rho0_scale, position, hilo):
    """A frequency table whose two elements of a lane pair differ (not what build_freqs makes, but what the ABI
    accepts): the state-update kernel then runs its second instantiation, with separate phases for the even and the
    odd element (src/model/attention.rs:305-321 takes cos/sin per element).  Against the sequential oracle and the
    all-scores form."""
    from burn_dragon_amd.recurrent import prefill_chunked

    B, h, d = 1, 2, 256
    x, v, rho0 = _prefill_case(5 * T + N, B, h, T, N, d, 0.2, rho0_scale)
    freqs = corc.build_freqs(N).copy()
    freqs[1::2] *= np.float32(1.25)
    q = corc.rotate(x.float().numpy(), freqs, orc.ROPE, position)
    out_ref, rho_ref = corc.recurrent_attention(q, v.float().numpy(), rho0.numpy(), sparse=True)
    ft = torch.from_numpy(freqs).to(DEV)
    rho = rho0.clone().to(DEV)
    print(f"chunk-recurrent prefill, unequal pair frequencies T={T} N={N} hilo={hilo}", flush=True)
    out = prefill_chunked(x.to(DEV), v.to(DEV), rho, ft, position, state_is_zero=(rho0_scale == 0.0), hilo=hilo)
    torch.cuda.synchronize()
    e_out, e_rho = rel_err(out.cpu().numpy(), out_ref), rel_err(rho.cpu().numpy(), rho_ref)
    print(f"   out rel err {e_out:.2e}, state rel err {e_rho:.2e}")
    assert e_out < 2e-2 and e_rho < 2e-2
    rho_s = rho0.clone().to(DEV)
    out_s = prefill_chunked(x.to(DEV), v.to(DEV), rho_s, ft, position, state_is_zero=(rho0_scale == 0.0), all_scores=True)
    d_out, d_rho = rel_err(out.cpu().numpy(), out_s.cpu().numpy()), rel_err(rho.cpu().numpy(), rho_s.cpu().numpy())
    assert d_out < 2e-2 and d_rho < 5e-3, (d_out, d_rho)


@pytest.mark.parametrize("B,h,T,N,chunk,rho0_scale,hilo", [
    (3, 3, 512, 768, 0, 0.0, False),      # 9 slices: a second, partly filled group of eight
    (1, 1, 1280, 2048, 512, 0.05, True),  # one slice, 32 neuron tiles, passes of 512 + 256 tokens
    (2, 5, 256, 256, 0, 0.05, False),     # 10 slices, a single chunk with a carried state
    (9, 1, 768, 512, 256, 0.0, False),    # three one-chunk passes, fresh state
    (1, 2, 2304, 1024, 0, 0.05, False)])  # a pass of 2 048 tokens and one of 256
def test_prefill_chunk_recurrent_form_equals_all_scores_form(bda, B, h, T, N, chunk, rho0_scale, hilo):
    """More slice counts, tile counts and pass structures of the chunk-recurrent kernels, against the all-scores form
    of the same call (itself checked against the sequential oracle above): slices that do not fill the groups of
    eight the grids are laid out in, one to 32 neuron tiles per slice, one to eight chunks per pass."""
    from burn_dragon_amd.recurrent import prefill_chunked

    d = 256
    x, v, rho0 = _prefill_case(B * 1000 + T + N, B, h, T, N, d, 0.1, rho0_scale)
    sys_freqs = orc.build_freqs(N)
    ft = torch.from_numpy(np.asarray(sys_freqs, dtype=np.float32)).to(DEV)
    zero = rho0_scale == 0.0
    print(f"chunk-recurrent against all-scores: B={B} h={h} T={T} N={N} chunk={chunk} hilo={hilo}", flush=True)
    rho_c, rho_s = rho0.clone().to(DEV), rho0.clone().to(DEV)
    out_c = prefill_chunked(x.to(DEV), v.to(DEV), rho_c, ft, 17, state_is_zero=zero, chunk=chunk, hilo=hilo)
    out_s = prefill_chunked(x.to(DEV), v.to(DEV), rho_s, ft, 17, state_is_zero=zero, chunk=chunk, all_scores=True)
    torch.cuda.synchronize()
    d_out, d_rho = rel_err(out_c.cpu().numpy(), out_s.cpu().numpy()), rel_err(rho_c.cpu().numpy(), rho_s.cpu().numpy())
    print(f"   out {d_out:.2e} state {d_rho:.2e}")
    assert d_out < 2e-2 and d_rho < 5e-3, (d_out, d_rho)


def test_prefill_in_four_calls_equals_one_call(bda, corc):
    """One prompt fed as four successive calls (the state carried in the caller's f32 rho, entering each call's
    product as a bf16 pair) against the sequential oracle and against the single call: T = 4096 in chunks of 512."""
    from burn_dragon_amd.recurrent import prefill_chunked

    B, h, T, N, d = 1, 2, 4096, 512, 256
    x, v, _ = _prefill_case(21, B, h, T, N, d, 0.1, 0.0)
    freqs = corc.build_freqs(N)
    q = corc.rotate(x.float().numpy(), freqs, orc.ROPE, 0)
    out_ref, rho_ref = corc.recurrent_attention(q, v.float().numpy(), np.zeros((B, h, N, d), np.float32), sparse=True)
    ft = torch.from_numpy(freqs).to(DEV)
    xd, vd = x.to(DEV), v.to(DEV)
    rho1 = torch.zeros((B, h, N, d), device=DEV)
    out1 = prefill_chunked(xd, vd, rho1, ft, 0, state_is_zero=True, chunk=512)
    rho4 = torch.zeros((B, h, N, d), device=DEV)
    outs = []
    for k in range(4):
        sl = slice(k * 1024, (k + 1) * 1024)
        outs.append(prefill_chunked(xd[:, :, sl].contiguous(), vd[:, sl].contiguous(), rho4, ft, k * 1024,
                                    state_is_zero=(k == 0), chunk=512, hilo=True))
    out4 = torch.cat(outs, dim=2)
    torch.cuda.synchronize()
    errs = (rel_err(out1.cpu().numpy(), out_ref), rel_err(rho1.cpu().numpy(), rho_ref),
            rel_err(out4.cpu().numpy(), out_ref), rel_err(rho4.cpu().numpy(), rho_ref),
            rel_err(out4.cpu().numpy(), out1.cpu().numpy()))
    print("one call / four calls against the oracle (out, rho, out, rho), four against one (out):", errs)
    assert max(errs) < 2e-2, errs
    d_rho = rel_err(rho4.cpu().numpy(), rho1.cpu().numpy())
    assert d_rho < 1e-5, d_rho  # the f32 state never passes through bf16


def test_prefill_chunked_then_decode_steps_continue_the_state(bda, corc):
    """Prefill T tokens on the matrix cores, then decode 3 tokens with bdh_state_step: the
    readouts must match the all-sequential oracle (2e-2: the prefilled state carries bf16 error)."""
    from burn_dragon_amd.recurrent import prefill_chunked, recurrent_attention

    B, h, T, N, d = 1, 2, 96, 256, 256
    x, v, _ = _prefill_case(9, B, h, T + 3, N, d, 0.1, 0.0)
    freqs = corc.build_freqs(N)
    q = corc.rotate(x.float().numpy(), freqs, orc.ROPE, 0)
    out_ref, rho_ref = corc.recurrent_attention(q, v.float().numpy(), np.zeros((B, h, N, d), np.float32), sparse=True)
    rho = torch.zeros((B, h, N, d), device=DEV)
    ft = torch.from_numpy(freqs).to(DEV)
    out_p = prefill_chunked(x[:, :, :T].contiguous().to(DEV), v[:, :T].contiguous().to(DEV), rho, ft, 0, state_is_zero=True)
    out_d = recurrent_attention(x[:, :, T:].float().contiguous().to(DEV), v[:, T:].float().contiguous().to(DEV), rho, ft,
                                T, bda.RotaryEmbedding.ROPE)
    torch.cuda.synchronize()
    assert rel_err(out_p.cpu().numpy(), out_ref[:, :, :T]) < 2e-2
    assert rel_err(out_d.cpu().numpy(), out_ref[:, :, T:]) < 2e-2
    assert rel_err(rho.cpu().numpy(), rho_ref) < 2e-2


@pytest.mark.parametrize("unequal_pairs", [False, True])
def test_prefill_chunked_config3_shape_properties(bda, corc, unequal_pairs):
    """BASELINE config 3 per-slice shape (T=2048, N=8192, d=256, 5 % density) on a reduced batch
    (B=1, h=2) so the oracle finishes in seconds.  Checks against the sequential oracle and the
    size-independent closed forms (first row zero, final state == Q^T V).  At this width two workgroups share a
    compute unit, which the small shapes above never reach; the second case takes the kernel instantiation for
    frequency tables whose pair elements differ."""
    from burn_dragon_amd.recurrent import prefill_chunked

    B, h, T, N, d = 1, 2, 2048, 8192, 256
    x, v, _ = _prefill_case(11, B, h, T, N, d, 0.05, 0.0)
    freqs = corc.build_freqs(N).copy()
    if unequal_pairs:
        freqs[1::2] *= np.float32(1.25)
    rho = torch.zeros((B, h, N, d), device=DEV)
    out = prefill_chunked(x.to(DEV), v.to(DEV), rho, torch.from_numpy(freqs).to(DEV), 0, state_is_zero=True)
    torch.cuda.synchronize()
    q = corc.rotate(x.float().numpy(), freqs, orc.ROPE, 0)
    out_ref, rho_ref = corc.recurrent_attention(q, v.float().numpy(), np.zeros((B, h, N, d), np.float32), sparse=True)
    assert rel_err(out.cpu().numpy(), out_ref) < 2e-2
    assert rel_err(rho.cpu().numpy(), rho_ref) < 2e-2
    assert not out[:, :, 0].any()
    qtv = torch.einsum("bhtn,btd->bhnd", torch.from_numpy(q).to(DEV), v.float().to(DEV))
    assert rel_err(rho.cpu().numpy(), qtv.cpu().numpy()) < 2e-2


def test_prefill_chunked_config3_at_its_own_batch(bda, corc):
    """BASELINE config 3 at its full size (B=8, h=4, T=2048, N=8192, d=256, 5 % density, fresh state): the 32-slice
    launch that bench.py times, checked without the oracle's token loop (too slow at this size):
      - the first token of every slice reads a zero state: out[:, :, 0] == 0;
      - the final state is Q^T V (src/model/bdh.rs:298 summed over the tokens), with Q = bf16(rope(x)) from the
        oracle's rotate and the product by a device einsum, one batch entry at a time;
      - slices are independent: (b=0, h=0..1) of this call hold the same bits as a B=1, h=2 call on those inputs
        (the call test_prefill_chunked_config3_shape_properties checks against the oracle);
      - out against the closed causal form tril(-1)(Q Q^T) V on the device for one slice."""
    from burn_dragon_amd.recurrent import prefill_chunked

    B, h, T, N, d = 8, 4, 2048, 8192, 256
    x, v, _ = _prefill_case(11, B, h, T, N, d, 0.05, 0.0)
    freqs = corc.build_freqs(N)
    ft = torch.from_numpy(freqs).to(DEV)
    xt, vt = x.to(DEV), v.to(DEV)
    rho = torch.zeros((B, h, N, d), device=DEV)
    print("prefill config 3 at B=8, h=4", flush=True)
    out = prefill_chunked(xt, vt, rho, ft, 0, state_is_zero=True)
    torch.cuda.synchronize()
    assert not out[:, :, 0].any()
    for b in range(B):  # Q of one batch entry: [h, T, N] f32 = 256 MiB
        q = torch.from_numpy(corc.rotate(x[b:b + 1].float().numpy(), freqs, orc.ROPE, 0)).to(DEV)
        q = q.to(torch.bfloat16).float()  # the products take the rotated activations rounded to bf16
        qtv = torch.einsum("htn,td->hnd", q[0], vt[b].float())
        err = float((rho[b] - qtv).abs().max()) / float(qtv.abs().max())
        assert err < 2e-2, f"batch entry {b}: {err}"
        if b == 0:  # the causal closed form for one slice
            s = torch.tril(q[0, 0] @ q[0, 0].T, -1)
            o = s @ vt[0].float()
            err_o = float((out[0, 0] - o).abs().max()) / float(o.abs().max())
            assert err_o < 2e-2, err_o
    rho2 = torch.zeros((1, 2, N, d), device=DEV)
    out2 = prefill_chunked(xt[:1, :2].contiguous(), vt[:1].contiguous(), rho2, ft, 0, state_is_zero=True)
    torch.cuda.synchronize()
    assert torch.equal(out2[0], out[0, :2]) and torch.equal(rho2[0], rho[0, :2])


def test_prefill_chunked_argument_errors(bda):
    from burn_dragon_amd import ffi

    ctx = ffi.default_context(0)
    t = torch.zeros(4096, device=DEV)
    p = t.data_ptr()
    assert ctx.lib.bdh_prefill_chunked(ctx.handle, 1, 1, 8, 12, 8, p, p, p, 0, 0, 1, p, p) == ffi.E_SHAPE  # N % 8
    assert ctx.lib.bdh_prefill_chunked(ctx.handle, 1, 1, 8, 16, 8, None, p, p, 0, 0, 1, p, p) == ffi.E_INVAL
    assert ctx.lib.bdh_prefill_chunked(ctx.handle, 1, 1, 8, 16, 8, p, p, p, 0, -1, 1, p, p) == ffi.E_INVAL  # chunk < 0
    assert ctx.lib.bdh_prefill_chunked(ctx.handle, 1, 1, 8, 16, 8, p, p, p, 0, 0, 64, p, p) == ffi.E_INVAL  # flag bits
    assert ctx.lib.bdh_prefill_chunked(ctx.handle, 0, 1, 8, 16, 8, None, None, None, 0, 0, 1, None, None) == ffi.OK


def test_prefill_state_copies_tight_against_a_device_restatement(bda, corc):
    """A tight check of the chunk-recurrent kernels' bf16 state copies (the stores of k_state_stream that need idle
    cycles before their data registers are rewritten): the second and third 256-token chunks of a call read
    bf16(rho_c) that the first kernel wrote.  The same quantities from plain f32 torch products on the device, with the
    same roundings (Q = bf16 of the oracle's rotation, scores and state copies rounded to bf16 once, f32 accumulation),
    must agree to 2e-3 of the output scale -- ten times tighter than the bf16 tolerance class, so a few corrupted
    elements of a copy show."""
    from burn_dragon_amd.recurrent import prefill_chunked

    B, h, T, N, d = 1, 2, 768, 512, 256
    x, v, _ = _prefill_case(77, B, h, T, N, d, 0.2, 0.0)
    freqs = corc.build_freqs(N)
    rho = torch.zeros((B, h, N, d), device=DEV)
    out = prefill_chunked(x.to(DEV), v.to(DEV), rho, torch.from_numpy(freqs).to(DEV), 0, state_is_zero=True)
    torch.cuda.synchronize()
    q = torch.from_numpy(corc.rotate(x.float().numpy(), freqs, orc.ROPE, 0)).to(DEV).to(torch.bfloat16).float()
    vf = v.float().to(DEV)
    state = torch.zeros((B, h, N, d), device=DEV)
    ref = torch.empty((B, h, T, d), device=DEV)
    for c in range(T // 256):
        sl = slice(c * 256, (c + 1) * 256)
        qc, vc = q[:, :, sl], vf[:, None, sl]
        scores = torch.tril(qc @ qc.transpose(2, 3), -1).to(torch.bfloat16).float()
        ref[:, :, sl] = scores @ vc + qc @ state.to(torch.bfloat16).float()
        state = state + qc.transpose(2, 3) @ vc
    scale = ref.abs().max().item()
    assert (out - ref).abs().max().item() < 2e-3 * scale
    assert (rho - state).abs().max().item() < 2e-3 * state.abs().max().item()
