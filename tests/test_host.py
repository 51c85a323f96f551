"""CPU-side checks of the host layer: the C-ABI library loads and exports every declared
symbol, the host mirror follows the reference's config rules, and the entry points that
need no device behave (no compute call is made here)."""
import ctypes
import os
import re

import numpy as np
import pytest

import burn_dragon_amd as bda
from burn_dragon_amd import ffi
from burn_dragon_amd.kernel.block_sparse import BlockPattern1d, BlockPattern2d
from burn_dragon_amd.kernel.linear_attention import build_freqs, default_alibi_slopes
from oracle import bdh_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(ffi.LIB_PATH):
        pytest.fail("libbdh_mi355x.so is not built (python -m burn_dragon_amd.build)")
    return ffi.load_library()


def test_library_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "bdh_mi355x.h")).read()
    declared = sorted(set(re.findall(r"\b(bdh_[a-z_0-9]+)\s*\(", header)))
    assert declared, "no declarations found"
    missing = [name for name in declared if not hasattr(lib, name)]
    assert not missing, f"declared but not exported: {missing}"
    assert sorted(ffi.EXPORTS) == declared
    assert b"gfx950" in lib.bdh_version()


def test_status_strings(lib):
    assert lib.bdh_status_string(0) == b"ok"
    for code in range(-6, 0):
        assert lib.bdh_status_string(code) not in (b"ok", b"unknown status")
    assert lib.bdh_status_string(-99) == b"unknown status"


def test_null_context_is_rejected_without_touching_a_device(lib):
    assert lib.bdh_layer_norm(None, 1, 4, None, None) == ffi.E_INVAL
    assert lib.bdh_state_step(None, 1, 1, 2, 4, 0, None, None, None, 0, None, None, None, 0, None, None, None) == ffi.E_INVAL
    assert lib.bdh_ctx_create(0, None, None) == ffi.E_INVAL
    assert lib.bdh_ctx_destroy(None) == ffi.OK
    assert lib.bdh_last_error(None) == b"null context"


def test_freqs_and_slopes_match_oracle_bit_for_bit(lib, corc):
    # both sides evaluate the same f32 expression with the host libm (src/model/attention.rs:351-373)
    for rotary in (orc.ROPE, orc.POPE, orc.ALIBI):
        for latent in (8, 32, 8192, 16384):
            got = build_freqs(latent, 65536.0, bda.RotaryEmbedding(rotary)).numpy().reshape(-1)
            assert np.array_equal(got, corc.build_freqs(latent, 65536.0, rotary))
    assert np.array_equal(np.array(default_alibi_slopes(8), np.float32), corc.default_alibi_slopes(8))
    assert default_alibi_slopes(0) == []
    out = np.zeros(4, np.float32)
    assert lib.bdh_build_freqs(4, 65536.0, 7, out.ctypes.data) == ffi.E_INVAL
    assert lib.bdh_build_freqs(4, 65536.0, 0, None) == ffi.E_INVAL


def test_config_defaults_and_latent_rule():
    """src/model/config.rs:20-31, :125-163."""
    cfg = bda.BDHConfig()
    assert (cfg.n_layer, cfg.n_embd, cfg.n_head, cfg.mlp_internal_dim_multiplier, cfg.vocab_size) == (6, 256, 4, 4, 256)
    assert cfg.latent_per_head() == 256 and cfg.latent_total() == 1024
    assert cfg.fused_kernels.rope_theta == 65536.0 and cfg.fused_kernels.relu_threshold == 0.0
    assert cfg.fused_kernels.rotary_embedding == bda.RotaryEmbedding.ALIBI and not cfg.fused_kernels.enabled
    cfg.mlp_internal_dim_multiplier = 128
    assert cfg.latent_per_head() == 8192
    bad = bda.BDHConfig(n_embd=10, n_head=3, mlp_internal_dim_multiplier=1)
    with pytest.raises(AssertionError):
        bad.latent_per_head()


def test_build_model_config_overrides():
    """src/inference.rs:4-40."""
    ov = bda.ModelOverrides(n_layer=2, n_embd=16, n_head=2, relu_threshold=0.5, fused_kernels=True,
                            rotary_embedding=bda.RotaryEmbedding.ROPE)
    cfg = bda.build_model_config(ov, 32)
    assert (cfg.n_layer, cfg.n_embd, cfg.n_head) == (2, 16, 2)
    assert cfg.fused_kernels.enabled and cfg.fused_kernels.relu_threshold == 0.5
    assert cfg.fused_kernels.rotary_embedding == bda.RotaryEmbedding.ROPE
    assert cfg.fused_kernels.block_sparse.latent.block_size == 32 and not cfg.fused_kernels.block_sparse.latent.is_sparse()
    assert bda.build_model_config(bda.ModelOverrides(block_size=0), 8).fused_kernels.block_sparse.time.block_size == 1


def test_block_patterns():
    """src/kernel/block_sparse.rs:11-117."""
    p = BlockPattern1d.from_blocks(3, [0, 2])
    assert p.is_sparse() and p.is_block_active(2) and not p.is_block_active(1)
    assert p.block_bytes(8) == bytes([1, 0, 1])
    assert np.array_equal(orc.block_mask_1d(8, 3, [0, 2]), [1, 1, 1, 0, 0, 0, 1, 1])
    assert BlockPattern1d.dense(0).block_size == 1 and not BlockPattern1d.dense(4).is_sparse()
    d2 = BlockPattern2d.dense(4)
    assert d2.is_active(2, 1) and d2.is_active(2, 2) and not d2.is_active(1, 2)
    assert d2.iter_cols(2, 5) == [0, 1, 2] and d2.iter_cols(7, 3) == [0, 1, 2] and d2.iter_cols(0, 0) == []
    s2 = BlockPattern2d.from_pairs(4, [(1, 0), (1, 1), (2, 5)])
    assert s2.iter_cols(1, 3) == [0, 1] and s2.iter_cols(2, 3) == [] and s2.is_active(2, 5)


def test_model_state_semantics():
    """src/model/state.rs:27-57."""
    st = bda.ModelState.new(3)
    assert len(st.layers) == 3 and st.position == 0 and st.is_empty()
    st.position = 5
    st.trim(2)  # a no-op in the reference
    assert st.len() == 5
    st.reset()
    assert st.position == 0 and all(l.rho is None for l in st.layers)


def test_rotary_enum():
    """src/positional.rs:8-31."""
    assert bda.RotaryEmbedding.default() == bda.RotaryEmbedding.ALIBI
    assert [r.as_str() for r in bda.RotaryEmbedding] == ["rope", "alibi", "pope"]
    assert bda.RotaryEmbedding.parse("pope") == bda.RotaryEmbedding.POPE
    assert int(bda.RotaryEmbedding.ROPE) == ffi.ROPE == orc.ROPE


def test_no_device_means_loud_failure(lib):
    """Without a HIP device context creation fails; nothing falls back to a CPU path."""
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    handle = ctypes.c_void_p()
    assert lib.bdh_ctx_create(0, None, ctypes.byref(handle)) == ffi.E_HIP
    assert not handle.value
    with pytest.raises(ffi.BdhError):
        ffi.Context(0, stream=0)


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "burn_dragon_amd")
    for dirpath, _, files in os.walk(pkg):
        for name in files:
            if name.endswith((".py", ".hip", ".h", ".cpp", ".hpp")):
                text = open(os.path.join(dirpath, name)).read()
                assert "oracle" not in text.lower(), f"{name} mentions the oracle"


def test_bench_refuses_more_than_one_gpu_and_fails_loudly_without_a_device():
    """bench.py --gpus N with N > 1 exits with a message (the path has no multi-GPU part); without a HIP
    device it fails instead of falling back to a CPU path."""
    import subprocess
    import sys

    bench = os.path.join(ROOT, "bench.py")
    two = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert two.returncode != 0 and "one GPU" in two.stderr and not two.stdout.strip()
    import torch

    if not torch.cuda.is_available():
        one = subprocess.run([sys.executable, bench, "--steps", "1", "--warmup", "0"], capture_output=True, text=True,
                             timeout=300)
        assert one.returncode != 0 and "no HIP device" in one.stderr and not one.stdout.strip()
