"""Writes the small golden vectors under tests/golden/.

The reference (mosure/burn_dragon) is Rust-only and cannot be run in this environment, and its own
tests hold no value vectors for the recurrent path, so these fixtures come from the C oracle
(oracle/bdh_oracle.c) AFTER it has been pinned by tests/test_oracle.py.  They freeze the oracle's
behaviour (a regression guard for later edits) and give the GPU tests a committed target.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import bdh_oracle as orc  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def state_step_case(corc, seed, B, h, T, N, d, rotary, position, slopes=None):
    rng = np.random.default_rng(seed)
    x = np.maximum(rng.standard_normal((B, h, T, N)) - 0.8, 0).astype(np.float32)
    v = rng.standard_normal((B, T, d)).astype(np.float32)
    Nq = 2 * N if rotary == orc.POPE else N
    rho0 = (0.05 * rng.standard_normal((B, h, Nq, d))).astype(np.float32)
    freqs = corc.build_freqs(N, 65536.0, rotary)
    decay = None if slopes is None else corc.alibi_decay(slopes)
    q = corc.rotate(x, freqs, rotary, position)
    out, rho1 = corc.recurrent_attention(q, v, rho0, decay)
    return dict(x=x, v=v, rho0=rho0, freqs=freqs, position=np.int64(position), rotary=np.int32(rotary),
                slopes=np.zeros(0, np.float32) if slopes is None else np.asarray(slopes, np.float32), out=out, rho1=rho1,
                bitmask=orc.active_bitmask(np.pad(x, ((0, 0), (0, 0), (0, 0), (0, (-N) % 64)))),
                rows=orc.pair_closed_rows(x).astype(np.int32))


def main():
    corc = orc.COracle()
    cases = {
        "rope_d256": state_step_case(corc, 1, 1, 1, 2, 64, 256, orc.ROPE, 1234),
        "rope_small": state_step_case(corc, 2, 2, 2, 3, 32, 16, orc.ROPE, 7),
        "alibi_small": state_step_case(corc, 3, 2, 2, 3, 32, 16, orc.ALIBI, 7, slopes=[0.5, 0.125]),
        "pope_small": state_step_case(corc, 4, 1, 2, 2, 32, 16, orc.POPE, 7),
    }
    flat = {f"{name}.{key}": val for name, case in cases.items() for key, val in case.items()}
    np.savez_compressed(os.path.join(HERE, "state_step.npz"), **flat)

    shape = orc.BDHShape(n_layer=2, n_embd=16, n_head=2, mlp_internal_dim_multiplier=4, vocab_size=32, rotary=orc.ROPE)
    w = orc.init_weights(shape, seed=11)
    tokens = np.arange(8).reshape(2, 4)
    rho = np.zeros((2, 2, 2, 32, 16), np.float32)
    logits, pos, _, _ = corc.forward_with_state(shape, w, tokens, rho, 0, sparse_state=False)
    np.savez_compressed(os.path.join(HERE, "model_paths_rope.npz"), tokens=tokens, logits=logits, rho=rho,
                        position=np.int64(pos), seed=np.int64(11))
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()
