"""Writes tests/golden/kda_vectors.npz: small seeded cases of every operator on the KDA path with the CPU oracle's
results, inputs included, so that a test needs neither the synthetic generator nor a rebuilt oracle to know what
the right answer was when the fixture was made.

The reference ships no tensor payloads for this path (its oracle/goldens/*/tensors.tsv name shapes only and the
.bin files are not in the repository), so these vectors are the oracle's own. What makes them worth trusting is
tests/test_oracle.py, which holds the oracle to the reference's hand-computed values
(crates/glm53f-kda/tests/cpu_reference.rs:36-207), to an f64 textbook recurrence and to the chunked/recurrent
identity. The fixture then serves two purposes: it detects drift of the oracle itself (another compiler, another
flag), bit for bit, and it gives the GPU tests inputs and answers that do not depend on the oracle being built.

Run from the repository root:  python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import kda_oracle as o  # noqa: E402

HEADS = 2
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kda_vectors.npz")


def inputs(prefix, p, conv, state, rows):
    return {
        f"{prefix}.conv_w": p.conv_w, f"{prefix}.a_log": p.a_log, f"{prefix}.dt_bias": p.dt_bias,
        f"{prefix}.norm_w": p.norm_w, f"{prefix}.conv": conv, f"{prefix}.state": state,
        f"{prefix}.qkv": rows.qkv, f"{prefix}.a": rows.a, f"{prefix}.b": rows.b, f"{prefix}.gate": rows.gate,
        f"{prefix}.rows": np.int32(rows.rows),
    }


def main():
    d = {"heads": np.int32(HEADS)}

    # Decode / verify chain, f32 state, 5 rows; its replay to 3 rows and the conv window after keeping 3.
    seed, r, keep = 7001, 5, 3
    p, conv, s0 = o.synth_layer(HEADS, seed), o.synth_conv_window(HEADS, seed), o.synth_state(HEADS, seed, 0.5)
    rows = o.synth_rows(HEADS, r, seed)
    c = o.chain(p, conv, s0, rows)
    d.update(inputs("chain", p, conv, s0, rows))
    d.update({"chain.out": c.out, "chain.state_out": c.state, "chain.save_k": c.saves.k, "chain.save_v": c.saves.v,
              "chain.save_g": c.saves.g, "chain.save_beta": c.saves.beta, "chain.keep": np.int32(keep),
              "chain.replay_state": o.replay(s0, c.saves, keep), "chain.conv_after": o.conv_shift(conv, rows, keep),
              "chain.literal_out": o.literal_chain(p, conv, s0, rows).out,
              "chain.literal_state": o.literal_chain(p, conv, s0, rows).state})

    # The same with a bf16 state (rounded after every row).
    seed = 7002
    p, conv = o.synth_layer(HEADS, seed), o.synth_conv_window(HEADS, seed)
    s0 = o.bf16_round(o.synth_state(HEADS, seed, 0.5))
    rows = o.synth_rows(HEADS, r, seed)
    c = o.chain_bf16_state(p, conv, s0, rows)
    d.update(inputs("chain16", p, conv, s0, rows))
    d.update({"chain16.out": c.out, "chain16.state_out": c.state, "chain16.keep": np.int32(keep),
              "chain16.replay_state": o.replay(s0, c.saves, keep, bf16_state=True)})

    # Prefill over 70 rows (one full chunk and a ragged tail): the FP32 recurrent reference in its literal form.
    seed, r = 7003, 70
    p, conv, s0 = o.synth_layer(HEADS, seed), o.synth_conv_window(HEADS, seed), o.synth_state(HEADS, seed, 0.5)
    rows = o.synth_rows(HEADS, r, seed)
    lit = o.literal_chain(p, conv, s0, rows)
    d.update(inputs("prefill", p, conv, s0, rows))
    d.update({"prefill.out": lit.out, "prefill.state_out": lit.state,
              "prefill.conv_after": o.conv_shift(conv, rows, r)})

    np.savez_compressed(OUT, **{k: np.asarray(v) for k, v in d.items()})
    print(f"wrote {OUT}: {len(d)} arrays, {os.path.getsize(OUT)} bytes")


if __name__ == "__main__":
    main()
