"""Writes the small regression fixtures in this directory from the CPU oracle.

The reference holds no tensor fixtures for this path (its tests read refs/, which is not in
its repository), so these are the oracle's own outputs on seeded inputs, frozen once the
oracle was pinned by the checks in tests/test_oracle_*.py. They let the GPU tests compare
against bytes on disk as well as against the oracle built from source, and they catch an
accidental change of the canonical arithmetic on either side.

    python tests/golden/make_golden.py        # rewrites *.npz / *.json next to this file
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import synth  # noqa: E402
import util  # noqa: E402


def main():
    rng = np.random.default_rng(20251)
    # 1. Q4_K mat-vec of BASELINE config 1's kind (fp32 x, fp32 y), 128 rows x 2048, plus float64
    O, K = 128, 2048
    qs, scales, dm = util.make_q4k(rng, 1, O, K)
    x = rng.standard_normal((1, K)).astype(np.float32)
    y = util.orc_qmv(util.Q4K, qs, scales, dm, O, K, x)
    w = util.orc_dequant(util.Q4K, qs, scales, dm, O * K // 256).reshape(O, K).astype(np.float64)
    np.savez_compressed(os.path.join(HERE, "q4k_qmv_128x2048.npz"), qs=qs, scales=scales, dm=dm, x=x,
                        y_oracle=y, y_float64=(w @ x[0].astype(np.float64)))
    # 2. Q6_K mat-vec, bf16 activations and outputs
    O6, K6 = 64, 1024
    q6 = util.make_q6k(rng, 1, O6, K6)
    xb = util.bf16_normal(rng, (2, K6))
    y6 = util.f32_to_bf16(util.orc_qmv(util.Q6K, *q6, O6, K6, util.bf16_to_f32(xb), round_bf16=True))
    np.savez_compressed(os.path.join(HERE, "q6k_qmv_64x1024.npz"), qs=q6[0], scales=q6[1], dm=q6[2], x=xb, y=y6)
    # 3. router: softmax + top-8 of 256 with planted ties
    gates = util.bf16_normal(rng, (4, 256))
    gates[1, 10:40] = gates[1, 5]
    gates[2, :] = gates[2, 0]
    probs = np.empty((4, 256), np.uint16); inds = np.empty((4, 8), np.uint32); scores = np.empty((4, 8), np.uint16)
    util.oracle().orc_softmax_bf16(util.p(gates), 4, 256, util.p(probs))
    util.oracle().orc_router_topk(util.p(probs), 4, 256, 8, util.p(inds), util.p(scores))
    np.savez_compressed(os.path.join(HERE, "router_topk_4x256.npz"), gates=gates, inds=inds, scores=scores, probs=probs)
    # 4. tiny model: greedy tokens, depth-2 speculative stats, sampled tokens
    s = synth.SynthModel(synth.TINY, seed=3)
    prompt = np.random.default_rng(7).integers(0, s.cfg["vocab_size"], 7).astype(np.uint32)
    orc = synth.OracleRun(s, 64)
    greedy = orc.generate(prompt, 12, prefill_step=4)
    orc.close()
    orc = synth.OracleRun(s, 64)
    toks, st = orc.mtp_generate(prompt, 2, 12, policy=1, prefill_step=4)
    orc.close()
    orc = synth.OracleRun(s, 64)
    orc.set_sampler(1, 0.8, 0.95, 20, 99)
    sampled = orc.generate(prompt, 12, prefill_step=4)
    orc.set_sampler(0)
    orc.close()
    assert toks == greedy
    json.dump({"config": "synth.TINY", "model_seed": 3, "prompt": [int(t) for t in prompt], "greedy": greedy,
               "mtp_depth2": {"cycles": int(st.cycles), "drafted": int(st.drafted), "accepted": int(st.accepted)},
               "sampled_t0.8_p0.95_k20_seed99": sampled},
              open(os.path.join(HERE, "tiny_model_tokens.json"), "w"), indent=1)
    print("fixtures written to", HERE)


if __name__ == "__main__":
    main()
