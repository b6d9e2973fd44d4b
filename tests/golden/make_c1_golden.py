"""Writes tests/golden/c1_golden.npz from the reference's own CPU path.

Run in the build container, where the reference checkout is mounted and
oracle/_ref/libref.so has been built from its sources (make -C oracle ref):

    python tests/golden/make_c1_golden.py

The fixture holds DATA only: for benchmark configuration 1 (64 tokens,
hidden = inter = 256, 8 experts, top-4, fp32, seed 0) the MoE input the
reference's forward() saw (run.cpp:660), and what it produced: router logits
(run.cpp:664-671), expert ids and softmaxed weights (run.cpp:673-676) and the
layer output e_agg (run.cpp:679-745).  It also holds the results of the
reference's topk() (run.cpp:388-421) on tie vectors, and digests of the
synthetic weights so that a drifting generator is detected.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from gpt_oss_amd import synth  # noqa: E402
from oracle import binding as ob  # noqa: E402


def tie_cases():
    cases = {
        "all_equal_32": np.zeros(32, np.float32),
        "pairs_8": np.array([0.1, 0.7, -0.2, 0.7, 0.3, 0.7, 0.9, 0.3], np.float32),
        "two_levels_16": np.array([1, 2] * 8, np.float32),
        "desc_plateau_12": np.array([5, 5, 5, 4, 4, 4, 3, 3, 3, 2, 2, 2], np.float32),
        "late_max_128": np.concatenate([np.full(127, -1.0, np.float32), np.array([3.0], np.float32)]),
        "neg_zero_8": np.array([0.0, -0.0, 0.0, -0.0, -1, -1, -1, -1], np.float32),
    }
    out = {}
    for name, score in cases.items():
        v = np.zeros(4, np.float32)
        i = np.zeros(4, np.int32)
        ob.ref().ref_topk(v, i, score.copy(), score.shape[0], 4)
        out[f"tie_{name}_score"] = score
        out[f"tie_{name}_idx"] = i
        out[f"tie_{name}_val"] = v
    return out


def main():
    if not ob.ref_available():
        raise SystemExit("oracle/_ref/libref.so missing: run `make -C oracle ref` first")
    sh = synth.CONFIGS["c1"]
    L = synth.make_layer(sh, seed=0)
    R = ob.ref_moe_forward(L["x"], L["w_router"], L["b_router"], L["w_mlp1"], L["b_mlp1"],
                           L["w_mlp2"], L["b_mlp2"], sh.topk, sh.limit)
    data = dict(
        t=R["t"], score=R["score"], topk_i=R["topk_i"], topk_v=R["topk_v"], e_agg=R["e_agg"],
        emb_digest=np.array(synth.digest(L["x"])),
        weights_digest=np.array(synth.digest(L["w_router"], L["b_router"], L["w_mlp1"], L["b_mlp1"],
                                             L["w_mlp2"], L["b_mlp2"])),
    )
    # softmax known answers from the reference (run.cpp:336-354)
    sm_in = np.array([[2.5, 1.0, 0.25, -3.0], [0.0, 0.0, 0.0, 0.0], [10.0, 9.999, -10.0, -10.0]], np.float32)
    sm_out = sm_in.copy()
    for r in sm_out:
        ob.ref().ref_softmax(r, 4)
    data["softmax_in"] = sm_in
    data["softmax_out"] = sm_out
    data.update(tie_cases())
    path = os.path.join(ROOT, "tests", "golden", "c1_golden.npz")
    np.savez_compressed(path, **data)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
