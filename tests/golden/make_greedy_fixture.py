"""Writes the greedy-decoding fixtures under tests/golden/ with the CPU oracle.

    python tests/golden/make_greedy_fixture.py llama7b_fp16 [seed [prompt_len [steps [flavour]]]]
    python tests/golden/make_greedy_fixture.py llama30b_u8 [seed [prompt_len [steps [flavour]]]]

Each fixture holds the model shape, the seeds, the 512 prompt token ids, the 128 greedy tokens the
oracle produces (temperature 0.8 as main.cpp:58), and for every step the two largest fp16 logits
with their token ids and the two largest probabilities.  Two fixtures per model:
  flavour 2 (default) -> <name>_seed<seed>_greedy.json: every sum in the order of the HIP kernels
    (the matrix cores' steps of eight products and the dispatcher's cut of K for the prompt, the
    lane and wavefront order of the decode kernels, v_dot2_f32_f16 for uint8 weights), so that the
    whole run can be held to the GPU bit for bit;
  flavour 1 -> <name>_seed<seed>_greedy_reference_order.json: the sums as the reference's own
    kernels order them (llama_cu.cu:150-366: 16-wide k steps per tile, sequential attention dots),
    which is what ties the full-depth run to the reference's arithmetic; the GPU is held to it
    within a tolerance, token for token except where the oracle's own two best logits nearly tie.
Only the oracle runs here; nothing from the reference is imported or executed.
"""
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as O  # noqa: E402

CONFIGS = {
    "llama7b_fp16": dict(dim=4096, multiple_of=256, n_heads=32, n_layers=32, n_vocab=32000, q_type=0),
    "llama30b_u8": dict(dim=6656, multiple_of=256, n_heads=52, n_layers=60, n_vocab=32000, q_type=1),
    "tiny_fp16": dict(dim=512, multiple_of=128, n_heads=4, n_layers=4, n_vocab=2048, q_type=0),
    "tiny_u8": dict(dim=512, multiple_of=128, n_heads=4, n_layers=4, n_vocab=2048, q_type=1),
}


def main():
    name = sys.argv[1]
    seed = int(sys.argv[2]) if len(sys.argv) > 2 else 0
    prompt_len = int(sys.argv[3]) if len(sys.argv) > 3 else 512
    steps = int(sys.argv[4]) if len(sys.argv) > 4 else 128
    flavour = int(sys.argv[5]) if len(sys.argv) > 5 else 2
    cfg = CONFIGS[name]
    t0 = time.time()
    model = O.Model(norm_eps=1e-6, qblock=128, seed=seed, weight_std=0.02, **cfg)
    print("model built in %.1fs (ffn %d)" % (time.time() - t0, model.ffn), flush=True)
    ctx = O.Context(model, context_len=2048, temperature=0.8, flavour=flavour)
    prompt = np.random.default_rng(seed).integers(0, cfg["n_vocab"], prompt_len).astype(np.int16)
    tokens, top, top_ids = [], [], []
    feed = prompt
    for step in range(steps):
        t1 = time.time()
        tok, _, logits, probs = ctx.next_token(feed, want=True)
        lf = logits.astype(np.float32)
        order = np.argsort(-lf, kind="stable")[:2]  # stable: the lower id first among equals
        lo = lf[order[::-1]]
        po = np.sort(probs.astype(np.float32))[-2:]
        tokens.append(int(tok))
        top.append([float(lo[1]), float(lo[0]), float(po[1]), float(po[0])])
        top_ids.append([int(order[0]), int(order[1])])
        feed = np.array([tok], dtype=np.int16)
        print("step %d token %d logit margin %.5f (%.1fs)" % (step, tok, lo[1] - lo[0], time.time() - t1), flush=True)
    out = dict(name=name, matmul_flavour=flavour, seed=seed, weight_std=0.02, norm_eps=1e-6, qblock=128, temperature=0.8, context_len=2048,
               prompt=[int(t) for t in prompt], tokens=tokens, top2_logits_probs=top, top2_ids=top_ids, **cfg)
    path = os.path.join(HERE, "%s_seed%d_greedy%s.json" % (name, seed, "" if flavour == 2 else "_reference_order"))
    with open(path, "w") as f:
        json.dump(out, f)
    print("wrote", path, "in %.1fs" % (time.time() - t0))


if __name__ == "__main__":
    main()
