#!/usr/bin/env python3
"""Where the time of two decode launches goes, read inside the kernels: the fused launch (attention + Wo
+ residual + FFN norm, one 1024-thread workgroup per compute unit) by phase, and the W2 launch with its
follower (2048 GEMV workgroups of two rows + one workgroup that normalises the new row) by workgroup.

    python llama.cu_amd/build.py --timeline      # libllama_cu_amd_timeline.so (diagnostic build)
    python llama.cu_amd/timeline.py [--steps K]

The diagnostic build notes the device's 100 MHz real-time counter at the end of every phase of
decode_attention_wo_norm_kernel (thread 0 of each workgroup, and the first lane of its first Wo
wavefront), one row per layer.  This script decodes a LLaMA-7B-shaped fp16 model after a 512-token
prompt, clears the notes before the last K steps' final one, and prints for every phase boundary the
time since the launch's first workgroup started: the median and the latest workgroup, median over the
layers of the step.  The step is replayed from the HIP graph like any other.
"""
import argparse
import ctypes as C
import importlib.util
import os
import sys

import numpy as np

PKG = os.path.dirname(os.path.abspath(__file__))
POINTS, LAUNCHES, GROUPS = 16, 64, 512
NAMES = {
    0: "workgroup started",
    1: "own scores written (K rows fetched, 72 dot products per slice at T = 576)",
    2: "the head's scores arrived (hand-over 1)",
    3: "barrier 1: row maximum known",
    4: "barrier 3: sum of exponentials known",
    5: "barrier 4: probabilities in LDS",
    6: "attention output of the 16 columns written (hand-over 2 begins)",
    7: "whole attention output gathered (hand-over 2), barrier 6",
    13: "Wo rows summed by the first Wo wavefront",
    8: "barrier 7: the 16 rows of x + Wo.att known",
    9: "new residual rows written (hand-over 3 begins)",
    10: "whole residual row gathered (hand-over 3), barrier 8",
    11: "norm written, workgroup done",
    12: "last Wo batch requested (first Wo wavefront)",
}
ORDER = [0, 1, 2, 3, 4, 12, 5, 6, 7, 13, 8, 9, 10, 11]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=16)
    args = ap.parse_args()
    lib_path = os.path.join(PKG, "libllama_cu_amd_timeline.so")
    if not os.path.exists(lib_path):
        sys.exit("build the diagnostic library first: python llama.cu_amd/build.py --timeline")
    os.environ["LLAMA_CU_AMD_LIB"] = lib_path
    spec = importlib.util.spec_from_file_location("llama_cu_amd", os.path.join(PKG, "__init__.py"),
                                                  submodule_search_locations=[PKG])
    P = importlib.util.module_from_spec(spec)
    sys.modules["llama_cu_amd"] = P
    spec.loader.exec_module(P)
    B = P.binding
    B.init(0)
    L = B.lib()
    read = L.lcu_debug_timeline_read
    read.restype = C.c_int
    read.argtypes = [C.c_void_p, C.c_size_t]
    cfg = dict(dim=4096, multiple_of=256, n_heads=32, n_layers=32, n_vocab=32000, q_type=0)
    model = P.Model(norm_eps=1e-6, qblock=128, seed=0, weight_std=0.02, **cfg)
    ctx = P.Context(model, context_len=2048, temperature=0.8)
    tok = ctx.next_token(np.random.default_rng(0).integers(0, cfg["n_vocab"], 512).astype(np.int16))
    for _ in range(args.steps - 1):
        tok = ctx.next_token([tok])
    read_proj = L.lcu_debug_timeline_read_proj
    read_proj.restype = C.c_int
    read_proj.argtypes = [C.c_void_p, C.c_size_t]
    B.check(read(None, 0), "clear")
    B.check(read_proj(None, 0), "clear")
    tok = ctx.next_token([tok])
    notes = np.zeros((LAUNCHES, GROUPS, POINTS), dtype=np.uint64)
    B.check(read(notes.ctypes.data, notes.nbytes), "read")
    proj = np.zeros((LAUNCHES, 4096, 4), dtype=np.uint64)
    B.check(read_proj(proj.ctypes.data, proj.nbytes), "read")
    layers, groups = cfg["n_layers"], 8 * cfg["n_heads"]
    t = notes[:layers, :groups, :].astype(np.int64)
    assert (t[:, :, 0] > 0).all(), "the fused launch did not run (diagnostic library not loaded?)"
    start = t[:, :, 0].min(axis=1)                       # first workgroup of each layer's launch
    rel = (t - start[:, None, None]) / 100.0             # microseconds
    print("decode_attention_wo_norm_kernel, LLaMA-7B fp16, %d cached rows, step replayed from the graph;" % (512 + args.steps))
    print("microseconds since the launch's first workgroup started; median over the %d layers of" % layers)
    print("(median workgroup, latest workgroup):")
    prev = 0.0
    for p in ORDER:
        med = float(np.median(np.median(rel[:, :, p], axis=1)))
        late = float(np.median(rel[:, :, p].max(axis=1)))
        print("  %6.2f  %6.2f  (+%5.2f)  %s" % (med, late, med - prev if p not in (12, 13) else 0.0, NAMES[p]))
        if p not in (12, 13):
            prev = med
    total = (t[:, :, 11].max(axis=1) - start) / 100.0
    print("launch, first start to last end: median %.2f us over the layers (min %.2f, max %.2f)"
          % (float(np.median(total)), float(total.min()), float(total.max())))
    gaps = (start[1:] - t[:-1, :, 11].max(axis=1)) / 100.0
    print("from the end of one layer's launch to the start of the next one's (three other launches lie between): "
          "median %.2f us" % float(np.median(gaps)))
    proj_report(proj.astype(np.int64), cfg)
    ctx.close()
    model.close()


def proj_report(p, cfg):
    """decode_proj_norm_kernel, W2 of layers 0 .. n_layers - 2 (the last layer's W2 has no norm behind it and is
    a plain GEMV): rows of p are [layer][workgroup][start, follower has every word in LDS, end, follower knows the sum of squares]."""
    n_rows, ffn = cfg["dim"], 11008
    gemv = n_rows // 2                      # workgroups of two rows; workgroup `gemv` is the follower
    layers = cfg["n_layers"] - 1
    med = lambda v: float(np.median(v))
    out = {k: [] for k in ("s25", "s50", "s75", "s100", "life10", "life50", "life90", "d50", "d90", "d99", "d100",
                           "f_start", "f_seen", "f_end", "f_sum", "peak", "first_done")}
    for l in range(layers):
        start, end = p[l, :gemv, 0], p[l, :gemv, 2]
        assert (start > 0).all() and (end >= start).all(), "the W2 launch of layer %d left no notes" % l
        t0 = start.min()
        s, e = np.sort(start - t0) / 100.0, np.sort(end - t0) / 100.0
        life = (end - start) / 100.0
        for k, q in (("s25", 0.25), ("s50", 0.5), ("s75", 0.75), ("s100", 1.0)):
            out[k].append(s[int(q * gemv) - 1])
        for k, q in (("d50", 0.5), ("d90", 0.9), ("d99", 0.99), ("d100", 1.0)):
            out[k].append(e[int(q * gemv) - 1])
        out["first_done"].append(e[0])
        for k, q in (("life10", 10), ("life50", 50), ("life90", 90)):
            out[k].append(np.percentile(life, q))
        events = np.concatenate([np.stack([start, np.ones_like(start)], 1), np.stack([end, -np.ones_like(end)], 1)])
        events = events[np.lexsort((events[:, 1], events[:, 0]))]
        out["peak"].append(np.cumsum(events[:, 1]).max())
        f = (p[l, gemv, :4] - t0) / 100.0
        out["f_start"].append(f[0]); out["f_seen"].append(f[1]); out["f_end"].append(f[2]); out["f_sum"].append(f[3])
    m = {k: med(v) for k, v in out.items()}
    print()
    print("decode_proj_norm_kernel<false, 2, 2, 0>, W2 (%d x %d fp16, 90.2 MB) + residual + the next attention norm;" % (n_rows, ffn))
    print("microseconds since the launch's first workgroup started, median over %d layers of one step:" % layers)
    print("  GEMV workgroups started: a quarter by %.2f, half by %.2f, three quarters by %.2f, all by %.2f" % (m["s25"], m["s50"], m["s75"], m["s100"]))
    print("  most workgroups alive at once: %d of %d (eight fit a compute unit: 2048 on the chip)" % (m["peak"], gemv))
    print("  a workgroup lives (start to result stored): %.2f / %.2f / %.2f (10th / 50th / 90th percentile)" % (m["life10"], m["life50"], m["life90"]))
    print("  results stored: first %.2f, half by %.2f, 90 %% by %.2f, 99 %% by %.2f, all by %.2f" % (m["first_done"], m["d50"], m["d90"], m["d99"], m["d100"]))
    print("  follower: started %.2f, every word seen and in LDS %.2f (+%.2f after the last store), sum of squares %.2f (+%.2f), "
          "norm written %.2f (+%.2f)" % (m["f_start"], m["f_seen"], m["f_seen"] - m["d100"], m["f_sum"],
                                         m["f_sum"] - m["f_seen"], m["f_end"], m["f_end"] - m["f_sum"]))
    print("  90.2 MB in %.2f us from first start to last GEMV store = %.0f GB/s; to the follower's end %.2f us"
          % (m["d100"], 90207744 / m["d100"] / 1e3, m["f_end"]))


if __name__ == "__main__":
    main()
