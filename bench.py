#!/usr/bin/env python3
"""Headline benchmark: batch-1 greedy decode of a LLaMA-7B-shaped fp16 model on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama7b_fp16|llama30b_u8]

A step is one decode step (one new token through all layers, logits, softmax, argmax, 4-byte
read-back) after a 512-token prompt; weights are seeded random values of the model's shape
(there are no checkpoints here), so `data` is "synthetic".  Prints one JSON line:
  value        tokens/s over exactly K timed steps (inputs and weights resident in HBM)
  roofline     achieved / frac: the whole decode step, all bytes a step must read (weights + KV
               cache) / the measured step time, against 8 TB/s -- the quantity the decode target is
               stated in; kernel_achieved / kernel_frac / us_per_launch: the dominant decode kernel
               (W1/W3 GEMV + SiLU*mul of one layer, on an already normalised row) launched back to
               back over the model's own layers, timed with HIP events on its stream: algorithmic
               bytes per launch / average launch time; traffic: that kernel's measured HBM bytes
  cpu_baseline the CPU oracle (a port of the reference's arithmetic, OpenMP) decoding on the host
               cores on a bounded sample, extrapolated to the full depth; reported only
  extra        per-shape GEMV GB/s, prefill GEMM TFLOP/s and prefill time measured in the same run,
               and the other model of the metric (LLaMA-30B shape, uint8 weights) decoded the same way
"""
import argparse
import ctypes as C
import importlib.util
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "llama.cu_amd")
HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
# HBM bytes per launch of the dominant kernel from rocprofv3 FETCH_SIZE / WRITE_SIZE, scaled by a
# 256 MiB copy kernel read under the same counters (FETCH_SIZE reads half the bytes here): see
# profiles/decode_ffn_up_kernel_llama7b_hbm_traffic.txt and decode_u8_kernels_llama30b_counters.txt.
# Counters are not read in this script.
MEASURED_TRAFFIC = {"llama7b_fp16": 180637530, "llama30b_u8": 244906771}
MFMA_F16_PEAK_TF = 2500.0  # dense fp16

WORKLOADS = {
    "llama7b_fp16": dict(dim=4096, multiple_of=256, n_heads=32, n_layers=32, n_vocab=32000, q_type=0),
    "llama30b_u8": dict(dim=6656, multiple_of=256, n_heads=52, n_layers=60, n_vocab=32000, q_type=1),
}
PROMPT = 512


def load_package():
    spec = importlib.util.spec_from_file_location("llama_cu_amd", os.path.join(PKG, "__init__.py"),
                                                  submodule_search_locations=[PKG])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["llama_cu_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


class Timer:
    """HIP events on a given stream (lcu_event_*)."""

    def __init__(self, B, stream):
        self.B, self.L, self.stream = B, B.lib(), stream
        self.e0, self.e1 = B.vp(), B.vp()
        B.check(self.L.lcu_event_create(C.byref(self.e0)))
        B.check(self.L.lcu_event_create(C.byref(self.e1)))

    def start(self):
        self.B.check(self.L.lcu_event_record(self.e0, self.stream))

    def stop_ms(self):
        self.B.check(self.L.lcu_event_record(self.e1, self.stream))
        ms = C.c_float()
        self.B.check(self.L.lcu_event_elapsed_ms(C.byref(ms), self.e0, self.e1))
        return float(ms.value)


def weight_bytes(cfg, ffn):
    d, v, L = cfg["dim"], cfg["n_vocab"], cfg["n_layers"]
    per_elem = 2.0 if cfg["q_type"] == 0 else 1.0 + 2.0 / 128
    layer = (4 * d * d + 3 * ffn * d) * per_elem + 2 * d * 2
    return L * layer + v * d * per_elem + d * 2 + d * per_elem  # + final norm + one embedding row


def decode_leg(P, cfg, steps, warmup):
    B = P.binding
    L = B.lib()
    model = P.Model(norm_eps=1e-6, qblock=128, seed=0, weight_std=0.02, **cfg)
    ctx = P.Context(model, context_len=2048, temperature=0.8)
    prompt = np.random.default_rng(0).integers(0, cfg["n_vocab"], PROMPT).astype(np.int16)
    B.check(L.lcu_sync(None))
    t0 = time.perf_counter()
    tok = ctx.next_token(prompt)
    B.check(L.lcu_sync(None))
    prefill_ms = (time.perf_counter() - t0) * 1e3
    for _ in range(warmup):
        tok = ctx.next_token([tok])
    B.check(L.lcu_sync(None))
    step_ms = []
    t0 = time.perf_counter()
    for _ in range(steps):
        t1 = time.perf_counter()
        tok = ctx.next_token([tok])  # returns after the 4-byte read-back: the step is complete
        step_ms.append((time.perf_counter() - t1) * 1e3)
    B.check(L.lcu_sync(None))
    total_s = time.perf_counter() - t0
    # a second, timed prefill on a cleared context (the first one paid one-off set-up costs)
    ctx.clear_tokens()
    B.check(L.lcu_sync(None))
    t0 = time.perf_counter()
    ctx.next_token(prompt)
    B.check(L.lcu_sync(None))
    prefill2_ms = (time.perf_counter() - t0) * 1e3
    T_mid = PROMPT + warmup + steps / 2.0
    kv_bytes = T_mid * cfg["dim"] * 2 * 2 * cfg["n_layers"]
    res = dict(tok_s=steps / total_s, ms_per_step=total_s / steps * 1e3, median_ms=float(np.median(step_ms)),
               prefill_first_ms=prefill_ms, prefill_ms=prefill2_ms,
               bytes_per_token=weight_bytes(cfg, model.ffn) + kv_bytes)
    return model, ctx, res


def ffn_up_kernel_leg(P, cfg, model, ctx, launches):
    """The dominant decode kernel on the real weights of consecutive layers (no two launches in a
    row touch the same weights, so no cache serves the stream)."""
    B = P.binding
    L = B.lib()
    d, ffn, nl = cfg["dim"], model.ffn, cfg["n_layers"]
    block = 128 if cfg["q_type"] == 1 else 0
    x = B.empty((d,), np.float16)
    out = B.empty((ffn,), np.float16)
    B.check(L.lcu_fill_normal_f16(x.ptr, d, 1, 999, 1.0, ctx.stream))
    ptrs = []
    for l in range(nl):
        w1, s1 = model.tensor_ptr(16 + 16 * l + 4)
        w3, s3 = model.tensor_ptr(16 + 16 * l + 6)
        ptrs.append((w1, w3, s1, s3))

    def launch(i):
        w1, w3, s1, s3 = ptrs[i % nl]
        # norm weights NULL: x is already normalised, as in the decode step (lcu_rmsnorm runs before)
        B.check(L.lcu_decode_ffn_up(out.ptr, x.ptr, None, w1, w3, s1, s3, block, d, ffn, 1e-6, ctx.stream))

    for i in range(nl):
        launch(i)
    t = Timer(B, ctx.stream)
    t.start()
    for i in range(launches):
        launch(i)
    us = t.stop_ms() * 1e3 / launches
    per_elem = 2.0 if cfg["q_type"] == 0 else 1.0 + 2.0 / 128
    algo = 2 * ffn * d * per_elem + d * 2 + ffn * 2  # W1 + W3 (+ scales), x, output
    return us, algo


def gemv_leg(P, stream):
    """The single matrix-vector products of the benchmark configurations (fp16 and uint8 weights, M = 1): GB/s of
    the plain GEMV entry point, weight copies rotated."""
    B = P.binding
    L = B.lib()
    out = {}
    for name, K, N, u8, copies in [("f16_11008x4096", 4096, 11008, False, 8), ("f16_4096x4096", 4096, 4096, False, 20),
                                   ("f16_4096x11008", 11008, 4096, False, 8), ("u8_4096x4096", 4096, 4096, True, 40),
                                   ("u8_11008x4096", 4096, 11008, True, 16), ("u8_4096x11008", 11008, 4096, True, 16)]:
        ws = []
        for c in range(copies):
            if u8:
                w = B.empty((N, K), np.uint8)
                B.check(L.lcu_fill_normal_f16(w.ptr, N * K // 2, 0, c, 0.02, stream))  # arbitrary code bytes
                s = B.empty((N, K // 128), np.float16)
                B.check(L.lcu_fill_f16(s.ptr, N * K // 128, 0x1400, stream))
                ws.append((w, s))
            else:
                w = B.empty((N, K), np.float16)
                B.check(L.lcu_fill_normal_f16(w.ptr, N * K, 0, c, 0.02, stream))
                ws.append((w, None))
        x = B.empty((K,), np.float16)
        B.check(L.lcu_fill_normal_f16(x.ptr, K, 0, 99, 1.0, stream))
        o = B.empty((N,), np.float16)

        def launch(i):
            w, s = ws[i % copies]
            if u8:
                B.check(L.lcu_gemm_f16u8_nt(o.ptr, x.ptr, w.ptr, s.ptr, 1, K, N, 128, 0.0, stream))
            else:
                B.check(L.lcu_gemm_f16_nt(o.ptr, x.ptr, w.ptr, 1, K, N, 0.0, stream))

        for i in range(copies):
            launch(i)
        t = Timer(B, stream)
        t.start()
        iters = 200
        for i in range(iters):
            launch(i)
        us = t.stop_ms() * 1e3 / iters
        algo = (N * K * (1 if u8 else 2)) + (N * (K // 128) * 2 if u8 else 0) + K * 2 + N * 2
        out[name] = dict(us=round(us, 2), gb_s=round(algo / us / 1e3, 1), frac_of_8tbs=round(algo / us / 1e3 / HBM_PEAK_GBS, 3))
        for w, s in ws:
            w.free()
            if s is not None:
                s.free()
    return out


def gemm_leg(P, stream):
    """512-token prefill GEMMs of the 7B shapes (fp16 and uint8 weights): TFLOP/s against dense fp16 MFMA peak."""
    B = P.binding
    L = B.lib()
    out = {}
    M = 512
    for name, K, N, u8 in [("f16_512x4096x4096", 4096, 4096, False), ("f16_512x4096x11008", 4096, 11008, False),
                           ("f16_512x11008x4096", 11008, 4096, False), ("u8_512x4096x4096", 4096, 4096, True),
                           ("u8_512x4096x11008", 4096, 11008, True), ("u8_512x11008x4096", 11008, 4096, True)]:
        # enough copies that neither the L2s nor the 256 MB memory-side cache can serve the weights
        copies = max(4, -(-640 * 2**20 // (N * K * (1 if u8 else 2))))
        ws = []
        for c in range(copies):
            if u8:
                w = B.empty((N, K), np.uint8)
                B.check(L.lcu_fill_normal_f16(w.ptr, N * K // 2, 0, c, 0.02, stream))
                s = B.empty((N, K // 128), np.float16)
                B.check(L.lcu_fill_f16(s.ptr, N * K // 128, 0x1400, stream))
                ws.append((w, s))
            else:
                w = B.empty((N, K), np.float16)
                B.check(L.lcu_fill_normal_f16(w.ptr, N * K, 0, c, 0.02, stream))
                ws.append((w, None))
        x = B.empty((M, K), np.float16)
        B.check(L.lcu_fill_normal_f16(x.ptr, M * K, 0, 99, 1.0, stream))
        o = B.empty((M, N), np.float16)

        def launch(i):
            w, s = ws[i % copies]
            if u8:
                B.check(L.lcu_gemm_f16u8_nt(o.ptr, x.ptr, w.ptr, s.ptr, M, K, N, 128, 0.0, stream))
            else:
                B.check(L.lcu_gemm_f16_nt(o.ptr, x.ptr, w.ptr, M, K, N, 0.0, stream))

        for i in range(copies):
            launch(i)
        t = Timer(B, stream)
        t.start()
        iters = max(50, 2 * copies)
        for i in range(iters):
            launch(i)
        us = t.stop_ms() * 1e3 / iters
        fl = 2.0 * M * K * N
        out[name] = dict(us=round(us, 2), tflops=round(fl / us / 1e6, 1), frac_of_mfma_peak=round(fl / us / 1e6 / MFMA_F16_PEAK_TF, 3))
        for w, s in ws:
            w.free()
            if s is not None:
                s.free()
    return out


def cpu_baseline_leg(cfg):
    """The CPU oracle (the checker, here only as the reported baseline) on 2- and 6-layer slices of
    the same model shape: per-layer and head costs measured, then extrapolated to the full depth."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as O
    small = dict(cfg)
    deep, shallow = (6, 2) if cfg["dim"] <= 4096 else (3, 1)
    small["n_layers"] = deep
    m2 = O.Model(norm_eps=1e-6, qblock=128, seed=0, weight_std=0.02, **small)
    small["n_layers"] = shallow
    m1 = O.Model(norm_eps=1e-6, qblock=128, seed=0, weight_std=0.02, **small)
    prompt = np.random.default_rng(0).integers(0, cfg["n_vocab"], PROMPT).astype(np.int16)
    times = []
    steps = 6
    for m in (m1, m2):
        c = O.Context(m, context_len=1024, temperature=0.8)
        tok = c.next_token(prompt)
        c.next_token([tok])
        t0 = time.perf_counter()
        for _ in range(steps):
            tok = c.next_token([tok])
        times.append((time.perf_counter() - t0) / steps)
        c.close()
    per_layer = max((times[1] - times[0]) / (deep - shallow), 1e-9)
    head = max(times[0] - per_layer * shallow, 0.0)
    full = head + per_layer * cfg["n_layers"]
    cores = O.lib().orc_num_threads()
    return dict(value=round(1.0 / full, 3), unit="tok/s", cores=int(cores), kind="port",
                sample="CPU oracle decode at T~%d on %d- and %d-layer models of the same shape, %d steps each; "
                       "per-layer %.1f ms and embedding+logits %.1f ms extrapolated to %d layers"
                       % (PROMPT + 2, shallow, deep, steps, per_layer * 1e3, head * 1e3, cfg["n_layers"]))


def batched_leg(P, model, cfg, sizes=(8, 32), prompt=64, steps=32, warmup=4):
    """llama_batch_context: aggregate decode tok/s of several sequences stepping together (every weight is
    read once per step for the whole batch); each sequence starts from its own random prompt."""
    import time
    out = {}
    rng = np.random.default_rng(7)
    for n_seq in sizes:
        bc = P.BatchContext(model, n_seq, context_len=512, temperature=0.8)
        last = [bc.next_token(b, rng.integers(0, cfg["n_vocab"], prompt).astype(np.int16)) for b in range(n_seq)]
        for _ in range(warmup):
            last = bc.next_tokens(last)
        t0 = time.perf_counter()
        for _ in range(steps):
            last = bc.next_tokens(last)   # blocks on the tokens coming back, as a serving loop would
        dt = time.perf_counter() - t0
        out["sequences_%d" % n_seq] = {"ms_per_step": round(dt / steps * 1e3, 3), "tok_s": round(n_seq * steps / dt, 1)}
        bc.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--workload", default="llama7b_fp16", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the per-shape GEMV / GEMM legs")
    ap.add_argument("--no-batched", action="store_true", help="skip the batched-decode leg of the extra figures")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 256 MiB device-to-device copy: a copy kernel of known size, against which "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings of the other kernels are scaled")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.stderr.write("bench.py: this build runs on one GPU (the whole model fits in one MI355X's HBM); "
                         "--gpus %d is not supported\n" % args.gpus)
        sys.exit(2)
    P = load_package()
    B = P.binding
    B.init(0)
    cfg = WORKLOADS[args.workload]
    model, ctx, dec = decode_leg(P, cfg, args.steps, args.warmup)
    k_us, k_bytes = ffn_up_kernel_leg(P, cfg, model, ctx, 4 * cfg["n_layers"])
    achieved = k_bytes / k_us / 1e3  # GB/s
    extra = dict(decode_median_ms=round(dec["median_ms"], 4), prefill_512_ms=round(dec["prefill_ms"], 3),
                 decode_bytes_per_token=int(dec["bytes_per_token"]),
                 decode_hbm_gb_s=round(dec["bytes_per_token"] / dec["ms_per_step"] / 1e6, 1),
                 decode_frac_of_hbm_roofline=round(dec["bytes_per_token"] / dec["ms_per_step"] / 1e6 / HBM_PEAK_GBS, 3))
    ctx.close()
    if not args.no_extra and not args.no_batched:
        extra["batched_decode"] = batched_leg(P, model, cfg)
    ffn = model.ffn
    model.close()
    if not args.no_extra and args.workload == "llama7b_fp16":
        # the other model the metric names: LLaMA-30B shape with uint8 weights, decoded the same way
        cfg30 = WORKLOADS["llama30b_u8"]
        m30, c30, d30 = decode_leg(P, cfg30, args.steps, args.warmup)
        extra["llama30b_u8"] = dict(tok_s=round(d30["tok_s"], 2), ms_per_step=round(d30["ms_per_step"], 4),
                                    prefill_512_ms=round(d30["prefill_ms"], 3),
                                    decode_bytes_per_token=int(d30["bytes_per_token"]),
                                    frac=round(d30["bytes_per_token"] / d30["ms_per_step"] / 1e6 / HBM_PEAK_GBS, 3))
        c30.close()
        m30.close()
    if args.copy_calibration:
        n = 256 << 20
        a, b = B.DeviceBuffer(n), B.DeviceBuffer(n)
        B.check(B.lib().lcu_memset(a.ptr, 1, n, None))
        B.check(B.lib().lcu_d2d(b.ptr, a.ptr, n, None))
        B.check(B.lib().lcu_sync(None))
        extra["copy_calibration_bytes"] = n
        a.free()
        b.free()
    if not args.no_extra:
        stream = None
        extra["gemv"] = gemv_leg(P, stream)
        extra["prefill_gemm"] = gemm_leg(P, stream)
    cpu = None if args.no_cpu else cpu_baseline_leg(cfg)
    props = B.device_props(0)
    line = {
        "metric": "decode tok/s (%s, 1 GPU)" % ("7B fp16" if args.workload == "llama7b_fp16" else "30B int8"),
        "value": round(dec["tok_s"], 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dec["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if cfg["q_type"] == 0 else "u8 weights, f16 activations", "data": "synthetic",
        "config": {"workload": "%s: %d-token random prompt, then batch-1 greedy decode, context 2048, temperature 0.8"
                               % (args.workload, PROMPT), "device": props.name.decode(errors="replace")},
        # achieved / frac: the whole decode step (every byte a step must read over the measured step
        # time), the quantity the decode target is stated in; kernel_*: its dominant kernel alone
        "roofline": {"bound": "hbm", "achieved": extra["decode_hbm_gb_s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": extra["decode_frac_of_hbm_roofline"], "traffic": MEASURED_TRAFFIC.get(args.workload),
                     "scope": "whole decode step: weights + KV cache bytes of one step / measured step time",
                     "kernel": "decode_ffn_up_kernel (W1,W3 GEMV + SiLU*mul), dim %d ffn %d" % (cfg["dim"], ffn),
                     "kernel_achieved": round(achieved, 1), "kernel_frac": round(achieved / HBM_PEAK_GBS, 4),
                     "bytes_per_launch": int(k_bytes), "us_per_launch": round(k_us, 3)},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
