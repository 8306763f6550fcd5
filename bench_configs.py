#!/usr/bin/env python3
"""Measures the other benchmark configurations on one MI355X (bench.py covers the headline one):

  C1  2-input in-place fp32 sum, 16,777,216 elements per buffer
  C2  8-input bf16 sum, 33,554,432 elements per buffer
  C3  datatype x op sweep, 4 inputs, 1 KiB ... 1 GiB per buffer (x4 steps)
  C4  fusion: 256 bf16 tensors, counts log-uniform [2,048, 2,097,152], 256-byte aligned offsets, 8-input sum against
      7 peer fusion buffers: pack + reduce + unpack, and the fused single pass

  types  every datatype x op at 512 MiB per buffer, 8 and 4 inputs
  align  buffers that disagree modulo 16 bytes: 8-input bf16 sum at 64 MiB per buffer with every input at its own
         alignment, and with only the output off; the reference's tight fusion layout (alignment 1) of 400 odd-sized
         tensors: pack, unpack and the fused reduce

  copy   ccl_comp_copy at 64 MiB, 512 MiB and 3 GiB, and the bf16 <-> fp32 array converters at 2^28 elements

    python bench_configs.py [--out results/configs.json] [--skip c3,types,align,copy]

Writes a JSON file and prints a markdown table.  Bytes are algorithmic: (N + 1) x chunk for a reduce, 2 x payload
for pack and unpack.  Buffers of 64 MiB rotate over several sets so that the 256 MB Infinity Cache cannot hold them.
"""
import argparse
import json
import math
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


def timed(torch, fn, steps, warm):
    for i in range(warm):
        fn(i)
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps * 1e3      # us


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default=os.path.join(ROOT, "results", "configs.json"))
    ap.add_argument("--skip", default="")
    args = ap.parse_args()
    import numpy as np
    import torch
    import oneccl_amd.comp as comp
    comp.lib()
    torch.cuda.set_device(0)
    res = {}
    rows = []

    def add(name, us, byts, extra=""):
        gbs = byts / us / 1e3
        res[name] = dict(us=round(us, 2), GBps=round(gbs, 1), bytes=byts, pct_hbm_peak=round(gbs / 80.0, 2))
        rows.append(f"| {name} | {byts:,} | {us:,.1f} | {gbs:,.0f} | {gbs / 80.0:.1f} % | {extra} |")

    # ---- C1
    n1 = 16_777_216
    sets = [[torch.empty(n1, dtype=torch.float32, device="cuda").uniform_(-1, 1) for _ in range(2)] for _ in range(8)]
    us = timed(torch, lambda i: comp.comp_reduce(comp.FLOAT32, comp.SUM, sets[i % 8][1], n1, sets[i % 8][0]), 64, 16)
    add("C1 fp32 sum, 2 inputs in place, 64 MiB", us, 3 * n1 * 4, "8 rotating buffer sets")
    del sets
    # ---- C2
    n2 = 33_554_432
    sets = [[torch.empty(n2, dtype=torch.bfloat16, device="cuda").normal_(0, 1) for _ in range(8)] for _ in range(6)]
    outs = [torch.empty_like(s[0]) for s in sets]
    us = timed(torch, lambda i: comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, sets[i % 6], outs[i % 6], n2,
                                                  lp_mode=comp.LP_KEEP_PRECISION), 64, 16)
    add("C2 bf16 sum, 8 inputs, 64 MiB (fp32 acc, RNE once)", us, 9 * n2 * 2, "6 rotating buffer sets")
    us = timed(torch, lambda i: comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, sets[0], outs[0], n2,
                                                  lp_mode=comp.LP_KEEP_PRECISION), 64, 16)
    add("C2 same, one buffer set (Infinity Cache assisted)", us, 9 * n2 * 2, "")
    del sets, outs
    # ---- C3
    if "c3" not in args.skip:
        cases = [("int8 sum", comp.INT8, comp.SUM, torch.int8, 1), ("int32 sum", comp.INT32, comp.SUM, torch.int32, 4),
                 ("int64 max", comp.INT64, comp.MAX, torch.int64, 8), ("fp16 sum", comp.FLOAT16, comp.SUM, torch.float16, 2),
                 ("fp32 min", comp.FLOAT32, comp.MIN, torch.float32, 4), ("fp64 prod", comp.FLOAT64, comp.PROD, torch.float64, 8)]
        for label, dt, op, tdt, esz in cases:
            for k in range(11):
                size = 1024 * 4 ** k
                cnt = size // esz
                nsets = max(1, min(8, (1 << 30) // (5 * size)))
                if tdt.is_floating_point:
                    lo, hi = (0.9, 1.1) if op == comp.PROD else (-2.0, 2.0)
                    mk = lambda: torch.empty(cnt, dtype=torch.float32, device="cuda").uniform_(lo, hi).to(tdt)
                else:
                    info = torch.iinfo(tdt)
                    mk = lambda: torch.randint(info.min, info.max, (cnt,), dtype=tdt, device="cuda")
                ss = [[mk() for _ in range(4)] for _ in range(nsets)]
                oo = [torch.empty_like(s[0]) for s in ss]
                steps = 200 if size <= (1 << 22) else 30
                us = timed(torch, lambda i: comp.comp_reduce_n(dt, op, ss[i % nsets], oo[i % nsets], cnt), steps, 10)
                add(f"C3 {label}, 4 inputs, {size >> 10} KiB per buffer", us, 5 * size, f"{nsets} set(s)")
                del ss, oo
    # ---- every datatype x op at 512 MiB per buffer, 8 and 4 inputs: is any of them bound by arithmetic?
    if "types" not in args.skip:
        size = 512 << 20
        tcases = [("int8", comp.INT8, torch.int8, None), ("int16", comp.INT16, torch.int16, None),
                  ("int32", comp.INT32, torch.int32, None), ("int64", comp.INT64, torch.int64, None),
                  ("fp16", comp.FLOAT16, torch.float16, None), ("fp32", comp.FLOAT32, torch.float32, None),
                  ("fp64", comp.FLOAT64, torch.float64, None),
                  ("bf16 pairwise", comp.BFLOAT16, torch.bfloat16, comp.LP_PAIRWISE),
                  ("bf16 fp32-acc", comp.BFLOAT16, torch.bfloat16, comp.LP_KEEP_PRECISION)]
        for nin in (8, 4):
            for label, dt, tdt, lp in tcases:
                cnt = size // torch.empty(0, dtype=tdt).element_size()
                if tdt.is_floating_point:
                    ss = [torch.empty(cnt, dtype=tdt, device="cuda").uniform_(0.9, 1.1) for _ in range(nin)]
                else:
                    ss = [torch.randint(-100, 100, (cnt,), dtype=tdt, device="cuda") for _ in range(nin)]
                oo = torch.empty_like(ss[0])
                cells = []
                for op, opn in ((comp.SUM, "sum"), (comp.PROD, "prod"), (comp.MIN, "min"), (comp.MAX, "max")):
                    us = timed(torch, lambda i: comp.comp_reduce_n(dt, op, ss, oo, cnt, lp_mode=lp or comp.LP_PAIRWISE), 10, 3)
                    gbs = (nin + 1) * size / us / 1e3
                    res[f"types {label} {opn} n={nin}"] = dict(us=round(us, 2), GBps=round(gbs, 1), bytes=(nin + 1) * size)
                    cells.append(f"{opn} {gbs:,.0f}")
                rows.append(f"| {label}, {nin} inputs, 512 MiB per buffer | {(nin + 1) * size:,} | | {' / '.join(cells)} | | GB/s per op |")
                del ss, oo
    # ---- buffers at different offsets from a 16-byte boundary
    if "align" not in args.skip:
        na = 33_554_432
        sets = [[torch.empty(na + 64, dtype=torch.bfloat16, device="cuda").normal_(0, 1) for _ in range(9)] for _ in range(6)]
        for label, shifts in (("all aligned", [0] * 9), ("every input at its own alignment", [1, 2, 3, 4, 5, 6, 7, 0, 0]),
                              ("only the output off by 6 bytes", [0] * 8 + [3])):
            ptrs = [[t.data_ptr() + 2 * sh for t, sh in zip(s_, shifts)] for s_ in sets]
            us = timed(torch, lambda i: comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, ptrs[i % 6][:8], ptrs[i % 6][8], na,
                                                          lp_mode=comp.LP_KEEP_PRECISION), 64, 16)
            add(f"align: bf16 sum, 8 inputs, 64 MiB, {label}", us, 9 * na * 2, "6 rotating buffer sets")
        del sets
        rng = np.random.default_rng(1)
        for label, odd in (("even", 0), ("odd", 1)):
            counts = [int(c) // 8 * 8 + odd for c in np.exp(rng.uniform(np.log(2048), np.log(4 << 20), 400))]
            payload = sum(counts) * 2
            plan = comp.FusionPlan(counts, comp.BFLOAT16, 1)
            nelem = plan.nbytes // 2 + 8
            tens = [torch.empty(c, dtype=torch.bfloat16, device="cuda").normal_(0, 0.02) for c in counts]
            outs = [torch.empty_like(t) for t in tens]
            fb = torch.empty(nelem, dtype=torch.bfloat16, device="cuda")
            peers = [torch.empty(nelem, dtype=torch.bfloat16, device="cuda").normal_(0, 0.02) for _ in range(7)]
            us = timed(torch, lambda i: plan.pack(tens, fb), 20, 5)
            add(f"align: pack, 400 {label}-sized bf16 tensors, tight layout, payload {payload:,} B", us, 2 * payload)
            us = timed(torch, lambda i: plan.unpack(fb, outs), 20, 5)
            add(f"align: unpack, {label}-sized", us, 2 * payload)
            us = timed(torch, lambda i: plan.reduce(comp.SUM, tens, peers, outs, lp_mode=comp.LP_KEEP_PRECISION), 20, 5)
            add(f"align: fused reduce against 7 peers, {label}-sized", us, 9 * payload)
            plan.close()
            del tens, outs, fb, peers
    # ---- copies and converters
    if "copy" not in args.skip:
        for mib in (64, 512, 3072):
            nb = mib << 20
            nsets = 4 if mib == 64 else 1
            src = [torch.empty(nb, dtype=torch.uint8, device="cuda").random_(0, 255) for _ in range(nsets)]
            dst = [torch.empty(nb, dtype=torch.uint8, device="cuda") for _ in range(nsets)]
            us = timed(torch, lambda i: comp.comp_copy(src[i % nsets], dst[i % nsets], nb, use_nontemporal=True), 20, 5)
            add(f"copy, {mib} MiB", us, 2 * nb, f"{nsets} set(s)")
            del src, dst
        nc = 1 << 28
        f32 = torch.empty(nc, dtype=torch.float32, device="cuda").normal_()
        b16 = torch.empty(nc, dtype=torch.bfloat16, device="cuda")
        us = timed(torch, lambda i: comp.convert_fp32_to_bf16_arrays(f32, b16, nc), 20, 5)
        add("convert fp32 -> bf16 (round to nearest even), 2^28 elements", us, 6 * nc)
        us = timed(torch, lambda i: comp.convert_bf16_to_fp32_arrays(b16, f32, nc), 20, 5)
        add("convert bf16 -> fp32, 2^28 elements", us, 6 * nc)
        f16 = torch.empty(nc, dtype=torch.float16, device="cuda")
        us = timed(torch, lambda i: comp.convert_fp32_to_fp16_arrays(f32, f16, nc), 20, 5)
        add("convert fp32 -> fp16, 2^28 elements", us, 6 * nc)
        us = timed(torch, lambda i: comp.convert_fp16_to_fp32_arrays(f16, f32, nc), 20, 5)
        add("convert fp16 -> fp32, 2^28 elements", us, 6 * nc)
        del f16
        del f32, b16
    # ---- C4
    rng = np.random.default_rng(4)
    counts = [int(round(math.exp(rng.uniform(math.log(2048), math.log(2_097_152))))) for _ in range(256)]
    payload = sum(counts) * 2
    plan = comp.FusionPlan(counts, comp.BFLOAT16, 256)
    nelem = plan.nbytes // 2
    tens = [torch.empty(c, dtype=torch.bfloat16, device="cuda").normal_(0, 0.02) for c in counts]
    outs = [torch.empty_like(t) for t in tens]
    fb = torch.empty(nelem, dtype=torch.bfloat16, device="cuda")
    peers = [torch.empty(nelem, dtype=torch.bfloat16, device="cuda").normal_(0, 0.02) for _ in range(7)]
    us_pack = timed(torch, lambda i: plan.pack(tens, fb), 50, 10)
    us_red = timed(torch, lambda i: comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, [fb] + peers, fb, nelem,
                                                      lp_mode=comp.LP_KEEP_PRECISION), 50, 10)
    us_unpack = timed(torch, lambda i: plan.unpack(fb, outs), 50, 10)

    def three(i):
        plan.pack(tens, fb)
        comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, [fb] + peers, fb, nelem, lp_mode=comp.LP_KEEP_PRECISION)
        plan.unpack(fb, outs)
    us_three = timed(torch, three, 50, 10)
    us_fused = timed(torch, lambda i: plan.reduce(comp.SUM, tens, peers, outs, lp_mode=comp.LP_KEEP_PRECISION), 50, 10)
    add(f"C4 pack, 256 tensors, payload {payload:,} B", us_pack, 2 * payload)
    add("C4 8-input reduce over the fusion buffer", us_red, 9 * payload)
    add("C4 unpack", us_unpack, 2 * payload)
    add("C4 pack + reduce + unpack (3 launches)", us_three, 13 * payload)
    add("C4 fused single pass (tensors + 7 peers -> tensors)", us_fused, 9 * payload,
        f"{us_three / us_fused:.2f}x faster than the 3-step sequence")
    plan.close()

    # small-message latency from C++ (no Python in the loop)
    lat = os.path.join(ROOT, "tests", "cpp", "bench_latency")
    lat_lines = []
    if os.path.exists(lat):
        import subprocess
        lat_lines = subprocess.run([lat], capture_output=True, text=True, timeout=120).stdout.strip().splitlines()
        res["latency_cpp"] = lat_lines

    os.makedirs(os.path.dirname(args.out), exist_ok=True)
    with open(args.out, "w") as f:
        json.dump(res, f, indent=1)
    print("| configuration | algorithmic bytes | us per call | GB/s | of 8 TB/s | note |")
    print("|---|---|---|---|---|---|")
    print("\n".join(rows))
    if lat_lines:
        print("\nSmall messages issued from C++ (tests/cpp/bench_latency, 4-input int32 sum):\n")
        print("\n".join("    " + l for l in lat_lines))


if __name__ == "__main__":
    main()
