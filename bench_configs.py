#!/usr/bin/env python3
"""Measures the other benchmark configurations on one MI355X (bench.py covers the headline one):

  C1  2-input in-place fp32 sum, 16,777,216 elements per buffer
  C2  8-input bf16 sum, 33,554,432 elements per buffer
  C3  datatype x op sweep, 4 inputs, 1 KiB ... 1 GiB per buffer (x4 steps)
  C4  fusion: 256 bf16 tensors, counts log-uniform [2,048, 2,097,152], 256-byte aligned offsets, 8-input sum against
      7 peer fusion buffers: pack + reduce + unpack, and the fused single pass

  batch  C3's small sizes (1 KiB ... 4 MiB per buffer) as 64 independent jobs: 64 calls against one call of
         mi_ccl_comp_reduce_batch (one launch)
  types  every datatype x op at 512 MiB per buffer, 8 and 4 inputs
  align  buffers that disagree modulo 16 bytes: 8-input bf16 sum at 64 MiB per buffer with every input at its own
         alignment, and with only the output off; buffers on the 16-byte boundary but off the 128-byte lines (all of
         them, the output alone, the peers); the reference's tight fusion layout (alignment 1) of 400 even- and
         odd-sized tensors: pack, unpack and the fused reduce
  write  a reduce stored to several buffers, and one buffer written to several (the all-gather write side), at 64 MiB
         and 1 GiB per buffer
  copy   ccl_comp_copy at 64 MiB, 512 MiB and 3 GiB, and the bf16 <-> fp32 array converters at 2^28 elements

    python bench_configs.py [--out results/configs.json] [--skip c3,batch,types,align,write,copy] [--only c1,c4] [--c3-k 7]
                            [--set realign=0]

--only runs just the named sections (c1, c2, c3, batch, types, align, write, copy, c4, latency), --c3-k just the named sizes of
the sweep (size = 1 KiB x 4^k): what a profiler run of one kernel wants.

EVERY row is checked before it is timed: the first buffer set goes through the call once and the result is compared,
bit for bit, with the CPU oracle (oracle/, the checker -- it is never the thing measured) on the same inputs: whole
buffers up to 64 MiB, beyond that the first 16 MiB and the last 1 MiB of every buffer.  A row that fails the check ends
the run.  Writes a JSON file and prints a markdown table.  Bytes are algorithmic: (N + 1) x chunk for a reduce,
2 x payload for pack and unpack.  Buffers of 64 MiB rotate over several sets so that the 256 MB Infinity Cache cannot
hold them.
"""
import argparse
import json
import math
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
for p_ in (ROOT, os.path.join(ROOT, "tests")):
    if p_ not in sys.path:
        sys.path.insert(0, p_)


MARK = {"on": False, "buf": None, "segments": 0, "comp": None}


def timed(torch, fn, steps, warm):
    """Microseconds per call over `steps` back-to-back calls after `warm` untimed ones.  With --markers the timed calls
    sit between two marker launches of the library's probe kernels (a four-store write probe before, a one-store
    write probe after, on a 4 KiB buffer), so that a profiler's list of dispatches can be cut into the rows of the
    table: the n-th pair of markers encloses the n-th timed loop."""
    for i in range(warm):
        fn(i)
    if MARK["on"]:
        MARK["comp"].probe_bandwidth(MARK["comp"].PROBE_WRITE_FOUR, [MARK["buf"]], 4096)
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        fn(i)
    e1.record()
    if MARK["on"]:
        MARK["comp"].probe_bandwidth(MARK["comp"].PROBE_WRITE_ONE, [MARK["buf"]], 4096)
    MARK["segments"] += 1
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps * 1e3      # us


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default=os.path.join(ROOT, "results", "configs.json"))
    ap.add_argument("--skip", default="")
    ap.add_argument("--only", default="")
    ap.add_argument("--c3-k", default="", help="comma-separated exponents k of the C3 sizes 1 KiB x 4^k (default: all 11)")
    ap.add_argument("--set", action="append", default=[], metavar="NAME=VALUE", help="launch knob (mi_ccl_set_param)")
    ap.add_argument("--markers", action="store_true", help="enclose every timed loop in two marker launches (for profiler runs)")
    args = ap.parse_args()
    only = [x for x in args.only.split(",") if x]
    skip = [x for x in args.skip.split(",") if x]
    c3_k = [int(x) for x in args.c3_k.split(",") if x] or list(range(11))

    def want(section):
        return (section in only) if only else (section not in skip)
    import numpy as np
    import torch
    import oneccl_amd.comp as comp
    import oracle_lib as O          # the checker
    comp.lib()
    torch.cuda.set_device(0)
    for kv in args.set:
        k_, v_ = kv.split("=")
        comp.set_param(k_, int(v_))
    res = {}
    rows = []
    checked = [0]
    if args.markers:
        MARK.update(on=True, buf=torch.zeros(4096, dtype=torch.uint8, device="cuda"), comp=comp)
    seen_segments = [0]

    def add(name, us, byts, extra=""):
        gbs = byts / us / 1e3
        res[name] = dict(us=round(us, 2), GBps=round(gbs, 1), bytes=byts, pct_hbm_peak=round(gbs / 80.0, 2), checked=True,
                         timed_loops=list(range(seen_segments[0], MARK["segments"])))     # which timed loops belong to the row
        seen_segments[0] = MARK["segments"]
        rows.append(f"| {name} | {byts:,} | {us:,.1f} | {gbs:,.0f} | {gbs / 80.0:.1f} % | {extra} |")

    INT_VIEW = {1: torch.int8, 2: torch.int16, 4: torch.int32, 8: torch.int64}
    NP_UINT = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}

    def host_bits(t, lo, hi):
        """Elements [lo, hi) of a device tensor as unsigned integers of the element's width."""
        esz = t.element_size()
        return t[lo:hi].view(INT_VIEW[esz]).cpu().numpy().view(NP_UINT[esz])

    def ranges(count, esz):
        """Element ranges that are compared: everything up to 64 MiB, else the first 16 MiB and the last 1 MiB."""
        if count * esz <= (64 << 20):
            return [(0, count)]
        return [(0, (16 << 20) // esz), (count - (1 << 20) // esz, count)]

    def verify_reduce(what, dt, op, srcs, out_fn, count, keep=0, in_place_out=None):
        """Runs out = out_fn() once on the given inputs and compares it with the oracle.  srcs are device tensors (their
        contents are read BEFORE the call, so an in-place output is fine)."""
        esz = O.DTYPE_SIZE[dt]
        np_t = O.NP_STORAGE[dt]
        want = []
        for lo, hi in ranges(count, esz):
            host = [host_bits(s_, lo, hi).view(np_t) for s_ in srcs]
            want.append((lo, hi, O.reduce_n(host, dt, op, keep=keep, threads=16)))
        out = out_fn()
        torch.cuda.synchronize()
        for lo, hi, w in want:
            g = host_bits(out, lo, hi)
            if not (g == w.view(g.dtype)).all():
                sys.exit(f"CHECK FAILED: {what}: elements [{lo}, {hi}) differ from the oracle")
        checked[0] += 1

    # ---- C1
    if want("c1"):
        n1 = 16_777_216
        sets = [[torch.empty(n1, dtype=torch.float32, device="cuda").uniform_(-1, 1) for _ in range(2)] for _ in range(8)]

        def c1_once():
            comp.comp_reduce(comp.FLOAT32, comp.SUM, sets[0][1], n1, sets[0][0])
            return sets[0][0]
        verify_reduce("C1", O.FLOAT32, O.SUM, [sets[0][0], sets[0][1]], c1_once, n1)
        us = timed(torch, lambda i: comp.comp_reduce(comp.FLOAT32, comp.SUM, sets[i % 8][1], n1, sets[i % 8][0]), 64, 16)
        add("C1 fp32 sum, 2 inputs in place, 64 MiB", us, 3 * n1 * 4, f"8 rotating buffer sets; {comp.last_kernel()}")
        us = timed(torch, lambda i: comp.comp_reduce(comp.FLOAT32, comp.SUM, sets[0][1], n1, sets[0][0]), 64, 16)
        add("C1 same, one buffer set (Infinity Cache assisted)", us, 3 * n1 * 4, "")
        del sets
    # ---- C2
    if want("c2"):
        n2 = 33_554_432
        sets = [[torch.empty(n2, dtype=torch.bfloat16, device="cuda").normal_(0, 1) for _ in range(8)] for _ in range(6)]
        outs = [torch.empty_like(s[0]) for s in sets]

        def c2_once():
            comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, sets[0], outs[0], n2, lp_mode=comp.LP_KEEP_PRECISION)
            return outs[0]
        verify_reduce("C2", O.BFLOAT16, O.SUM, sets[0], c2_once, n2, keep=1)
        us = timed(torch, lambda i: comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, sets[i % 6], outs[i % 6], n2,
                                                      lp_mode=comp.LP_KEEP_PRECISION), 64, 16)
        add("C2 bf16 sum, 8 inputs, 64 MiB (fp32 acc, RNE once)", us, 9 * n2 * 2, f"6 rotating buffer sets; {comp.last_kernel()}")
        us = timed(torch, lambda i: comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, sets[0], outs[0], n2,
                                                      lp_mode=comp.LP_KEEP_PRECISION), 64, 16)
        add("C2 same, one buffer set (Infinity Cache assisted)", us, 9 * n2 * 2, "")
        del sets, outs

    c3_cases = [("int8 sum", comp.INT8, comp.SUM, torch.int8, 1), ("int32 sum", comp.INT32, comp.SUM, torch.int32, 4),
                ("int64 max", comp.INT64, comp.MAX, torch.int64, 8), ("fp16 sum", comp.FLOAT16, comp.SUM, torch.float16, 2),
                ("fp32 min", comp.FLOAT32, comp.MIN, torch.float32, 4), ("fp64 prod", comp.FLOAT64, comp.PROD, torch.float64, 8)]

    def maker(tdt, op, cnt):
        if tdt.is_floating_point:
            lo, hi = (0.9, 1.1) if op == comp.PROD else (-2.0, 2.0)
            return lambda: torch.empty(cnt, dtype=torch.float32, device="cuda").uniform_(lo, hi).to(tdt)
        info = torch.iinfo(tdt)
        return lambda: torch.randint(info.min, info.max, (cnt,), dtype=tdt, device="cuda")

    # ---- C3
    if want("c3"):
        for label, dt, op, tdt, esz in c3_cases:
            for k in c3_k:
                size = 1024 * 4 ** k
                cnt = size // esz
                nsets = max(1, min(8, (1 << 30) // (5 * size)))
                mk = maker(tdt, op, cnt)
                ss = [[mk() for _ in range(4)] for _ in range(nsets)]
                oo = [torch.empty_like(s[0]) for s in ss]

                def once():
                    comp.comp_reduce_n(dt, op, ss[0], oo[0], cnt)
                    return oo[0]
                verify_reduce(f"C3 {label} {size >> 10} KiB", dt, op, ss[0], once, cnt)
                steps = 200 if size <= (1 << 22) else 30
                us = timed(torch, lambda i: comp.comp_reduce_n(dt, op, ss[i % nsets], oo[i % nsets], cnt), steps, 10)
                add(f"C3 {label}, 4 inputs, {size >> 10} KiB per buffer", us, 5 * size, f"{nsets} set(s)")
                del ss, oo
    # ---- C3's small sizes as 64 independent jobs: one call each against one batched call
    if want("batch"):
        for label, dt, op, tdt, esz in c3_cases:
            for k in range(7):
                size = 1024 * 4 ** k
                cnt = size // esz
                mk = maker(tdt, op, cnt)
                jobs_in = [[mk() for _ in range(4)] for _ in range(64)]
                jobs_out = [torch.empty_like(j[0]) for j in jobs_in]
                jobs = [(s_, o_, cnt) for s_, o_ in zip(jobs_in, jobs_out)]
                for j in (0, 63):
                    def once(j=j):
                        jobs_out[j].zero_()
                        comp.comp_reduce_batch(dt, op, jobs)
                        return jobs_out[j]
                    verify_reduce(f"batch {label} {size >> 10} KiB job {j}", dt, op, jobs_in[j], once, cnt)

                def calls(i):
                    for s_, o_, c_ in jobs:
                        comp.comp_reduce_n(dt, op, s_, o_, c_)
                us_calls = timed(torch, calls, 10, 3)
                table = comp.BatchJobs(jobs)      # pointer tables built once, as a native caller would hold them
                us_batch = timed(torch, lambda i: table.reduce(dt, op), 100, 10)
                add(f"batch {label}, 64 jobs x 4 inputs x {size >> 10} KiB, one launch", us_batch, 5 * size * 64,
                    f"{us_batch / 64:.2f} us per job; as 64 calls through this binding {us_calls / 64:.2f} us per job")
                del table
                del jobs_in, jobs_out, jobs
    # ---- every datatype x op at 512 MiB per buffer, 8 and 4 inputs: is any of them bound by arithmetic?
    if want("types"):
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
                    def once():
                        comp.comp_reduce_n(dt, op, ss, oo, cnt, lp_mode=lp or comp.LP_PAIRWISE)
                        return oo
                    verify_reduce(f"types {label} {opn} n={nin}", dt, op, ss, once, cnt, keep=1 if lp == comp.LP_KEEP_PRECISION else 0)
                    us = timed(torch, lambda i: comp.comp_reduce_n(dt, op, ss, oo, cnt, lp_mode=lp or comp.LP_PAIRWISE), 10, 3)
                    gbs = (nin + 1) * size / us / 1e3
                    res[f"types {label} {opn} n={nin}"] = dict(us=round(us, 2), GBps=round(gbs, 1), bytes=(nin + 1) * size, checked=True)
                    cells.append(f"{opn} {gbs:,.0f}")
                rows.append(f"| {label}, {nin} inputs, 512 MiB per buffer | {(nin + 1) * size:,} | | {' / '.join(cells)} | | GB/s per op |")
                del ss, oo

    def verify_fusion(what, plan, counts, align, tens, peers, fb_after_pack=None, outs_after=None, mode="fused"):
        """pack: fusion buffer payload == tensors; unpack / fused: every tensor against the oracle's reduce of the
        tensor with the peers' slices (the oracle's pack -> reduce -> unpack gives the same, tensor by tensor)."""
        offs, total = O.fusion_offsets(counts, 2, align)
        if mode == "pack":
            fb = fb_after_pack.view(torch.int16).cpu().numpy().view(np.uint16)
            for i, c in enumerate(counts):
                o = int(offs[i]) // 2 if int(offs[i]) % 2 == 0 else None
                t = tens[i].view(torch.int16).cpu().numpy().view(np.uint16)
                got = fb[o:o + c] if o is not None else fb.view(np.uint8)[int(offs[i]):int(offs[i]) + 2 * c].copy().view(np.uint16)
                if not (got == t).all():
                    sys.exit(f"CHECK FAILED: {what}: tensor {i} is not where the layout puts it")
        else:
            hp = [p.view(torch.int16).cpu().numpy().view(np.uint16) for p in peers]
            for i, c in enumerate(counts):
                b0 = int(offs[i])
                t = tens[i].view(torch.int16).cpu().numpy().view(np.uint16)
                sl = [p.view(np.uint8)[b0:b0 + 2 * c].copy().view(np.uint16) for p in hp]
                want = O.reduce_n([t] + sl, O.BFLOAT16, O.SUM, keep=1) if peers else t
                got = outs_after[i].view(torch.int16).cpu().numpy().view(np.uint16)
                if not (got == want).all():
                    sys.exit(f"CHECK FAILED: {what}: tensor {i} of {c} elements differs from the oracle")
        checked[0] += 1

    # ---- buffers at different offsets from a 16-byte boundary
    if want("align"):
        na = 33_554_432
        sets = [[torch.empty(na + 64, dtype=torch.bfloat16, device="cuda").normal_(0, 1) for _ in range(9)] for _ in range(6)]
        for label, shifts in (("all aligned", [0] * 9), ("every input at its own alignment", [1, 2, 3, 4, 5, 6, 7, 0, 0]),
                              ("only the output off by 6 bytes", [0] * 8 + [3]),
                              ("every buffer 16 bytes past a 128-byte line", [8] * 9), ("every buffer 2 bytes past a line", [1] * 9),
                              ("only the output 16 bytes past a line", [0] * 8 + [8]), ("the peers 16 bytes past a line", [0] + [8] * 7 + [0])):
            ptrs = [[t.data_ptr() + 2 * sh for t, sh in zip(s_, shifts)] for s_ in sets]

            def once():
                comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, ptrs[0][:8], ptrs[0][8], na, lp_mode=comp.LP_KEEP_PRECISION)
                return sets[0][8][shifts[8]:shifts[8] + na]
            verify_reduce(f"align {label}", O.BFLOAT16, O.SUM, [t[sh:sh + na] for t, sh in zip(sets[0][:8], shifts)], once, na, keep=1)
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
            outs = [torch.zeros_like(t) for t in tens]
            fb = torch.zeros(nelem, dtype=torch.bfloat16, device="cuda")
            peers = [torch.empty(nelem, dtype=torch.bfloat16, device="cuda").normal_(0, 0.02) for _ in range(7)]
            plan.pack(tens, fb)
            torch.cuda.synchronize()
            verify_fusion(f"align pack {label}", plan, counts, 1, tens, None, fb_after_pack=fb, mode="pack")
            us = timed(torch, lambda i: plan.pack(tens, fb), 20, 5)
            add(f"align: pack, 400 {label}-sized bf16 tensors, tight layout, payload {payload:,} B", us, 2 * payload)
            plan.unpack(fb, outs)
            torch.cuda.synchronize()
            verify_fusion(f"align unpack {label}", plan, counts, 1, tens, [], outs_after=outs)
            us = timed(torch, lambda i: plan.unpack(fb, outs), 20, 5)
            add(f"align: unpack, {label}-sized", us, 2 * payload)
            plan.reduce(comp.SUM, tens, peers, outs, lp_mode=comp.LP_KEEP_PRECISION)
            torch.cuda.synchronize()
            verify_fusion(f"align fused {label}", plan, counts, 1, tens, peers, outs_after=outs)
            us = timed(torch, lambda i: plan.reduce(comp.SUM, tens, peers, outs, lp_mode=comp.LP_KEEP_PRECISION), 20, 5)
            add(f"align: fused reduce against 7 peers, {label}-sized", us, 9 * payload, comp.last_kernel())
            plan.close()
            del tens, outs, fb, peers
    # ---- several destinations (the write side: a reduce stored to M buffers, one buffer written to M)
    if want("write"):
        for n, m, mib in ((8, 8, 1024), (8, 2, 1024), (4, 4, 1024), (2, 2, 1024), (1, 7, 1024), (1, 2, 1024), (8, 8, 64), (2, 2, 64), (1, 7, 64), (1, 2, 64)):
            cnt = (mib << 20) // 2
            nsets = 1 if mib >= 512 else max(1, min(4, (3 << 30) // ((n + m) * (mib << 20))))
            srcs = [[torch.empty(cnt, dtype=torch.bfloat16, device="cuda").normal_(0, 1) for _ in range(n)] for _ in range(nsets)]
            dsts = [[torch.zeros(cnt, dtype=torch.bfloat16, device="cuda") for _ in range(m)] for _ in range(nsets)]
            lp = comp.LP_KEEP_PRECISION if n > 1 else comp.LP_PAIRWISE
            for k in range(m):
                def once(k=k):
                    for d in dsts[0]:
                        d.zero_()
                    comp.comp_reduce_write_n(comp.BFLOAT16, comp.SUM, srcs[0], dsts[0], cnt, lp_mode=lp)
                    return dsts[0][k]
                if k in (0, m - 1):
                    verify_reduce(f"write {n}->{m} {mib} MiB, destination {k}", O.BFLOAT16, O.SUM, srcs[0], once, cnt, keep=1 if n > 1 else 0)
            us = timed(torch, lambda i: comp.comp_reduce_write_n(comp.BFLOAT16, comp.SUM, srcs[i % nsets], dsts[i % nsets], cnt, lp_mode=lp),
                       10 if mib >= 512 else 40, 3)
            add(f"write: bf16 sum of {n} input{'s' if n > 1 else ''} stored to {m} buffers, {mib} MiB each", us, (n + m) * cnt * 2,
                f"{nsets} set(s); {comp.last_kernel()}")
            del srcs, dsts
    # ---- copies and converters
    if want("copy"):
        for mib in (64, 512, 3072):
            nb = mib << 20
            nsets = 4 if mib == 64 else 1
            src = [torch.empty(nb, dtype=torch.uint8, device="cuda").random_(0, 255) for _ in range(nsets)]
            dst = [torch.zeros(nb, dtype=torch.uint8, device="cuda") for _ in range(nsets)]
            comp.comp_copy(src[0], dst[0], nb, use_nontemporal=True)
            torch.cuda.synchronize()
            for lo in range(0, nb, 1 << 30):
                if not torch.equal(src[0][lo:lo + (1 << 30)], dst[0][lo:lo + (1 << 30)]):
                    sys.exit(f"CHECK FAILED: copy of {mib} MiB")
            checked[0] += 1
            us = timed(torch, lambda i: comp.comp_copy(src[i % nsets], dst[i % nsets], nb, use_nontemporal=True), 20, 5)
            add(f"copy, {mib} MiB", us, 2 * nb, f"{nsets} set(s)")
            del src, dst
        nc = 1 << 28
        f32 = torch.empty(nc, dtype=torch.float32, device="cuda").normal_()
        b16 = torch.zeros(nc, dtype=torch.bfloat16, device="cuda")
        f16 = torch.zeros(nc, dtype=torch.float16, device="cuda")
        L = O.lib()

        def check_cvt(what, src_t, dst_t, orc, extra=()):
            for lo, hi in ranges(nc, 4):
                a = host_bits(src_t, lo, hi)
                want = np.empty(hi - lo, NP_UINT[dst_t.element_size()])
                getattr(L, orc)(a.ctypes.data, want.ctypes.data, hi - lo, *extra)
                if not (host_bits(dst_t, lo, hi) == want).all():
                    sys.exit(f"CHECK FAILED: {what}")
            checked[0] += 1
        comp.convert_fp32_to_bf16_arrays(f32, b16, nc)
        torch.cuda.synchronize()
        check_cvt("fp32 -> bf16", f32, b16, "orc_convert_fp32_to_bf16_arrays", (2,))
        us = timed(torch, lambda i: comp.convert_fp32_to_bf16_arrays(f32, b16, nc), 20, 5)
        add("convert fp32 -> bf16 (round to nearest even), 2^28 elements", us, 6 * nc)
        f32b = torch.zeros_like(f32)
        comp.convert_bf16_to_fp32_arrays(b16, f32b, nc)
        torch.cuda.synchronize()
        check_cvt("bf16 -> fp32", b16, f32b, "orc_convert_bf16_to_fp32_arrays", (2,))
        us = timed(torch, lambda i: comp.convert_bf16_to_fp32_arrays(b16, f32b, nc), 20, 5)
        add("convert bf16 -> fp32, 2^28 elements", us, 6 * nc)
        comp.convert_fp32_to_fp16_arrays(f32, f16, nc)
        torch.cuda.synchronize()
        check_cvt("fp32 -> fp16", f32, f16, "orc_convert_fp32_to_fp16_arrays")
        us = timed(torch, lambda i: comp.convert_fp32_to_fp16_arrays(f32, f16, nc), 20, 5)
        add("convert fp32 -> fp16, 2^28 elements", us, 6 * nc)
        comp.convert_fp16_to_fp32_arrays(f16, f32b, nc)
        torch.cuda.synchronize()
        check_cvt("fp16 -> fp32", f16, f32b, "orc_convert_fp16_to_fp32_arrays")
        us = timed(torch, lambda i: comp.convert_fp16_to_fp32_arrays(f16, f32b, nc), 20, 5)
        add("convert fp16 -> fp32, 2^28 elements", us, 6 * nc)
        del f16, f32, f32b, b16
    # ---- C4
    if want("c4"):
        rng = np.random.default_rng(4)
        counts = [int(round(math.exp(rng.uniform(math.log(2048), math.log(2_097_152))))) for _ in range(256)]
        payload = sum(counts) * 2
        plan = comp.FusionPlan(counts, comp.BFLOAT16, 256)
        nelem = plan.nbytes // 2
        tens = [torch.empty(c, dtype=torch.bfloat16, device="cuda").normal_(0, 0.02) for c in counts]
        outs = [torch.zeros_like(t) for t in tens]
        fb = torch.zeros(nelem, dtype=torch.bfloat16, device="cuda")
        peers = [torch.empty(nelem, dtype=torch.bfloat16, device="cuda").normal_(0, 0.02) for _ in range(7)]
        plan.pack(tens, fb)
        torch.cuda.synchronize()
        verify_fusion("C4 pack", plan, counts, 256, tens, None, fb_after_pack=fb, mode="pack")
        us_pack = timed(torch, lambda i: plan.pack(tens, fb), 50, 10)
        fb2 = torch.empty_like(fb)

        def c4_reduce_once():
            comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, [fb] + peers, fb2, nelem, lp_mode=comp.LP_KEEP_PRECISION)
            return fb2
        verify_reduce("C4 reduce over the fusion buffer", O.BFLOAT16, O.SUM, [fb] + peers, c4_reduce_once, nelem, keep=1)
        us_red = timed(torch, lambda i: comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, [fb] + peers, fb2, nelem,
                                                          lp_mode=comp.LP_KEEP_PRECISION), 50, 10)
        plan.unpack(fb2, outs)
        torch.cuda.synchronize()
        verify_fusion("C4 pack + reduce + unpack", plan, counts, 256, tens, peers, outs_after=outs)
        us_unpack = timed(torch, lambda i: plan.unpack(fb2, outs), 50, 10)

        def three(i):
            plan.pack(tens, fb)
            comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, [fb] + peers, fb, nelem, lp_mode=comp.LP_KEEP_PRECISION)
            plan.unpack(fb, outs)
        for o_ in outs:
            o_.zero_()
        three(0)
        torch.cuda.synchronize()
        verify_fusion("C4 three launches", plan, counts, 256, tens, peers, outs_after=outs)
        us_three = timed(torch, three, 50, 10)
        for o_ in outs:
            o_.zero_()
        plan.reduce(comp.SUM, tens, peers, outs, lp_mode=comp.LP_KEEP_PRECISION)
        torch.cuda.synchronize()
        verify_fusion("C4 fused", plan, counts, 256, tens, peers, outs_after=outs)
        fused_kernel = comp.last_kernel()
        us_fused = timed(torch, lambda i: plan.reduce(comp.SUM, tens, peers, outs, lp_mode=comp.LP_KEEP_PRECISION), 50, 10)
        add(f"C4 pack, 256 tensors, payload {payload:,} B", us_pack, 2 * payload)
        add("C4 8-input reduce over the fusion buffer", us_red, 9 * payload)
        add("C4 unpack", us_unpack, 2 * payload)
        add("C4 pack + reduce + unpack (3 launches)", us_three, 13 * payload)
        add("C4 fused single pass (tensors + 7 peers -> tensors)", us_fused, 9 * payload,
            f"{us_three / us_fused:.2f}x faster than the 3-step sequence; {fused_kernel}")
        plan.close()

    # small-message latency from C++ (no Python in the loop); the program checks its own results
    lat = os.path.join(ROOT, "tests", "cpp", "bench_latency")
    lat_lines = []
    if want("latency") and os.path.exists(lat):
        import subprocess
        pr = subprocess.run([lat], capture_output=True, text=True, timeout=300)
        if pr.returncode != 0:
            sys.exit("CHECK FAILED: tests/cpp/bench_latency: " + pr.stdout[-500:])
        lat_lines = pr.stdout.strip().splitlines()
        res["latency_cpp"] = lat_lines

    res["rows_checked_against_the_oracle"] = checked[0]
    os.makedirs(os.path.dirname(args.out), exist_ok=True)
    with open(args.out, "w") as f:
        json.dump(res, f, indent=1)
    print(f"Every row below was checked bit for bit against the CPU oracle before it was timed ({checked[0]} checks).\n")
    print("| configuration | algorithmic bytes | us per call | GB/s | of 8 TB/s | note |")
    print("|---|---|---|---|---|---|")
    print("\n".join(rows))
    if lat_lines:
        print("\nSmall messages issued from C++ (tests/cpp/bench_latency, 4-input int32 sum; results checked in closed form):\n")
        print("\n".join("    " + l for l in lat_lines))


if __name__ == "__main__":
    main()
