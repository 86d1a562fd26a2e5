#!/usr/bin/env python3
"""Benchmark of the block-causal attention path on one MI355X.

One step = one forward + backward of the cosmos3-shape attention call (bf16, B4
H64 Hkv8 D128, S = 4352 prefix + 50 action tokens, seeded synthetic inputs)
through the C ABI.  ``value`` is TFLOP/s on unmasked FLOPs only
(``14 * D * H * pairs`` per step: 4 for the forward's two products, 10 for the
backward's five), inputs resident in HBM.  Every part of the step is bracketed
by HIP events on the launch stream inside the timed region, which gives the
per-kernel durations behind ``roofline``.  The pi0.5 denoise attention (18
prefix calls + 180 cached-suffix calls at B=8) is timed after it and reported
under ``denoise``.  ``cpu_baseline`` is the eager CPU oracle on a bounded slice
of the same workload.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-denoise]
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0


# HBM bytes per launch (fetched + written) of the kernels of the default workload, from two
# counter runs (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE; KiB per dispatch), each scaled by what
# the same counter reads for a plain 1 GiB device copy (FETCH_SIZE reads half the bytes: factor 2.0;
# WRITE_SIZE: factor 1.0).  Other workloads have no such measurement and report null.
HBM_TRAFFIC_BYTES = {
    ("c5", "fwd"): int((286503.7 * 2.0 + 286134.8) * 1024),
    ("c5", "bwd_dq"): int((437434.9 * 2.0 + 281728.0) * 1024),
    ("c5", "bwd_dkv"): int((675657.6 * 2.0 + 70432.0) * 1024),
}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-denoise", action="store_true", help="skip the pi0.5 denoise leg")
    ap.add_argument("--no-others", action="store_true", help="skip the C3 / C4 steps reported beside the headline")
    ap.add_argument("--serial", action="store_true",
                    help="keep the backward's two big kernels on one stream (for per-kernel profiles)")
    ap.add_argument("--workload", default="c5", choices=["c3", "c4", "c5"])
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                    help="only run a plain device copy of MIB MiB a few times (reference for the "
                         "FETCH_SIZE / WRITE_SIZE counters) and exit")
    ap.add_argument("--rope-only", action="store_true",
                    help="only run the rotary-embedding leg and print its record (for profiles of that kernel)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        return 2
    if args.serial:
        os.environ["BCATTN_SERIAL_BACKWARD"] = "1"  # read by the library when it first runs a backward

    import torch

    from opentau_amd import flash_attn_hip as fa
    from opentau_amd.flash_attn_hip import _loader
    from opentau_amd.workloads import make_denoise_workload, make_workload

    if not fa.is_available():
        print(f"bench.py: HIP kernels unavailable: {fa.load_error()}", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.rope_only:
        print(json.dumps({"rope": bench_rope(torch, dev)}))
        return 0
    if args.copy_calibration:
        n = args.copy_calibration << 20
        src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes": n, "launches": 5}))
        return 0

    w = make_workload(args.workload)
    pairs = w.pairs()
    unit = w.D * w.H * pairs  # FLOPs per "GEMM unit" / 2
    ids = [t.to(dev) for t in w.block_ids()]
    q, k, v, go = (t.to(dev) for t in (w.q, w.k, w.v, w.d_out))
    grads = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
    out = torch.empty_like(q)
    ws_f = torch.empty(1 << 20, dtype=torch.uint8, device=dev)
    ws_b = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
    parts = ("fwd", "bwd_delta", "bwd_dq", "bwd_dkv")

    def step(ready=False):
        """One pass of the hot path: the forward call and the backward call, each with the pass
        over the ids that makes its tile summaries (a model would make them once for all its
        layers; here every step pays for them)."""
        _, lse = fa.forward_raw(q, k, v, *ids, w.scale, workspace=ws_f, summary_ready=ready, out=out)
        fa.backward_raw(go, q, k, v, out, lse, *ids, w.scale, workspace=ws_b, summary_ready=ready, grads=grads)
        return lse

    def step_by_kernel(ev):
        """The same work with the backward's kernels launched one call each, timed apart."""
        ev[0].record()
        _, lse = fa.forward_raw(q, k, v, *ids, w.scale, workspace=ws_f, summary_ready=True, out=out)
        ev[1].record()
        for n, st in enumerate((_loader.BWD_DELTA, _loader.BWD_DQ, _loader.BWD_DKV)):
            fa.backward_raw(go, q, k, v, out, lse, *ids, w.scale, stages=st, workspace=ws_b,
                            summary_ready=True, grads=grads)
            ev[2 + n].record()

    step()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    # per-kernel durations (HIP events on the stream of the launches), outside the timed region
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(args.steps)]
    for s in range(args.steps):
        step_by_kernel(events[s])
    torch.cuda.synchronize()
    part_ms = {p: sum(e[i].elapsed_time(e[i + 1]) for e in events) / args.steps for i, p in enumerate(parts)}
    tflops = 14 * unit / (ms_per_step * 1e-3) / 1e12

    # Unmasked FLOPs each kernel is credited with.  The backward's five products
    # (10*unit) are S, dP, dV, dK, dQ; S and dP are formed in both backward kernels
    # and are credited half to each, so the parts sum to the 14*unit of the step.
    credit = {"fwd": 4 * unit, "bwd_delta": 0, "bwd_dq": 4 * unit, "bwd_dkv": 6 * unit}
    dom = max(("fwd", "bwd_dq", "bwd_dkv"), key=lambda p: part_ms[p])
    achieved = credit[dom] / (part_ms[dom] * 1e-3) / 1e12
    roofline = {
        "bound": "mfma",
        "kernel": {"fwd": "fwd_mfma_kernel", "bwd_dq": "bwd_dq_kernel",
                   "bwd_dkv": "bwd_dkv_pair_kernel" if w.D == 128 else "bwd_dkv_kernel"}[dom],
        "achieved": round(achieved, 2),
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
        "traffic": HBM_TRAFFIC_BYTES.get((w.name, dom)),
        "kernel_ms": {p: round(part_ms[p], 4) for p in parts},
        "kernel_tflops": {p: round(credit[p] / (part_ms[p] * 1e-3) / 1e12, 2) for p in parts if credit[p]},
        "step_frac": round(tflops / PEAK_BF16_TFLOPS, 4),
    }

    result = {
        "metric": "block-causal attn fwd+bwd TFLOP/s on unmasked FLOPs (cosmos3 shape, 1 GPU)",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{w.name}: bf16 fwd+bwd B{w.B} H{w.H} Hkv{w.Hkv} D{w.D} S{w.S} "
                        f"({w.n_prefix} prefix in block 0, text valid {w.text_lo}..{w.text_hi}, "
                        f"{w.n_causal} causal, {w.n_action}-token action block)",
            "unmasked_pairs": pairs,
            "flops_per_step": 14 * unit,
            "pct_of_bf16_mfma_peak": round(100 * tflops / PEAK_BF16_TFLOPS, 2),
        },
        "roofline": roofline,
    }

    if not args.no_denoise:
        result["denoise"] = bench_denoise(torch, fa, make_denoise_workload, dev)
        if args.workload == "c5" and not args.no_others:
            result["other_workloads"] = {n: bench_step_only(torch, fa, make_workload, dev, n) for n in ("c3", "c4")}
            result["rope"] = bench_rope(torch, dev)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, make_workload, args.workload)
    print(json.dumps(result))
    return 0


def bench_step_only(torch, fa, make_workload, dev, name, steps=20, warmup=3):
    """Forward + backward step of another training configuration (the head_dim 256 shapes):
    the same measurement as the headline, without the per-kernel breakdown."""
    w = make_workload(name)
    ids = [t.to(dev) for t in w.block_ids()]
    q, k, v, go = (t.to(dev) for t in (w.q, w.k, w.v, w.d_out))
    grads = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
    out = torch.empty_like(q)
    ws_f = torch.empty(1 << 20, dtype=torch.uint8, device=dev)
    ws_b = torch.empty(64 << 20, dtype=torch.uint8, device=dev)

    def step():
        _, lse = fa.forward_raw(q, k, v, *ids, w.scale, workspace=ws_f, out=out)
        fa.backward_raw(go, q, k, v, out, lse, *ids, w.scale, workspace=ws_b, grads=grads)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    flops = 14 * w.D * w.H * w.pairs()
    return {
        "workload": f"{w.name}: bf16 fwd+bwd B{w.B} H{w.H} Hkv{w.Hkv} D{w.D} S{w.S}",
        "ms_per_step": round(ms, 4),
        "tflops": round(flops / (ms * 1e-3) / 1e12, 2),
        "pct_of_bf16_mfma_peak": round(100 * flops / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 2),
    }


def bench_rope(torch, dev, calls=50, warmup=5):
    """The rotary-embedding pass that feeds the attention call (queries and keys of one layer,
    in place, bf16), at the training shapes: an HBM-bound kernel, so GB/s on its algorithmic
    bytes (every element read once and written once, plus the positions) against the HBM peak."""
    from opentau_amd import rope

    out = {}
    shapes = {"c3": (32, 754, 8, 1, 256, False), "c5": (4, 4402, 64, 8, 128, False),
              "c5_cos_sin": (4, 4402, 64, 8, 128, True)}
    for name, (b, length, h, hkv, d, tables) in shapes.items():
        gen = torch.Generator(device="cpu").manual_seed(0)
        q = torch.randn(b, length, h, d, generator=gen).to(dev, torch.bfloat16)
        k = torch.randn(b, length, hkv, d, generator=gen).to(dev, torch.bfloat16)
        pos = torch.arange(length, dtype=torch.int32, device=dev)[None].expand(b, length).contiguous()
        kw = {}
        if tables:  # cosmos3's form: cos / sin tables from the backbone, arithmetic in bf16
            ang = pos[..., None].float() / (1e6 ** (torch.arange(d // 2, device=dev).float() * (2.0 / d)))
            emb = torch.cat([ang, ang], -1)
            kw = {"cos": emb.cos().to(torch.bfloat16), "sin": emb.sin().to(torch.bfloat16)}
        for _ in range(warmup):
            rope.rope_raw(q, k, pos, q_out=q, k_out=k, **kw)
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0.record()
        for _ in range(calls):
            rope.rope_raw(q, k, pos, q_out=q, k_out=k, **kw)
        t1.record()
        torch.cuda.synchronize()
        us = t0.elapsed_time(t1) * 1e3 / calls
        nbytes = 2 * 2 * (q.numel() + k.numel()) + (2 * 2 * b * length * d if tables else 4 * pos.numel())
        gbps = nbytes / (us * 1e-6) / 1e9
        out[name] = {
            "workload": f"rope of q and k in place{' from cos/sin tables' if tables else ''}, "
                        f"bf16 B{b} L{length} H{h} Hkv{hkv} D{d}",
            "us_per_call": round(us, 2),
            "algorithmic_bytes": nbytes,
            "gbps": round(gbps, 1),
            "hbm_frac": round(gbps / PEAK_HBM_GBPS, 4),
        }
    return out


def bench_denoise(torch, fa, make_denoise_workload, dev):
    """pi0.5 inference attention: 18 prefix calls, then 10 steps x 18 cached-suffix calls."""
    layers, steps = 18, 10
    dw = make_denoise_workload("c2", layers=layers, steps=steps, device=dev, distinct=36)
    w = dw.base
    npre, nact = w.n_prefix, w.n_action
    scale = w.scale
    pre_ids, suf_ids = dw.prefix_ids, dw.suffix_ids
    caches = [(kk[:, :npre], vv[:, :npre]) for (_, kk, vv) in dw.prefix]
    ws_p = torch.empty(1 << 20, dtype=torch.uint8, device=dev)
    ws_s = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
    out_p = torch.empty_like(dw.prefix[0][0])
    out_s = torch.empty_like(dw.suffix[0][0])

    def run(ev=None):
        if ev:
            ev[0].record()
        for li in range(layers):
            qq, kk, vv = dw.prefix[li]
            fa.forward_raw(qq, kk, vv, *pre_ids, scale, workspace=ws_p, summary_ready=li > 0, out=out_p,
                           want_lse=False)
        if ev:
            ev[1].record()
        n = 0
        for _ in range(steps):
            for li in range(layers):
                qs, kn, vn = dw.suffix[n % len(dw.suffix)]
                kc, vc = caches[li]
                fa.forward_raw(qs, kc, vc, *suf_ids, scale, kn, vn, kvcache=True, workspace=ws_s,
                               summary_ready=n > 0, out=out_s, want_lse=False)
                n += 1
        if ev:
            ev[2].record()

    for _ in range(2):
        run()
    reps = 5
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(reps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for r in range(reps):
        run(evs[r])
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / reps
    pre_ms = sum(e[0].elapsed_time(e[1]) for e in evs) / reps
    suf_ms = sum(e[1].elapsed_time(e[2]) for e in evs) / reps
    valid = w.pad[:, :npre].sum().item()  # valid cached keys over the batch
    kv_bytes = 2 * (valid + w.B * nact) * w.Hkv * w.D * 2
    qo_bytes = 2 * w.B * nact * w.H * w.D * 2
    id_bytes = w.B * (npre + 2 * nact) * 5
    bytes_call = kv_bytes + qo_bytes + id_bytes
    suf_call_us = suf_ms * 1e3 / (layers * steps)
    gbps = bytes_call / (suf_call_us * 1e-6) / 1e9
    pairs_pre = int((w.pad[:, :npre].sum(1) ** 2).sum())
    pre_tflops = 4 * w.D * w.H * pairs_pre * layers / (pre_ms * 1e-3) / 1e12
    return {
        "workload": f"c2: pi0.5 inference bf16 B{w.B} H{w.H} Hkv{w.Hkv} D{w.D}, {layers} prefix calls "
                    f"(S{npre}) + {steps}x{layers} suffix calls (Sq{nact}, Sk{npre + nact})",
        "total_ms": round(pre_ms + suf_ms, 3),
        "wall_ms": round(wall_ms, 3),
        "prefix_ms": round(pre_ms, 3),
        "prefix_tflops": round(pre_tflops, 1),
        "suffix_ms": round(suf_ms, 3),
        "suffix_us_per_call": round(suf_call_us, 2),
        "suffix_algorithmic_bytes_per_call": int(bytes_call),
        "suffix_GBps": round(gbps, 1),
        "suffix_hbm_frac": round(gbps / PEAK_HBM_GBPS, 4),
    }


def cpu_baseline(torch, make_workload, name, budget_s=12.0):
    """The eager CPU oracle (reference algorithm) on a bounded part of the same workload.

    The workload is walked one (sample, kv head) slice at a time -- the kv head's
    K/V with the query heads of its group, forward + backward by autograd -- until
    about ``budget_s`` seconds of CPU work are done; the rate is unmasked FLOPs of
    the slices done over the time they took.
    """
    from oracle import eager

    w = make_workload(name)
    grp = w.H // w.Hkv
    ids = w.block_ids()
    cores = torch.get_num_threads()
    flops, dt, done = 0, 0.0, 0
    for b in range(w.B):
        sl = [t[b : b + 1] for t in ids]
        pairs_b = int(eager.dense_mask_from_block_ids(*sl).sum())
        for hk in range(w.Hkv):
            hs = slice(hk * grp, (hk + 1) * grp)
            # (fp32 copies: the oracle is the reference's eager arithmetic, not a bf16 CPU kernel)
            q, go = w.q[b : b + 1, :, hs].float(), w.d_out[b : b + 1, :, hs].float()
            k, v = w.k[b : b + 1, :, hk : hk + 1].float(), w.v[b : b + 1, :, hk : hk + 1].float()
            t0 = time.perf_counter()
            eager.eager_grads(q, k, v, go, *sl, w.scale)
            dt += time.perf_counter() - t0
            flops += 14 * w.D * grp * pairs_b
            done += 1
            if dt >= budget_s:
                break
        if dt >= budget_s:
            break
    return {
        "value": round(flops / dt / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "seconds": round(dt, 2),
        "sample": f"{name}: first {done} of {w.B * w.Hkv} (sample, kv head) slices, each the kv head with its "
                  f"{grp} query heads, eager fwd+bwd by autograd, {flops / 1e9:.0f} GFLOP unmasked; "
                  f"torch CPU {cores} threads of {os.cpu_count()} cpus",
    }


if __name__ == "__main__":
    sys.exit(main())
