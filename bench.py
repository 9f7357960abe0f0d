#!/usr/bin/env python3
"""Benchmark of the contraction hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only NAME]

A step is one pass of the hot path over one batch of synthetic input that is
already resident in HBM.  The headline workload is the bf16 4096^3 GEMM; the
int8 MLP layer, the bf16 MLP chain, fused attention, decode-shaped GEMMs (32
rows against Llama FFN weights, HBM bound), the f32 plumbing case, the vendor
libraries on the same shapes, the headline GEMM through the partition API, the
llama-2 MLP block through the textual-MLIR entry point and its RMSNorm alone at
prefill size (a fused group with a generated kernel, HBM bound) are measured in
the same run and reported under "others" (--only picks some of them).  One JSON
line goes to stdout; progress goes to stderr.

Time basis: `value`, `ms_per_step` and `roofline.achieved` all come from ONE
clock: the timed region of K back-to-back launches between two
synchronizations, bracketed by a HIP event pair on the stream the kernels are
launched on (torch's current stream); that time divided by K is the step time.
The wall clock around the same region is reported beside it
(`kernel_ms.wall_ms_per_step`: it adds the host's wake-up from the final
synchronize, 20-30 us per region).  A second pass brackets every launch with its own event pair;
those figures are reported under `kernel_ms` only (they include the event
pair's own overhead and isolate launches from each other).  `roofline.traffic`
is not measured in this run: it is the HBM-side byte count of the committed
counter profile named in `roofline.traffic_source`.  Inputs rotate over several
buffer sets so that no launch finds its operands in the 256 MiB Infinity Cache
from the previous one.
"""
import argparse
import importlib.util
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SETTLE_MIN_S, SETTLE_MAX_S = 0.3, 2.0  # untimed load in front of every timed region, see time_launches
PEAK = {"bf16": 2500.0, "int8": 5000.0, "f32": 157.3}  # dense MFMA, TFLOP/s | TOP/s
HBM_PEAK_GBS = 8000.0


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def load_package():
    pkg_dir = os.path.join(ROOT, "graph-compiler_amd")
    spec = importlib.util.spec_from_file_location("graph_compiler_amd", os.path.join(pkg_dir, "__init__.py"),
                                                  submodule_search_locations=[pkg_dir])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["graph_compiler_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


def time_launches(torch, fn, nsets, steps, warmup):
    """fn(i) launches one step on buffer set i.  Two passes of `steps` launches:
    the first is bracketed by one event pair (ms_per_step: the basis of `value`
    AND of the roofline figure) and by the wall clock; the second brackets every
    launch with its own event pair (kernel_ms_*: extra keys, not used for any
    headline figure).

    Before the `warmup` steps the board is brought to its working clocks: an
    idle MI355X raises them under load, most of the way within tens of
    milliseconds (the first 100 launches of the 4096^3 GEMM run 15-20 % slower
    than the 300th) and the last 3-5 % over a few hundred (20 timed launches
    right after 300 untimed ones: 97-101 us; the same 20 after 0.3 s of load:
    the 94 us that 2000 timed launches average).  So groups of 50 untimed
    launches run for at least SETTLE_MIN_S seconds and until three groups in a
    row agree to 0.5 % (at most SETTLE_MAX_S); `settle_launches` says how many
    that took."""
    settle, times, t_begin = 0, [], time.perf_counter()
    while True:
        g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        g0.record()
        for i in range(50):
            fn(i % nsets)
        g1.record()
        torch.cuda.synchronize()
        settle += 50
        times.append(g0.elapsed_time(g1))
        loaded = time.perf_counter() - t_begin
        steady = len(times) >= 3 and max(times[-3:]) <= 1.005 * min(times[-3:])
        if (steady and loaded >= SETTLE_MIN_S) or loaded >= SETTLE_MAX_S:
            break
    for i in range(warmup):
        fn(i % nsets)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        fn(i % nsets)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    region_ms = e0.elapsed_time(e1)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(steps):
        starts[i].record()
        fn(i % nsets)
        stops[i].record()
    torch.cuda.synchronize()
    per = sorted(s.elapsed_time(e) for s, e in zip(starts, stops))
    # The step time is the device's: the HIP-event pair around the K launches on the stream they run on.  The wall
    # clock around the same region (kept beside it) adds the host's wake-up from the final synchronize, 20-30 us per
    # region whatever its length: 1 % of 20 steps of the headline GEMM, nothing of 2000.
    return {"ms_per_step": region_ms / steps, "wall_ms_per_step": wall_ms / steps,
            "event_ms_per_step": region_ms / steps, "settle_launches": settle,
            "kernel_ms_mean": sum(per) / len(per), "kernel_ms_min": per[0], "kernel_ms_median": per[len(per) // 2]}


# HBM-side bytes per launch (fabric reads + writes of the L2s), from
# `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of this script with
# --copy-calibration: a 1 GiB copy reads FETCH_SIZE = 524304 KiB (scale 2.0)
# and WRITE_SIZE = 1048580 KiB (scale 1.0).
# bytes the main kernel of a decode-shaped GEMM fetches per launch (FETCH_SIZE, scaled as above), by (N, K)
DECODE_TRAFFIC = {(4096, 4096): 35_800_000, (11008, 4096): 92_500_000, (4096, 11008): 95_900_000}
TRAFFIC = {  # (bytes per launch of the dominant kernel, the committed profile they come from)
    "gemm": (235414490, "profiles/gemm_tile256_w4_bf16_4096cubed.md"),
    "int8": (384693096, "profiles/gemm_tile256_w4_int8_mlp_layer.md"),
    "chain": (684027008 + 575145347, "profiles/gemm_tile256_w4_bf16_mlp_chain.md"),  # both launches
    "mha": (362734179, "profiles/mha_fwd_fast_b4_h32_s2048_d128_every_block.md"),
    "mha_skip": (330983112, "profiles/mha_fwd_fast_b4_h32_s2048_d128.md"),
}


def roofline(ops, ms, peak_tops, traffic=None, unit="TFLOP/s"):
    """ops per launch / the step time of the timed region (the same ms that gives `value`)."""
    ach = ops / (ms * 1e-3) / 1e12
    r = {"bound": "mfma", "achieved": round(ach, 2), "peak": peak_tops, "unit": unit, "frac": round(ach / peak_tops, 4),
         "traffic": traffic[0] if traffic else None}
    if traffic:
        r["traffic_source"] = traffic[1]
    return r


def cpu_int8_layer(torch, wl, log):
    """Config 3 on the host cores, bounded: the oracle's u8 x s8 deep-tile nest + compensation, dequantise, bias, GELU
    on 256 of the 4096 rows (all 4096 x 11008 weights)."""
    from oracle import gc_oracle as orc
    rows = 256
    A, W, sc, bs = wl.int8_mlp_layer(M=rows, seed=0)
    nt = orc.num_threads()
    t0 = time.perf_counter()
    orc.int8_layer(A.numpy(), W.numpy(), sc.numpy(), bs.numpy(), 128, "gelu_erf")
    dt = time.perf_counter() - t0
    out = {"value": round(2.0 * rows * 4096 * 11008 / dt / 1e12, 5), "unit": "TOP/s", "cores": nt, "kind": "port",
           "sample": "%d of 4096 rows of the int8 MLP layer (oracle: deep-tile nest over the u8 x s8 brgemm restatement, "
                     "compensation, dequantise + bias + GELU), %.2f s" % (rows, dt)}
    log("cpu int8 layer (oracle): %.4f TOP/s on %d threads (%.2f s)" % (out["value"], nt, dt))
    if hasattr(torch, "_int_mm"):
        try:  # torch's own int8 x int8 -> int32 on the CPU (oneDNN), if this build has it there
            a8 = (A.to(torch.int16) - 128).to(torch.int8)
            torch._int_mm(a8[:32], W)
            t0 = time.perf_counter()
            torch._int_mm(a8, W)
            dt2 = time.perf_counter() - t0
            out["torch_int_mm"] = {"value": round(2.0 * rows * 4096 * 11008 / dt2 / 1e12, 5), "unit": "TOP/s",
                                   "cores": torch.get_num_threads(), "sample": "torch._int_mm on the same %d rows (GEMM only)" % rows}
        except Exception as e:  # not built for the CPU in this torch
            out["torch_int_mm"] = {"error": str(e)[:100]}
    return out


def cpu_mlp_chain(torch, wl, log):
    """Config 4 on the host cores, bounded: the oracle's chain (deep-tile nest per layer, bf16 rounding points) on 256 of
    the 4096 rows -- `kind: "port"` -- and torch CPU (oneDNN bf16) on 512 rows beside it."""
    from oracle import gc_oracle as orc
    rows = 256
    x, W1, W2, b2 = wl.bf16_mlp_chain(M=rows, seed=0)
    t0 = time.perf_counter()
    orc.mlp_chain_bf16(wl.bf16_bits(x), wl.bf16_bits(W1), wl.bf16_bits(W2), wl.bf16_bits(b2))
    dt = time.perf_counter() - t0
    out = {"value": round(2 * 2.0 * rows * 4096 * 11008 / dt / 1e12, 5), "unit": "TFLOP/s", "cores": orc.num_threads(),
           "kind": "port", "sample": "%d of 4096 rows through both layers of the oracle's chain, %.2f s" % (rows, dt)}
    rows_t = 512
    x, W1, W2, b2 = wl.bf16_mlp_chain(M=rows_t, seed=0)
    torch.mm(x[:32], W1)
    t0 = time.perf_counter()
    h = torch.relu(torch.mm(x, W1))
    y = torch.mm(h, W2) + b2
    dt_t = time.perf_counter() - t0
    del y
    out["torch_mm_bf16"] = {"value": round(2 * 2.0 * rows_t * 4096 * 11008 / dt_t / 1e12, 5), "unit": "TFLOP/s",
                            "cores": torch.get_num_threads(),
                            "sample": "%d of 4096 rows with torch.mm on the CPU (oneDNN bf16: the closest stand-in for the "
                                      "reference's tiling + oneDNN brgemm), %.2f s" % (rows_t, dt_t)}
    log("cpu mlp chain: oracle %.4f TFLOP/s on %d threads (%.2f s); torch.mm %.4f TFLOP/s" %
        (out["value"], out["cores"], dt, out["torch_mm_bf16"]["value"]))
    return out


def cpu_mha(torch, wl, log):
    """Config 5 on the host cores, bounded: the oracle's attention on 2 of the 128 (batch, head) pairs -- `kind: "port"` --
    and the composition bmm -> scale -> +mask -> softmax -> bmm with torch on the CPU for 4 pairs beside it."""
    from oracle import gc_oracle as orc
    Q, K, V, mask, scale = wl.bf16_mha(B=1, H=4, seed=0)
    per_head = 4.0 * 2048 * 2048 * 128
    t0 = time.perf_counter()
    orc.mha_bf16(wl.bf16_bits(Q[:, :2]), wl.bf16_bits(K[:, :2]), wl.bf16_bits(V[:, :2]), mask.numpy(), scale)
    dt1 = time.perf_counter() - t0
    out = {"value": round(2 * per_head / dt1 / 1e12, 5), "unit": "TFLOP/s (dense count)", "cores": orc.num_threads(),
           "kind": "port", "sample": "2 of 128 (batch, head) pairs through the oracle's attention, %.2f s" % dt1}
    t0 = time.perf_counter()
    S = torch.matmul(Q.float(), K.float().transpose(-1, -2)) * scale + mask
    P = torch.softmax(S, -1).to(torch.bfloat16)
    O = torch.matmul(P.float(), V.float()).to(torch.bfloat16)
    dt = time.perf_counter() - t0
    del S, P, O
    out["torch_composition"] = {"value": round(4 * per_head / dt / 1e12, 5), "unit": "TFLOP/s (dense count)",
                                "cores": torch.get_num_threads(),
                                "sample": "4 of 128 (batch, head) pairs, torch CPU composition bmm/scale/mask/softmax/bmm in "
                                          "f32 with P rounded to bf16, %.2f s" % dt}
    log("cpu mha: oracle %.4f TFLOP/s, torch composition %.4f TFLOP/s" % (out["value"], out["torch_composition"]["value"]))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="comma list of: gemm,int8,chain,mha,f32,decode,api,block,norm,brgemm,ragged,few_tiles")
    ap.add_argument("--cpu-rows", type=int, default=4096, help="rows of the 4096^3 GEMM the CPU baseline computes")
    ap.add_argument("--mha-mode", default="both", choices=["both", "skip", "every"],
                    help="attention: time the default entry point (masked key blocks skipped), the every-block mode, or both")
    ap.add_argument("--no-vendor", action="store_true",
                    help="skip the torch.mm (hipBLASLt) / torch SDPA timings reported under others.vendor_libraries")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch three 1 GiB device copies (known traffic: 1 GiB read + 1 GiB written each) so that "
                         "FETCH_SIZE / WRITE_SIZE counter readings of the other kernels can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU (no sharding, no collectives); --gpus %d is not supported. "
            "Every workload shards without communication over rows / (batch, head) -- run one process per GPU." % args.gpus)
        sys.exit(2)

    import torch
    gc = load_package()
    import importlib
    wl = importlib.import_module("graph_compiler_amd.workloads")
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible; there is no CPU fallback for the product path")
        sys.exit(3)
    dev = torch.device("cuda:0")
    gc.check(gc.lib().gcmi_init(0), "gcmi_init")
    only = set(x for x in args.only.split(",") if x)
    want = lambda n: not only or n in only  # noqa: E731
    K, W = args.steps, args.warmup
    others = {}

    # ---------------- headline: bf16 GEMM 4096^3 (BASELINE configs[1])
    M = N = Kd = 4096
    flops = 2.0 * M * N * Kd
    res = None
    if want("gemm"):
        nsets = 4  # 4 x 100 MB of operands+result > 256 MiB Infinity Cache
        sets = []
        for s in range(nsets):
            A, B = wl.bf16_gemm(seed=10 * s)
            sets.append((A.to(dev), B.to(dev), torch.empty(M, N, device=dev, dtype=torch.bfloat16)))
        t = time_launches(torch, lambda i: gc.gemm_bf16(sets[i][0], sets[i][1], out=sets[i][2]), nsets, K, W)
        res = t
        log("bf16 gemm 4096^3: %.4f ms/step  %.1f TFLOP/s" % (t["ms_per_step"], flops / t["ms_per_step"] / 1e9))
        del sets
        torch.cuda.empty_cache()

    # ---------------- int8 MLP layer (configs[2])
    if want("int8"):
        Mi, Ki, Ni = 4096, 4096, 11008
        ops = 2.0 * Mi * Ki * Ni
        nsets = 3
        sets = []
        for s in range(nsets):
            A, Wt, sc, bs = wl.int8_mlp_layer(seed=10 * s)
            Wd = Wt.to(dev)
            sets.append((A.to(dev), Wd, gc.colsum_s8(Wd), sc.to(dev), bs.to(dev),
                         torch.empty(Mi, Ni, device=dev, dtype=torch.bfloat16)))
        t = time_launches(torch, lambda i: gc.gemm_int8(sets[i][0], sets[i][1], sets[i][2], 128, sets[i][3], sets[i][4],
                                                        "gelu_erf", gc.BF16, sets[i][5]), nsets, K, W)
        tc = time_launches(torch, lambda i: gc.colsum_s8(sets[i][1]), nsets, 10, 2)
        others["int8_mlp_layer"] = {"workload": "u8[4096x4096] x s8[4096x11008] -> s32 -> dequant+bias+GELU -> bf16",
                                    "value": round(ops / t["ms_per_step"] / 1e9, 2), "unit": "TOP/s", "dtype": "int8",
                                    "ms_per_step": round(t["ms_per_step"], 5),
                                    "roofline": roofline(ops, t["ms_per_step"], PEAK["int8"], TRAFFIC["int8"], "TOP/s"),
                                    "kernel_ms": {k: round(v, 5) for k, v in t.items()},
                                    "weight_colsum_precompute_ms": round(tc["ms_per_step"], 5)}
        log("int8 mlp layer: %.4f ms  %.1f TOP/s" % (t["ms_per_step"], ops / t["ms_per_step"] / 1e9))
        if not args.no_cpu:
            others["int8_mlp_layer"]["cpu_baseline"] = cpu_int8_layer(torch, wl, log)
        del sets
        torch.cuda.empty_cache()

    # ---------------- bf16 MLP chain (configs[3]): two launches per step
    if want("chain"):
        Mc, Kc, Hc = 4096, 4096, 11008
        ops = 2 * 2.0 * Mc * Kc * Hc
        nsets = 2
        sets = []
        for s in range(nsets):
            x, W1, W2, b2 = wl.bf16_mlp_chain(seed=10 * s)
            sets.append((x.to(dev), W1.to(dev), W2.to(dev), b2.to(dev),
                         torch.empty(Mc, Hc, device=dev, dtype=torch.bfloat16),
                         torch.empty(Mc, Kc, device=dev, dtype=torch.bfloat16)))

        def chain(i):
            x, W1, W2, b2, h, y = sets[i]
            gc.gemm_bf16(x, W1, None, "relu", out=h)
            gc.gemm_bf16(h, W2, b2, None, out=y)

        t = time_launches(torch, chain, nsets, K, W)
        others["bf16_mlp_chain"] = {"workload": "x[4096x4096] -> W1[4096x11008]+ReLU -> W2[11008x4096]+bias, bf16",
                                    "value": round(ops / t["ms_per_step"] / 1e9, 2), "unit": "TFLOP/s", "dtype": "bf16",
                                    "ms_per_step": round(t["ms_per_step"], 5),
                                    "roofline": roofline(ops, t["ms_per_step"], PEAK["bf16"], TRAFFIC["chain"]),
                                    "kernel_ms": {k: round(v, 5) for k, v in t.items()}}
        log("bf16 mlp chain: %.4f ms  %.1f TFLOP/s" % (t["ms_per_step"], ops / t["ms_per_step"] / 1e9))
        if not args.no_cpu:
            others["bf16_mlp_chain"]["cpu_baseline"] = cpu_mlp_chain(torch, wl, log)
        del sets
        torch.cuda.empty_cache()

    # ---------------- fused attention (configs[4])
    if want("mha"):
        Bm, Hm, Sm, Dm = 4, 32, 2048, 128
        ops = 4.0 * Bm * Hm * Sm * Sm * Dm  # dense count: the mask is data
        nsets = 2
        sets = []
        for s in range(nsets):
            Q, Kk, V, mask, scale = wl.bf16_mha(seed=10 * s)
            sets.append((Q.to(dev), Kk.to(dev), V.to(dev), mask.to(dev), torch.empty(Bm, Hm, Sm, Dm, device=dev, dtype=torch.bfloat16)))
        def mha(skip):
            return time_launches(torch, lambda i: gc.mha_fwd_bf16(sets[i][0], sets[i][1], sets[i][2], sets[i][3], scale,
                                                                  sets[i][4], skip_masked=skip), nsets, K, W)

        # The graded figure visits EVERY key block (dense operation count, the mask read as data).  The default
        # entry point skips key blocks whose mask tile is all -inf for a whole 128-row query block (their softmax
        # weight is exactly 0: identical results); it is reported separately, with the operations it really
        # executed as the roofline numerator and the dense-count figure beside it.
        td = mha(False) if args.mha_mode != "skip" else None
        t = mha(True) if args.mha_mode != "every" else None
        entry = {"workload": "B4 H32 S2048 D128, additive causal mask f32[2048,2048] read as data, every key block visited",
                 "unit": "TFLOP/s (dense count 4*B*H*S*S*D)", "dtype": "bf16"}
        if td:
            entry.update({"value": round(ops / td["ms_per_step"] / 1e9, 2), "ms_per_step": round(td["ms_per_step"], 5),
                          "roofline": roofline(ops, td["ms_per_step"], PEAK["bf16"], TRAFFIC["mha"]),
                          "kernel_ms": {k: round(v, 5) for k, v in td.items()}})
            log("bf16 mha visiting every block: %.4f ms  %.1f TFLOP/s" % (td["ms_per_step"], ops / td["ms_per_step"] / 1e9))
        if td:
            # the same every-block run for a mask that is a constant of the partition: its tile classes are prepared
            # once (as dnnl_graph_compiler_execute does for a mask with property_type "constant"), so a step is the
            # attention kernel alone.  Reported beside the figure above, never instead of it.
            classes = [gc.mha_mask_classes(sets[i][3], Sm, Sm, Dm) for i in range(nsets)]
            tp = time_launches(torch, lambda i: gc.mha_fwd_bf16_classified(sets[i][0], sets[i][1], sets[i][2], sets[i][3],
                                                                           classes[i], scale, sets[i][4], skip_masked=False),
                               nsets, K, W)
            entry["constant_mask_classes_prepared_once"] = {
                "ms_per_step": round(tp["ms_per_step"], 5), "value": round(ops / tp["ms_per_step"] / 1e9, 2),
                "roofline": roofline(ops, tp["ms_per_step"], PEAK["bf16"], TRAFFIC["mha"])}
            log("bf16 mha visiting every block, constant mask (classes prepared once): %.4f ms  %.1f TFLOP/s" %
                (tp["ms_per_step"], ops / tp["ms_per_step"] / 1e9))
        if t:
            m = sets[0][3]
            blk = (m.view(Sm // 128, 128, Sm // 64, 64) == float("-inf")).all(dim=3).all(dim=1)  # [query block, key block]
            visited = int((~blk).sum().item())
            frac_exec = visited / blk.numel()
            entry["masked_blocks_skipped"] = {
                "workload": "the same call through the default entry point: key blocks that are -inf for a whole 128-row "
                            "query block are not visited (%d of %d visited)" % (visited, blk.numel()),
                "ms_per_step": round(t["ms_per_step"], 5),
                "effective_value_dense_count": round(ops / t["ms_per_step"] / 1e9, 2),
                "executed_ops": ops * frac_exec,
                "roofline_executed_ops": roofline(ops * frac_exec, t["ms_per_step"], PEAK["bf16"], TRAFFIC["mha_skip"]),
                "kernel_ms": {k: round(v, 5) for k, v in t.items()}}
            log("bf16 mha, masked blocks skipped: %.4f ms  %.1f TFLOP/s dense count, %.1f TFLOP/s executed" %
                (t["ms_per_step"], ops / t["ms_per_step"] / 1e9, ops * frac_exec / t["ms_per_step"] / 1e9))
        if not args.no_cpu:
            entry["cpu_baseline"] = cpu_mha(torch, wl, log)
        others["bf16_mha"] = entry
        del sets
        torch.cuda.empty_cache()

    # ---------------- decode-style GEMM: 32 rows against Llama-7B FFN weights (split-K path, HBM bound)
    if want("decode"):
        dec = {}
        for (Md, Nd, Kdd) in [(32, 4096, 4096), (32, 11008, 4096), (32, 4096, 11008)]:
            # weight buffers in rotation: 600 MB or more of them, so that none is left in the 256 MB last-level cache
            # when its turn comes again (4 x 32 MB would be served from that cache)
            nsets = max(4, -(-600_000_000 // (2 * Nd * Kdd)))
            sets = []
            for s in range(nsets):
                torch.manual_seed(100 + s)
                sets.append(((torch.randn(Md, Kdd) * 0.1).to(torch.bfloat16).to(dev),
                             (torch.randn(Kdd, Nd) * 0.02).to(torch.bfloat16).to(dev),
                             torch.empty(Md, Nd, device=dev, dtype=torch.bfloat16)))
            byts = 2.0 * (Md * Kdd + Kdd * Nd + Md * Nd)
            entry = {}
            for layout in ("kn", "nk"):
                if layout == "nk":  # the same weights stored [N,K], as torch.nn.Linear and the reference's llama2 case do
                    sets = [(a, b.t().contiguous(), c) for (a, b, c) in sets]
                    fn = lambda i: gc.gemm_bf16_nt(sets[i][0], sets[i][1], out=sets[i][2])  # noqa: E731
                else:
                    fn = lambda i: gc.gemm_bf16(sets[i][0], sets[i][1], out=sets[i][2])  # noqa: E731
                t = time_launches(torch, fn, nsets, K, W)
                gbs = byts / (t["ms_per_step"] * 1e-3) / 1e9
                entry["weights_" + layout] = {
                    "ms_per_step": round(t["ms_per_step"], 5), "kernel_ms_mean": round(t["kernel_ms_mean"], 5),
                    "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                 "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": DECODE_TRAFFIC.get((Nd, Kdd)),
                                 "traffic_source": "profiles/gemm_rows32_bf16_decode_shapes.md"}}
                log("bf16 decode gemm %dx%dx%d weights [%s]: %.4f ms  %.0f GB/s of operands" %
                    (Md, Nd, Kdd, layout, t["ms_per_step"], gbs))
            dec["%dx%dx%d" % (Md, Nd, Kdd)] = entry
            del sets
            torch.cuda.empty_cache()
        others["bf16_decode_gemm"] = {"workload": "A[32 x K] . W bf16 with W stored [K,N] and [N,K]: the 8-wave weight-streaming kernel "
                                                  "on panels of 64 columns (one launch for N = 11008; K slices + reduction and epilogue "
                                                  "in a second launch for N = 4096); algorithmic bytes = A + W + C once",
                                      "shapes": dec}

    # ---------------- the same kernels on shapes off their tile sizes (parity cases elsewhere; here: no cliff)
    if want("ragged"):
        rag = {}
        Mr, Nr, Kr = 4000, 4000, 4096
        Ar = (torch.randn(Mr, Kr) * 0.1).to(torch.bfloat16).to(dev)
        Br = (torch.randn(Kr, Nr) * 0.1).to(torch.bfloat16).to(dev)
        Cr = torch.empty(Mr, Nr, dtype=torch.bfloat16, device=dev)
        t = time_launches(torch, lambda i: gc.gemm_bf16(Ar, Br, out=Cr), 1, max(20, K // 2), W)
        rag["bf16_gemm_4000x4000x4096"] = {"ms_per_step": round(t["ms_per_step"], 5),
                                           "value": round(2.0 * Mr * Nr * Kr / t["ms_per_step"] / 1e9, 1), "unit": "TFLOP/s"}
        del Ar, Br, Cr
        for name, S, D in (("bf16_mha_b4_h32_s2000_d128_causal", 2000, 128), ("bf16_mha_b4_h32_s2048_d64_causal", 2048, 64)):
            Q, Kk, V, mask, scale = wl.bf16_mha(4, 32, S, D)
            Qd, Kkd, Vd, md = Q.to(dev), Kk.to(dev), V.to(dev), mask.to(dev)
            Od = torch.empty_like(Qd)
            t = time_launches(torch, lambda i: gc.mha_fwd_bf16(Qd, Kkd, Vd, md, scale, out=Od), 1, max(10, K // 4), 5)
            rag[name] = {"ms_per_step": round(t["ms_per_step"], 5),
                         "value": round(4.0 * 4 * 32 * S * S * D / t["ms_per_step"] / 1e9, 1),
                         "unit": "TFLOP/s (dense count, masked blocks skipped)"}
            del Qd, Kkd, Vd, md, Od
        others["shapes_off_the_tile_sizes"] = {
            "workload": "M and N of a GEMM not multiples of 256 (edge tiles of the whole-tile kernel), a sequence length "
                        "that is not a multiple of 128 / 64 (overlapping last windows on the pipelined attention kernel), "
                        "head dim 64 (the pipelined attention kernel's second instantiation)", "cases": rag}
        log("off the tile sizes: %s" % json.dumps(rag))
        torch.cuda.empty_cache()

    # ---------------- bf16 GEMMs whose 256 x 256 tiles would not fill the GPU: 128 x 128 tiles and / or K slices
    if want("few_tiles"):
        few = {}
        for Mf, Nf, Kf in ((2048, 2048, 2048), (1024, 4096, 4096), (512, 4096, 4096), (1024, 1024, 8192), (2048, 4096, 4096),
                           (4096, 5120, 4096)):  # the last: 320 large tiles, a round and a thin one (run on small tiles)
            Af = (torch.randn(Mf, Kf) * 0.1).to(torch.bfloat16).to(dev)
            Bf = (torch.randn(Kf, Nf) * 0.1).to(torch.bfloat16).to(dev)
            Cf = torch.empty(Mf, Nf, dtype=torch.bfloat16, device=dev)
            t = time_launches(torch, lambda i: gc.gemm_bf16(Af, Bf, out=Cf), 1, max(20, K // 2), W)
            cfgf, _ = gc.tile_config(Mf, Nf, Kf)
            few["%dx%dx%d" % (Mf, Nf, Kf)] = {"ms_per_step": round(t["ms_per_step"], 5),
                                              "value": round(2.0 * Mf * Nf * Kf / t["ms_per_step"] / 1e9, 1), "unit": "TFLOP/s",
                                              "tile": int(cfgf.bm), "k_slices": int(cfgf.split_k), "workgroups": int(cfgf.workgroups)}
            del Af, Bf, Cf
        # the int8 layer at a quarter of its rows: 172 tiles of 256 x 256, or 688 of 128 x 128
        Mi, Ni, Ki = 1024, 4096, 4096
        Ai = torch.randint(0, 256, (Mi, Ki), dtype=torch.uint8, device=dev)
        Wi = torch.randint(-127, 128, (Ki, Ni), dtype=torch.int8, device=dev)
        csi = gc.colsum_s8(Wi)
        sci, bii = (torch.rand(Ni, device=dev) * 0.009 + 0.001).float(), torch.randn(Ni, device=dev).float()
        Oi = torch.empty(Mi, Ni, dtype=torch.bfloat16, device=dev)
        t = time_launches(torch, lambda i: gc.gemm_int8(Ai, Wi, csi, 128, sci, bii, "gelu_erf", gc.BF16, out=Oi), 1, max(20, K // 2), W)
        cfgf, _ = gc.tile_config(Mi, Ni, Ki, a_dtype=gc.U8)
        few["int8_%dx%dx%d_dequant_bias_gelu" % (Mi, Ni, Ki)] = {
            "ms_per_step": round(t["ms_per_step"], 5), "value": round(2.0 * Mi * Ni * Ki / t["ms_per_step"] / 1e9, 1), "unit": "TOP/s",
            "tile": int(cfgf.bm), "k_slices": int(cfgf.split_k), "workgroups": int(cfgf.workgroups)}
        del Ai, Wi, Oi
        others["bf16_gemm_few_tiles"] = {
            "workload": "bf16 GEMMs of 16 to 128 tiles of 256 x 256 (one compute unit works 1.9 us per tile and 128 of K): the "
                        "launcher gives them to more workgroups by 128 x 128 tiles, K slices, or both; one of 320 tiles (a "
                        "full round on large tiles, the 64 left over on small ones); and one 8-bit layer of 64 large "
                        "tiles (128 x 128 tiles)", "cases": few}
        log("few tiles: %s" % json.dumps(few))
        torch.cuda.empty_cache()

    # ---------------- f32 plumbing case (configs[0])
    if want("f32"):
        A, B, bias = wl.f32_matmul_bias_relu()
        Ad, Bd, bd = A.to(dev), B.to(dev), bias.to(dev)
        out = torch.empty(128, 256, device=dev)
        t = time_launches(torch, lambda i: gc.gemm_f32(Ad, Bd, bd, "relu", out=out), 1, K, W)
        others["f32_matmul_bias_relu"] = {"workload": "A[128x512].B[512x256]+bias+ReLU f32 (launch bound)",
                                          "ms_per_step": round(t["ms_per_step"], 5),
                                          "value": round(2.0 * 128 * 512 * 256 / t["ms_per_step"] / 1e9, 4), "unit": "TFLOP/s"}

    # ---------------- the microkernel ABI (dnnl_brgemm_*, device pointers) at the size the reference's nest calls it with
    if want("brgemm"):
        import ctypes as C
        L = gc.lib()
        legs = {}
        for name, dtA, dtB, es, Kk in (("f32", 3, 3, 4, 32), ("bf16_vnni2", 2, 2, 2, 32), ("u8s8_vnni4", 6, 5, 1, 64)):
            Mb = Nb = 32
            num = 16
            Ab = torch.randint(0, 120, (num * Mb * Kk * es,), dtype=torch.uint8, device=dev)
            Bb = torch.randint(0, 120, (num * Kk * Nb * es,), dtype=torch.uint8, device=dev)
            Cb = torch.zeros(Mb * Nb, dtype=torch.int32, device=dev)
            h = L.dnnl_brgemm_dispatch(Mb, Nb, Kk, Kk, Nb, Nb, Mb * Kk, Kk * Nb, 0.0, dtA, dtB)
            a, b, c = C.c_void_p(Ab.data_ptr()), C.c_void_p(Bb.data_ptr()), C.c_void_p(Cb.data_ptr())
            t = time_launches(torch, lambda i: L.dnnl_brgemm_execute(h, a, 0, b, 0, c, 0, num), 1, K, W)
            legs[name] = {"M": Mb, "N": Nb, "K": Kk, "num": num, "us_per_call": round(t["ms_per_step"] * 1e3, 2),
                          "GFLOP/s": round(2.0 * Mb * Nb * Kk * num / t["ms_per_step"] / 1e6, 1)}
        others["brgemm_microkernel_abi"] = {
            "workload": "one dnnl_brgemm_execute per step: 32x32 C tile, batch of 16 K blocks (the call the reference's "
                        "deep-tile nest makes per innermost tile); launch bound by construction -- the GPU path of the "
                        "nest is the whole-problem kernel above, this ABI exists for callers that bind the microkernel",
            "legs": legs}
        log("brgemm microkernel: %s" % json.dumps(legs))

    # ---------------- the vendor libraries on the same shapes, same process, same timing code (context only)
    if not args.no_vendor and not only:
        import torch.nn.functional as F
        vend = {}
        sets = []
        for s in range(4):
            A, B = wl.bf16_gemm(seed=10 * s)
            sets.append((A.to(dev), B.to(dev), torch.empty(M, N, device=dev, dtype=torch.bfloat16)))
        t = time_launches(torch, lambda i: torch.mm(sets[i][0], sets[i][1], out=sets[i][2]), 4, K, W)
        vend["torch_mm_bf16_4096"] = {"ms_per_step": round(t["ms_per_step"], 5),
                                      "value": round(flops / t["ms_per_step"] / 1e9, 1), "unit": "TFLOP/s"}
        del sets
        # the vendor library's s8 x s8 -> s32 GEMM at the int8 layer's shape: raw accumulators only (no zero point, no
        # dequantise / bias / GELU, and 4 bytes per result written instead of 2) -- a same-box yardstick for the main
        # loop, not the same work
        try:
            Ai = torch.randint(-128, 128, (4096, 4096), dtype=torch.int8, device=dev)
            Wi = torch.randint(-127, 128, (4096, 11008), dtype=torch.int8, device=dev)
            t = time_launches(torch, lambda i: torch._int_mm(Ai, Wi), 1, max(10, K // 2), 5)
            vend["torch_int_mm_s8s8s32_4096x11008x4096"] = {
                "ms_per_step": round(t["ms_per_step"], 5), "value": round(2.0 * 4096 * 4096 * 11008 / t["ms_per_step"] / 1e9, 1),
                "unit": "TOP/s"}
            del Ai, Wi
        except Exception as e:
            vend["torch_int_mm_s8s8s32_4096x11008x4096"] = {"error": str(e)[:120]}
        Q, Kk, V, mask, scale = wl.bf16_mha(seed=0)
        Qv, Kv, Vv = Q.to(dev), Kk.to(dev), V.to(dev)
        mops = 4.0 * 4 * 32 * 2048 * 2048 * 128
        try:
            t = time_launches(torch, lambda i: F.scaled_dot_product_attention(Qv, Kv, Vv, is_causal=True, scale=scale), 1,
                              max(10, K // 4), 5)
            vend["torch_sdpa_is_causal"] = {"ms_per_step": round(t["ms_per_step"], 5),
                                            "value": round(mops / t["ms_per_step"] / 1e9, 1),
                                            "unit": "TFLOP/s (dense count)"}
        except Exception as e:  # the library may lack a kernel for this build
            vend["torch_sdpa_is_causal"] = {"error": str(e)[:120]}
        others["vendor_libraries"] = vend
        log("vendor libraries: %s" % json.dumps(vend))
        del Qv, Kv, Vv
        torch.cuda.empty_cache()

    # ---------------- the same GEMM through dnnl_graph_compiler_execute (the drop-in boundary)
    if want("api"):
        ga = importlib.import_module("graph_compiler_amd.graph_api")
        A, B = wl.bf16_gemm(seed=0)
        comp = ga.Compiler()
        st, exe = comp.compile(ga.gemm_json(M, Kd, N, "bf16"))
        if st:
            log("bench.py: compile of the GEMM partition failed with status %d" % st)
            sys.exit(4)
        Ad, Bd = A.to(dev), B.to(dev)
        Cd = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
        Ch = torch.empty(M, N, dtype=torch.bfloat16)

        def wall(fn, n):
            fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3 / n

        t_dev = wall(exe.bind([(0, Ad), (1, Bd)], [(2, Cd)]), max(10, K // 2))  # tensor structs built once, as a C caller's
        t_host = wall(exe.bind([(0, A), (1, B)], [(2, Ch)]), 5)
        exe.close()
        comp.close()
        others["api_execute_bf16_gemm"] = {
            "workload": "the headline GEMM as a one-MatMul JSON partition through dnnl_graph_compiler_execute "
                        "(returns after completion; wall clock per call)",
            "device_pointers": {"ms_per_call": round(t_dev, 4), "value": round(flops / t_dev / 1e9, 2), "unit": "TFLOP/s"},
            "host_pointers_pcie_inclusive": {"ms_per_call": round(t_host, 3), "value": round(flops / t_host / 1e9, 2),
                                             "unit": "TFLOP/s", "note": "pageable host buffers: 64 MiB in, 32 MiB out per call"}}
        log("api execute: %.4f ms with device pointers, %.2f ms with host pointers" % (t_dev, t_host))
        del Ad, Bd, Cd

    # ---------------- the llama-2 decoder MLP block of the reference's benchgc case, as textual MLIR through the API
    if want("block"):
        ga = importlib.import_module("graph_compiler_amd.graph_api")
        mlm = importlib.import_module("graph_compiler_amd.mlir_modules")
        T, H, Fd = 32, 4096, 11008
        comp = ga.Compiler()
        st, exe = comp.compile_mlir(mlm.decoder_mlp_block(T, H, Fd))
        if st:
            log("bench.py: compile_mlir of the decoder block failed with status %d: %s" %
                (st, ga.api().dnnl_graph_compiler_last_error().decode()))
            sys.exit(4)
        bf = torch.bfloat16
        torch.manual_seed(7)
        rn = lambda *sh: torch.randn(*sh, device=dev)  # noqa: E731
        nsets = 3  # 3 x 304 MB of weights: beyond the 256 MB Infinity Cache in rotation
        sets = []
        for _ in range(nsets):
            sets.append([rn(1, T, H).to(bf), (rn(H, H) / H ** 0.5).to(bf), rn(1, T, H).to(bf),
                         torch.full((1,), 1e-5, device=dev), (1 + 0.1 * rn(H)).to(bf), (rn(Fd, H) / H ** 0.5).to(bf),
                         (rn(Fd, H) / H ** 0.5).to(bf), (rn(H, Fd) / Fd ** 0.5).to(bf), torch.full((1,), 1e-5, device=dev),
                         (1 + 0.1 * rn(H)).to(bf)])
        o1 = torch.empty(1, T, H, device=dev, dtype=bf)
        o2 = torch.empty(1, T, H, device=dev, dtype=bf)
        st_plan, plan = ga.explain_mlir(mlm.decoder_mlp_block(T, H, Fd))
        n_launch = len([ln for ln in plan.splitlines() if not ln.startswith(("arena", "target"))])

        bound = [exe.bind(list(enumerate(st_)), [(10, o1), (11, o2)]) for st_ in sets]  # tensor structs built once

        def run_block(i):
            rc = bound[i % nsets]()
            if rc:
                raise RuntimeError("execute -> %d" % rc)

        for i in range(3):
            run_block(i)
        torch.cuda.synchronize()
        n = max(12, K // 2)
        t0 = time.perf_counter()
        for i in range(n):
            run_block(i)
        torch.cuda.synchronize()
        t_blk = (time.perf_counter() - t0) * 1e3 / n
        # the same through execute_async on torch's stream: launches only, one wait at the end (a serving loop that
        # keeps its tensors on the GPU)
        cur = torch.cuda.current_stream().cuda_stream
        bound_async = [exe.bind(list(enumerate(st_)), [(10, o1), (11, o2)], stream=cur) for st_ in sets]
        for i in range(3):
            bound_async[i % nsets]()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            if bound_async[i % nsets]():
                raise RuntimeError("execute_async failed")
        torch.cuda.synchronize()
        t_blk_async = (time.perf_counter() - t0) * 1e3 / n
        # and recorded once per buffer set into a HIP graph, then replayed
        side = torch.cuda.Stream()
        graphs = []
        with torch.cuda.stream(side):
            for st_ in sets:
                call = exe.bind(list(enumerate(st_)), [(10, o1), (11, o2)], stream=side.cuda_stream)
                call()
                side.synchronize()
                gr = torch.cuda.CUDAGraph()
                gr.capture_begin()
                call()
                gr.capture_end()
                graphs.append((gr, call))
        side.synchronize()
        for i in range(3):
            graphs[i % nsets][0].replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            graphs[i % nsets][0].replay()
        torch.cuda.synchronize()
        t_blk_graph = (time.perf_counter() - t0) * 1e3 / n
        del graphs
        exe.close()
        comp.close()
        byts = 2.0 * (H * H + 3 * H * Fd) + 2.0 * 4 * T * H
        gbs = byts / (t_blk * 1e-3) / 1e9
        others["mlir_llama2_mlp_block"] = {
            "workload": "test/benchgc/cases/llama2.mlir shape (32 tokens, hidden 4096, ffn 11008): o-proj + residual, RMSNorm, "
                        "gated FFN, residual, RMSNorm; textual MLIR through compile_mlir/execute with device pointers; wall "
                        "clock per execute (returns after completion); algorithmic bytes = the four weights + activations once",
            "launches_per_execute": n_launch, "ms_per_execute": round(t_blk, 4),
            "ms_per_execute_async_back_to_back": round(t_blk_async, 4),
            "ms_per_hip_graph_replay_back_to_back": round(t_blk_graph, 4),
            "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None}}
        log("mlir llama2 block: %.4f ms per execute, %d launches, %.0f GB/s of weights; back to back: %.4f ms through execute_async, %.4f ms as HIP graph replays"
            % (t_blk, n_launch, gbs, t_blk_async, t_blk_graph))
        del sets
        torch.cuda.empty_cache()

    # ---------------- a fused group alone: the RMSNorm of the same case at prefill size (HBM bound)
    if want("norm"):
        ga = importlib.import_module("graph_compiler_amd.graph_api")
        mlm = importlib.import_module("graph_compiler_amd.mlir_modules")
        T, H = 16384, 4096
        comp = ga.Compiler()
        st, exe = comp.compile_mlir(mlm.rmsnorm(T, H))
        if st:
            log("bench.py: compile_mlir of the RMSNorm failed with status %d: %s" %
                (st, ga.api().dnnl_graph_compiler_last_error().decode()))
            sys.exit(4)
        torch.manual_seed(8)
        nsets = 3  # 3 x 256 MiB of rows in rotation: beyond the Infinity Cache
        xs = [torch.randn(1, T, H, device=dev).to(torch.bfloat16) for _ in range(nsets)]
        outs = [torch.empty(1, T, H, device=dev, dtype=torch.bfloat16) for _ in range(nsets)]
        eps = torch.full((1,), 1e-5, device=dev)
        gamma = (1 + 0.1 * torch.randn(H, device=dev)).to(torch.bfloat16)
        before = ga.generated_kernel_launches()

        bound = [exe.bind([(0, xs[j]), (1, eps), (2, gamma)], [(3, outs[j])]) for j in range(nsets)]

        def run_norm(i):
            rc = bound[i % nsets]()
            if rc:
                raise RuntimeError("execute -> %d" % rc)

        for i in range(3):
            run_norm(i)
        torch.cuda.synchronize()
        n = max(12, K // 2)
        t0 = time.perf_counter()
        for i in range(n):
            run_norm(i)
        torch.cuda.synchronize()
        t_norm = (time.perf_counter() - t0) * 1e3 / n
        generated = ga.generated_kernel_launches() - before == n + 3
        exe.close()
        comp.close()
        byts = 2.0 * 2 * T * H  # each row read once and written once
        gbs = byts / (t_norm * 1e-3) / 1e9
        others["mlir_rmsnorm_16384x4096"] = {
            "workload": "RMSNorm of test/benchgc/cases/llama2.mlir on 16384 tokens x 4096 (bf16 in and out, f32 inside): 13 linalg/"
                        "tensor ops, one launch; textual MLIR through compile_mlir/execute with device pointers; wall clock per "
                        "execute (returns after completion); algorithmic bytes = the rows read once and written once",
            "kernel": "generated at compile time (hiprtc)" if generated else "the library's generic row kernel",
            "ms_per_execute": round(t_norm, 4),
            "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None}}
        log("mlir rmsnorm %dx%d: %.4f ms per execute, %.0f GB/s (%s kernel)" % (T, H, t_norm, gbs, "generated" if generated else "library"))
        del xs, outs
        torch.cuda.empty_cache()

    if args.copy_calibration:
        src = torch.empty(1 << 28, device=dev, dtype=torch.float32).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---------------- CPU baseline: the oracle's deep-tile nest on a bounded sample
    cpu = None
    if not args.no_cpu and want("gemm"):
        from oracle import gc_oracle as orc
        rows = args.cpu_rows
        A, B = wl.bf16_gemm(M=rows, seed=0)
        a16, b16 = wl.bf16_bits(A), wl.bf16_bits(B)
        nt = orc.num_threads()
        t0 = time.perf_counter()
        orc.matmul_bf16(a16, b16)
        dt = time.perf_counter() - t0
        cpu = {"value": round(2.0 * rows * N * Kd / dt / 1e12, 5), "unit": "TFLOP/s", "cores": nt, "kind": "port",
               "sample": "%d of 4096 rows of the same bf16 4096^3 GEMM (deep-tile nest, 32^3 brgemm restatement, "
                         "gcc -O3 -march=native, OpenMP), %.2f s" % (rows, dt)}
        log("cpu baseline: %.4f TFLOP/s on %d threads (%.2f s)" % (cpu["value"], nt, dt))
        # second CPU figure: torch's bundled oneDNN kernels on the same operands
        # (the closest stand-in here for the reference's tiling + oneDNN brgemm)
        torch.mm(A[:128], B)
        t0 = time.perf_counter()
        reps = 0
        while reps < 1 or (time.perf_counter() - t0 < 5.0 and reps < 20):
            torch.mm(A, B)
            reps += 1
        dt2 = (time.perf_counter() - t0) / reps
        cpu["torch_mm_bf16"] = {"value": round(2.0 * rows * N * Kd / dt2 / 1e12, 5), "unit": "TFLOP/s",
                                "cores": torch.get_num_threads(), "sample": "torch.mm on the same operands, mean of %d" % reps}
        log("cpu torch.mm bf16: %.4f TFLOP/s on %d threads" % (cpu["torch_mm_bf16"]["value"], torch.get_num_threads()))

    line = {
        "metric": "TFLOPS/TOPS + % of MI355X MFMA peak: bf16 4096^3 GEMM, int8 MLP, bf16 MHA",
        "value": round(flops / res["ms_per_step"] / 1e9, 2) if res else None,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(res["ms_per_step"], 5) if res else None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "bf16 GEMM M=N=K=4096, row-major A and B, N(0,1)*0.1, f32 accumulate, bf16 out, no post-op",
                   "buffer_sets": 4},
        "roofline": roofline(flops, res["ms_per_step"], PEAK["bf16"], TRAFFIC["gemm"]) if res else None,
        "cpu_baseline": cpu,
        "kernel_ms": {k: round(v, 5) for k, v in res.items()} if res else None,
        "others": others,
    }
    # The whole record (workload descriptions, per-launch event timings of every entry) goes to stderr; the line on
    # stdout is the same record without the prose and the per-launch sub-dicts, so that it stays a few KB.
    log("full record: " + json.dumps(line))

    def compact(v, depth=0):
        if isinstance(v, dict):
            return {k: compact(x, depth + 1) for k, x in v.items()
                    if not (depth >= 1 and k in ("workload", "kernel_ms", "note", "sample", "traffic_source"))}
        return v

    short = dict(line)
    short["others"] = compact(others, 1)
    print(json.dumps(short, separators=(",", ":")), flush=True)
    # the three other named configurations once more, last on stderr
    for key, name in (("int8_mlp_layer", "C3 int8 layer"), ("bf16_mlp_chain", "C4 bf16 mlp chain"),
                      ("bf16_mha", "C5 attention, every key block")):
        e = others.get(key)
        if e and "roofline" in e:
            log("%s: %.4f ms, %.1f %s, frac %.4f of the dense MFMA peak" %
                (name, e["ms_per_step"], e["value"], e["unit"].split(" ")[0], e["roofline"]["frac"]))
    if res:
        log("C2 bf16 gemm 4096^3: %.4f ms, %.1f TFLOP/s, frac %.4f of the dense MFMA peak" %
            (res["ms_per_step"], flops / res["ms_per_step"] / 1e9, flops / res["ms_per_step"] / 1e9 / PEAK["bf16"]))


if __name__ == "__main__":
    main()
