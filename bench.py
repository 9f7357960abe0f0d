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

Kernel durations come from HIP events recorded on the stream the kernels are
launched on (torch's current stream), one pair per launch.  Inputs rotate over
several buffer sets so that no launch finds its operands in the 256 MiB
Infinity Cache from the previous one.
"""
import argparse
import importlib.util
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

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
    the first is bracketed by one event pair and the wall clock (ms_per_step,
    the throughput figure); the second brackets every launch with its own
    event pair (kernel_ms_*, the roofline figure -- an event pair around an
    empty launch reads about 6 us on this runtime, so these run a few percent
    above the kernel-trace durations)."""
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
    return {"ms_per_step": max(region_ms, wall_ms) / steps, "wall_ms_per_step": wall_ms / steps,
            "event_ms_per_step": region_ms / steps,
            "kernel_ms_mean": sum(per) / len(per), "kernel_ms_min": per[0], "kernel_ms_median": per[len(per) // 2]}


# HBM-side bytes per launch (fabric reads + writes of the L2s), from
# `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of this script with
# --copy-calibration: a 1 GiB copy reads FETCH_SIZE = 524304 KiB (scale 2.0)
# and WRITE_SIZE = 1048580 KiB (scale 1.0).
TRAFFIC = {
    "gemm": int((98541.8 * 2.0 + 32791.1) * 1024),    # algorithmic 64 MiB read + 32 MiB written
    "int8": int((144003.5 * 2.0 + 88175.4) * 1024),   # algorithmic 59 MiB read + 86 MiB written
    "mha": int((129697.3 * 2.0 + 65681.9) * 1024),    # algorithmic 208 MiB read + 64 MiB written (default mode)
}


def roofline(ops, ms, peak_tops, traffic=None):
    ach = ops / (ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": round(ach, 2), "peak": peak_tops, "unit": "TFLOP/s", "frac": round(ach / peak_tops, 4),
            "traffic": traffic}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="comma list of: gemm,int8,chain,mha,f32,decode,api,block,norm")
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
        log("bf16 gemm 4096^3: %.4f ms/launch  %.1f TFLOP/s" % (t["kernel_ms_mean"], flops / t["kernel_ms_mean"] / 1e9))
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
                                    "roofline": roofline(ops, t["kernel_ms_mean"], PEAK["int8"], TRAFFIC["int8"]),
                                    "weight_colsum_precompute_ms": round(tc["kernel_ms_mean"], 5)}
        others["int8_mlp_layer"]["roofline"]["unit"] = "TOP/s"
        log("int8 mlp layer: %.4f ms  %.1f TOP/s" % (t["kernel_ms_mean"], ops / t["kernel_ms_mean"] / 1e9))
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
                                    "roofline": roofline(ops, t["kernel_ms_mean"], PEAK["bf16"])}
        log("bf16 mlp chain: %.4f ms  %.1f TFLOP/s" % (t["kernel_ms_mean"], ops / t["kernel_ms_mean"] / 1e9))
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

        # default entry point: key blocks whose mask tile is all -inf for a whole
        # query block are skipped (their softmax weight is exactly 0, so results
        # are identical); "every_block" visits all of them.
        t = mha(True) if args.mha_mode != "every" else None
        td = mha(False) if args.mha_mode != "skip" else None
        entry = {"workload": "B4 H32 S2048 D128, additive causal mask f32[2048,2048] read as data",
                 "unit": "TFLOP/s (dense count 4*B*H*S*S*D)", "dtype": "bf16"}
        if t:
            entry.update({"value": round(ops / t["ms_per_step"] / 1e9, 2), "ms_per_step": round(t["ms_per_step"], 5),
                          "roofline": roofline(ops, t["kernel_ms_mean"], PEAK["bf16"], TRAFFIC["mha"])})
            log("bf16 mha: %.4f ms  %.1f TFLOP/s (dense count)" % (t["kernel_ms_mean"], ops / t["kernel_ms_mean"] / 1e9))
        if td:
            entry["every_block"] = {"value": round(ops / td["ms_per_step"] / 1e9, 2), "ms_per_step": round(td["ms_per_step"], 5),
                                    "roofline": roofline(ops, td["kernel_ms_mean"], PEAK["bf16"])}
            log("bf16 mha visiting every block: %.4f ms  %.1f TFLOP/s" % (td["kernel_ms_mean"], ops / td["kernel_ms_mean"] / 1e9))
        others["bf16_mha"] = entry
        del sets
        torch.cuda.empty_cache()

    # ---------------- decode-style GEMM: 32 rows against Llama-7B FFN weights (split-K path, HBM bound)
    if want("decode"):
        dec = {}
        for (Md, Nd, Kdd) in [(32, 4096, 4096), (32, 11008, 4096), (32, 4096, 11008)]:
            nsets = 4  # 4 x 32..90 MB of weights: beyond the Infinity Cache in rotation
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
                gbs = byts / (t["kernel_ms_mean"] * 1e-3) / 1e9
                entry["weights_" + layout] = {
                    "ms_per_step": round(t["ms_per_step"], 5), "kernel_ms_mean": round(t["kernel_ms_mean"], 5),
                    "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                 "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None}}
                log("bf16 decode gemm %dx%dx%d weights [%s]: %.4f ms  %.0f GB/s of operands" %
                    (Md, Nd, Kdd, layout, t["kernel_ms_mean"], gbs))
            dec["%dx%dx%d" % (Md, Nd, Kdd)] = entry
            del sets
            torch.cuda.empty_cache()
        others["bf16_decode_gemm"] = {"workload": "A[32 x K] . W bf16 with W stored [K,N] (tile kernel over K slices) and [N,K] "
                                                  "(weight-streaming kernel); two launches each (partial sums, then reduction + "
                                                  "epilogue); algorithmic bytes = A + W + C once", "shapes": dec}

    # ---------------- f32 plumbing case (configs[0])
    if want("f32"):
        A, B, bias = wl.f32_matmul_bias_relu()
        Ad, Bd, bd = A.to(dev), B.to(dev), bias.to(dev)
        out = torch.empty(128, 256, device=dev)
        t = time_launches(torch, lambda i: gc.gemm_f32(Ad, Bd, bd, "relu", out=out), 1, K, W)
        others["f32_matmul_bias_relu"] = {"workload": "A[128x512].B[512x256]+bias+ReLU f32 (launch bound)",
                                          "ms_per_step": round(t["ms_per_step"], 5),
                                          "value": round(2.0 * 128 * 512 * 256 / t["kernel_ms_mean"] / 1e9, 4), "unit": "TFLOP/s"}

    # ---------------- the vendor libraries on the same shapes, same process, same timing code (context only)
    if not args.no_vendor and not only:
        import torch.nn.functional as F
        vend = {}
        sets = []
        for s in range(4):
            A, B = wl.bf16_gemm(seed=10 * s)
            sets.append((A.to(dev), B.to(dev), torch.empty(M, N, device=dev, dtype=torch.bfloat16)))
        t = time_launches(torch, lambda i: torch.mm(sets[i][0], sets[i][1], out=sets[i][2]), 4, K, W)
        vend["torch_mm_bf16_4096"] = {"kernel_ms_mean": round(t["kernel_ms_mean"], 5),
                                      "value": round(flops / t["kernel_ms_mean"] / 1e9, 1), "unit": "TFLOP/s"}
        del sets
        Q, Kk, V, mask, scale = wl.bf16_mha(seed=0)
        Qv, Kv, Vv = Q.to(dev), Kk.to(dev), V.to(dev)
        mops = 4.0 * 4 * 32 * 2048 * 2048 * 128
        try:
            t = time_launches(torch, lambda i: F.scaled_dot_product_attention(Qv, Kv, Vv, is_causal=True, scale=scale), 1,
                              max(10, K // 4), 5)
            vend["torch_sdpa_is_causal"] = {"kernel_ms_mean": round(t["kernel_ms_mean"], 5),
                                            "value": round(mops / t["kernel_ms_mean"] / 1e9, 1),
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
        "roofline": roofline(flops, res["kernel_ms_mean"], PEAK["bf16"], TRAFFIC["gemm"]) if res else None,
        "cpu_baseline": cpu,
        "kernel_ms": {k: round(v, 5) for k, v in res.items()} if res else None,
        "others": others,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
