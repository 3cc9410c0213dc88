#!/usr/bin/env python3
"""Benchmark of the CAM MoE hot path on one MI355X.

One "step" = one dispatch pass (routing plan + permute with per-token int8 quantisation, 4096 tokens x
7168 bf16, 256 experts, top-8) followed by one combine pass (32768 bf16 rows x 7168 gathered back to
4096 tokens).  `value` is the algorithmic HBM bytes of both passes divided by the measured time, with all
inputs resident in HBM.  The same run also reports the grouped w8a8 GEMM (32 local experts, 8192 rows,
hidden 7168, intermediate 2048) in TOPS and whole fused layers in microseconds.

Every timed region is a HIP graph replayed on torch's current stream and bracketed by HIP events on that
stream; inside a graph the operator is issued several times on rotating buffer sets, so that no pass finds
its inputs in the 256 MB last-level cache.  All launches go through the C ABI (libcam_mi355x.so).
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12      # B/s, MI355X HBM3E
INT8_PEAK = 5.0e15     # op/s, MI355X dense int8 MFMA


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


def graph_of(fn):
    fn()  # warm: first-use initialisation outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g


def time_graph(g, replays, warmup):
    for _ in range(warmup):
        g.replay()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / replays  # seconds per replay


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--skip-gemm", action="store_true")
    ap.add_argument("--skip-layer", action="store_true")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--only", default="", help="comma list of sections: dispatch,combine,gemm,layer")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build is single-GPU; every figure is measured on one MI355X. "
              "--gpus %d is not supported (expert-parallel exchange over xGMI is design-only)." % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    only = set(s for s in args.only.split(",") if s)

    def want(section):
        return not only or section in only

    import umdk_original_amd as cam
    from umdk_original_amd import _lib, synth

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(dev)
    log("device: %s, %d CUs" % (props.name, props.multi_processor_count))
    NBUF = 4   # rotating buffer sets
    ROT = 16   # passes per graph (buffer set = pass % NBUF): one replay = ROT steps, which amortises
               # the ~8 us a graph launch costs
    replays = max(1, (args.steps + ROT - 1) // ROT)
    warm = max(1, (args.warmup + ROT - 1) // ROT)

    result = {}
    kernels = {}

    # ------------------------------------------------------------------ counter calibration (on request)
    if "copy" in only:
        # A plain device-to-device copy of known size: 256 MiB read + 256 MiB written per launch.  Profiling
        # runs include it so that FETCH_SIZE / WRITE_SIZE readings can be scaled by what they show here.
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        log("copy calibration: 5 launches, 268435456 B read + 268435456 B written each")
        del src, dst

    # ------------------------------------------------------------------ dispatch (config 2)
    T, H, E, K = 4096, 7168, 256, 8
    A = T * K
    ids64, gate_w = synth.sigmoid_zipf_routing(T, E, K, seed=44)
    ids = ids64.to(torch.int32).to(dev)
    disp_bytes = synth.dispatch_bytes(T, H, K, E)
    comb_bytes = synth.combine_bytes(T, H, K)
    t_disp = t_plan = t_perm = t_comb = None

    if want("dispatch"):
        xs = [synth.normal_bf16(T, H, seed=44 + i).to(dev) for i in range(NBUF)]
        i32 = dict(dtype=torch.int32, device=dev)
        plan_bufs = [dict(pos=torch.empty((T, K), **i32), cnt=torch.empty(E, **i32), off=torch.empty(E, **i32),
                          roff=torch.empty(E, **i32), rcnt=torch.empty(E, **i32),
                          tpe=torch.empty(E, dtype=torch.int64, device=dev),
                          total=torch.empty(1, dtype=torch.int64, device=dev),
                          ws=torch.empty(1 << 18, dtype=torch.uint8, device=dev)) for _ in range(NBUF)]
        outs = [dict(rx=torch.empty((A, H), dtype=torch.int8, device=dev),
                     sc=torch.empty(A, dtype=torch.float32, device=dev),
                     info=torch.empty(3 * A, **i32)) for _ in range(NBUF)]

        def run_plan(i):
            p = plan_bufs[i % NBUF]
            _lib.call("MoeDispatchPlan", [ids, E, 1, 0, p["pos"], p["cnt"], p["off"], p["roff"], p["rcnt"], p["tpe"],
                                          p["total"]], workspace=p["ws"])

        def run_permute(i):
            p, o, i = plan_bufs[i % NBUF], outs[i % NBUF], i % NBUF
            _lib.call("MoeDispatchNormal", [xs[i], ids, p["off"], p["pos"], p["roff"], p["rcnt"], "", 1, 0, "", 1, 0,
                                            E, 2, 0, o["rx"], o["sc"], o["info"]])

        def disp_all():
            for i in range(ROT):
                run_plan(i)
                run_permute(i)

        def plan_only():
            for i in range(ROT):
                run_plan(i)

        def perm_only():
            for i in range(ROT):
                run_permute(i)

        t_disp = time_graph(graph_of(disp_all), replays, warm) / ROT
        t_plan = time_graph(graph_of(plan_only), replays, warm) / ROT
        t_perm = time_graph(graph_of(perm_only), replays, warm) / ROT
        log("dispatch: %.1f us (plan kernel %.1f us, permute+quant kernel %.1f us) -> %.0f GB/s = %.1f%% of HBM peak"
            % (t_disp * 1e6, t_plan * 1e6, t_perm * 1e6, disp_bytes / t_disp / 1e9, 100 * disp_bytes / t_disp / HBM_PEAK))
        perm_bytes = T * H * 2 + A * 4 + A * H + A * 4 + A * 12  # x, row ids, int8 rows, scales, triples
        kernels["dispatch_permute_quant"] = dict(bound="hbm", us=t_perm * 1e6, bytes=perm_bytes,
                                                 achieved=perm_bytes / t_perm / 1e9, peak=HBM_PEAK / 1e9, unit="GB/s",
                                                 frac=perm_bytes / t_perm / HBM_PEAK)
        kernels["dispatch_plan"] = dict(bound="latency", us=t_plan * 1e6)
        del xs, outs
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ combine (config 4)
    if want("combine"):
        import numpy as np
        plan = cam.moe_dispatch_plan(ids, E)
        ys = [synth.normal_bf16(A, H, seed=46 + i).to(dev) for i in range(NBUF)]
        # triples as the dispatch kernel writes them
        dummy = torch.empty((A, 1024), dtype=torch.bfloat16, device=dev)
        _, _, info = cam.moe_dispatch_normal(torch.zeros((T, 1024), dtype=torch.bfloat16, device=dev), ids,
                                             plan["send_offset"], plan["send_token_idx"], plan["recv_offset"],
                                             plan["recv_count"], A, E)
        del dummy
        gw = gate_w.to(dev)
        couts = [torch.empty((T, H), dtype=torch.bfloat16, device=dev) for _ in range(NBUF)]
        wss = [torch.empty(T * K * 4 + 256, dtype=torch.uint8, device=dev) for _ in range(NBUF)]

        def comb_all():
            for i in range(ROT):
                _lib.call("MoeCombineNormal", [ys[i % NBUF], info, plan["recv_count"], gw, None, "", 1, 0, "", 1, 0, E,
                                               0, couts[i % NBUF]], workspace=wss[i % NBUF])

        t_comb = time_graph(graph_of(comb_all), replays, warm) / ROT
        # The operator is two kernels (inverse map, then gather); the two halves exist as operators of their
        # own, which lets the gather kernel be timed alone.
        slots = [torch.empty((T, K), dtype=torch.int32, device=dev) for _ in range(NBUF)]

        def index_only():
            for i in range(ROT):
                _lib.call("MoeCombineIndex", [info, A, slots[i % NBUF]])

        def gather_only():
            for i in range(ROT):
                _lib.call("MoeCombineGather", [ys[i % NBUF], info, slots[i % NBUF], gw, couts[i % NBUF]])

        t_index = time_graph(graph_of(index_only), replays, warm) / ROT
        t_gather = time_graph(graph_of(gather_only), replays, warm) / ROT
        log("combine: %.1f us (inverse-map kernel %.1f us, gather kernel %.1f us) -> %.0f GB/s = %.1f%% of HBM peak"
            % (t_comb * 1e6, t_index * 1e6, t_gather * 1e6, comb_bytes / t_comb / 1e9,
               100 * comb_bytes / t_comb / HBM_PEAK))
        gather_bytes = A * H * 2 + A * 4 + A * 4 + T * H * 2  # rows, weights, map, output
        kernels["combine_gather"] = dict(bound="hbm", us=t_gather * 1e6, bytes=gather_bytes,
                                         achieved=gather_bytes / t_gather / 1e9, peak=HBM_PEAK / 1e9, unit="GB/s",
                                         frac=gather_bytes / t_gather / HBM_PEAK)
        kernels["combine_index"] = dict(bound="latency", us=t_index * 1e6)
        # decode-shaped variant
        Td = 128
        idd, gwd = synth.sigmoid_zipf_routing(Td, E, K, seed=47)
        idd32 = idd.to(torch.int32).to(dev)
        pland = cam.moe_dispatch_plan(idd32, E)
        _, _, infod = cam.moe_dispatch_normal(torch.zeros((Td, 1024), dtype=torch.bfloat16, device=dev), idd32,
                                              pland["send_offset"], pland["send_token_idx"], pland["recv_offset"],
                                              pland["recv_count"], Td * K, E)
        yd = [synth.normal_bf16(Td * K, H, seed=48 + i).to(dev) for i in range(NBUF)]
        od = [torch.empty((Td, H), dtype=torch.bfloat16, device=dev) for _ in range(NBUF)]
        gwd = gwd.to(dev)

        def comb_decode():
            for i in range(ROT):
                _lib.call("MoeCombineNormal", [yd[i % NBUF], infod, pland["recv_count"], gwd, None, "", 1, 0, "", 1, 0,
                                               E, 0, od[i % NBUF]], workspace=wss[i % NBUF])

        t_cd = time_graph(graph_of(comb_decode), replays, warm) / ROT
        cd_bytes = synth.combine_bytes(Td, H, K)
        log("combine decode (T=128): %.2f us -> %.0f GB/s" % (t_cd * 1e6, cd_bytes / t_cd / 1e9))
        result["combine_decode"] = dict(tokens=Td, us=t_cd * 1e6, gb_per_s=cd_bytes / t_cd / 1e9, bytes=cd_bytes)
        del ys, couts
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ grouped GEMM (config 3)
    if want("gemm") and not args.skip_gemm:
        G, I, rows = 32, 2048, 8192
        sizes = synth.zipf_group_sizes(G, rows, seed=45)
        gl = torch.cumsum(sizes, 0).to(dev)
        a = synth.uniform_int8((rows, H), 45).to(dev)
        xsc = synth.channel_scales((rows,), 451, 0.005, 0.05).to(dev)
        gen = torch.Generator(device=dev).manual_seed(452)
        w1 = torch.randint(-127, 128, (G, H, 2 * I), generator=gen, dtype=torch.int8, device=dev)
        w2 = torch.randint(-127, 128, (G, I, H), generator=gen, dtype=torch.int8, device=dev)
        w1p = cam.prepack_weight(w1, True)
        w2p = cam.prepack_weight(w2, False)
        del w1, w2
        w1s = synth.channel_scales((G, 2 * I), 453).to(dev)
        w2s = synth.channel_scales((G, H), 454).to(dev)
        y = torch.empty((rows, I), dtype=torch.int8, device=dev)
        ysc = torch.empty(rows, dtype=torch.float32, device=dev)
        out = torch.empty((rows, H), dtype=torch.bfloat16, device=dev)
        ws1 = torch.empty(rows * I * 4 + (1 << 16), dtype=torch.uint8, device=dev)
        ws2 = torch.empty(1 << 16, dtype=torch.uint8, device=dev)

        def gmm1():
            _lib.call("GroupedMatmulSwigluQuant", [a, xsc, [w1p], [w1s], gl, 0, y, ysc], workspace=ws1)

        def gmm2():
            _lib.call("GroupedMatmulDequant", [y, ysc, [w2p], [w2s], gl, 0, out], workspace=ws2)

        def both():
            gmm1()
            gmm2()

        n = max(10, args.steps // 4)
        t_g1 = time_graph(graph_of(gmm1), n, 5)
        t_g2 = time_graph(graph_of(gmm2), n, 5)
        t_g = time_graph(graph_of(both), n, 5)
        ops1 = 2 * rows * H * 2 * I
        ops2 = 2 * rows * I * H
        gemm_bytes = G * (H * 2 * I + I * H) + rows * H + 2 * rows * I + rows * H * 2
        log("grouped GEMM: %.1f us total (GMM1 op %.1f us, GMM2 op %.1f us) -> %.0f TOPS = %.1f%% of int8 peak; "
            "%.0f GB/s" % (t_g * 1e6, t_g1 * 1e6, t_g2 * 1e6, (ops1 + ops2) / t_g / 1e12,
                           100 * (ops1 + ops2) / t_g / INT8_PEAK, gemm_bytes / t_g / 1e9))
        result["grouped_gemm"] = dict(us=t_g * 1e6, tops=(ops1 + ops2) / t_g / 1e12, ops=ops1 + ops2,
                                      frac_int8_peak=(ops1 + ops2) / t_g / INT8_PEAK, gb_per_s=gemm_bytes / t_g / 1e9,
                                      rows=rows, experts=G, empty_experts=int((sizes == 0).sum()),
                                      max_rows_per_expert=int(sizes.max()))
        kernels["gmm1_swiglu_quant"] = dict(bound="mfma", us=t_g1 * 1e6, ops=ops1, achieved=ops1 / t_g1 / 1e12,
                                            peak=INT8_PEAK / 1e12, unit="TOP/s", frac=ops1 / t_g1 / INT8_PEAK,
                                            note="operator time: tile table + GEMM + re-quant kernels")
        kernels["gmm2_dequant"] = dict(bound="mfma", us=t_g2 * 1e6, ops=ops2, achieved=ops2 / t_g2 / 1e12,
                                       peak=INT8_PEAK / 1e12, unit="TOP/s", frac=ops2 / t_g2 / INT8_PEAK,
                                       note="operator time: tile table + GEMM kernels")
        del w1p, w2p, a, y, out, ws1
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ whole fused layers
    if want("layer") and not args.skip_layer:
        layers = {}
        for name, (Tl, Hl, El, Kl, Il) in {
            "qwen3_235b_shape_prefill_w8a8": (8192, 4096, 128, 8, 1536),
            "qwen3_235b_shape_decode_w8a8": (128, 4096, 128, 8, 1536),
            "cpu_golden_config": (128, 1024, 8, 2, 512),
        }.items():
            idl, gl_w = synth.sigmoid_zipf_routing(Tl, El, Kl, seed=47) if El > 8 else \
                synth.softmax_topk_routing(Tl, El, Kl, seed=43)
            gen = torch.Generator(device=dev).manual_seed(471)
            w1 = cam.prepack_weight(torch.randint(-127, 128, (El, Hl, 2 * Il), generator=gen, dtype=torch.int8,
                                                  device=dev), True)
            w2 = cam.prepack_weight(torch.randint(-127, 128, (El, Il, Hl), generator=gen, dtype=torch.int8,
                                                  device=dev), False)
            w1s = synth.channel_scales((El, 2 * Il), 472).to(dev)
            w2s = synth.channel_scales((El, Hl), 473).to(dev)
            xl = synth.normal_bf16(Tl, Hl, seed=474).to(dev)
            idl32 = idl.to(torch.int32).to(dev)
            gl_w = gl_w.to(dev)
            outl = torch.empty((Tl, Hl), dtype=torch.bfloat16, device=dev)
            etn = torch.empty(El, dtype=torch.int64, device=dev)
            st, ws_bytes, msg = _lib.phase1("FusedDeepMoe", [xl, idl32, [w1], [w1s], [w2], [w2s], gl_w, None, None, "",
                                                             1, 0, El, 1, 0, 0, 0, outl, etn])
            assert st == 0, msg
            wsl = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

            def layer():
                _lib.call("FusedDeepMoe", [xl, idl32, [w1], [w1s], [w2], [w2s], gl_w, None, None, "", 1, 0, El, 1, 0,
                                           0, 0, outl, etn], workspace=wsl)

            n = max(10, args.steps // 4)
            t_l = time_graph(graph_of(layer), n, 5)
            ops = synth.gemm_ops(Tl * Kl, Hl, Il)
            log("fused layer %s: %.1f us (%.0f TOPS)" % (name, t_l * 1e6, ops / t_l / 1e12))
            layers[name] = dict(us=t_l * 1e6, tokens=Tl, hidden=Hl, experts=El, top_k=Kl, intermediate=Il,
                                tops=ops / t_l / 1e12, dtype="int8 weights and activations (w8a8)")
            del w1, w2, wsl, xl, outl
            torch.cuda.empty_cache()
        result["fused_layer_us"] = layers

    # ------------------------------------------------------------------ CPU baseline (oracle, bounded sample)
    cpu = None
    if not args.skip_cpu and want("dispatch") and want("combine"):
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import cam_oracle
        import numpy as np
        Ts = 1024  # a quarter of the workload's tokens, same H / E / K
        ids_s = ids64[:Ts].numpy()
        x_s = synth.bf16_bits(synth.normal_bf16(Ts, H, seed=44))
        y_s = synth.bf16_bits(synth.normal_bf16(Ts * K, H, seed=46))
        gw_s = gate_w[:Ts].numpy()
        t0 = time.perf_counter()
        reps = 0
        while True:
            _, cnt, _ = cam_oracle.layout(ids_s, E, 1)
            off, _ = cam_oracle.offsets(cnt, Ts)
            pos = cam_oracle.send_token_idx(ids_s, E)
            cam_oracle.dispatch(x_s, ids_s, off, pos, E, 1, Ts * K)
            row_of = cam_oracle.rows_from_pos(ids_s, off, pos, E)
            cam_oracle.combine(y_s, row_of, gw_s)
            reps += 1
            el = time.perf_counter() - t0
            if el > 12.0:
                break
        sample_bytes = synth.dispatch_bytes(Ts, H, K, E) + synth.combine_bytes(Ts, H, K)
        cpu = dict(value=sample_bytes * reps / el / 1e9, unit="GB/s", cores=cam_oracle.num_threads(), kind="port",
                   sample="%d of %d tokens of the same dispatch+combine workload (H=%d, E=%d, top-%d), %d passes in "
                          "%.1f s, OpenMP over rows" % (Ts, T, H, E, K, reps, el))
        log("cpu baseline: %.2f GB/s on %d threads" % (cpu["value"], cpu["cores"]))

    # ------------------------------------------------------------------ the JSON line
    line = {
        "metric": "dispatch+combine HBM GB/s; w8a8 grouped GEMM TOPS; us per MoE layer",
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "dtype_detail": "dispatch: bf16 in, fp32 scale arithmetic, int8 out; GEMM: int8 x int8 -> int32, fp32 "
                        "dequantisation; combine: fp32 accumulate -> bf16",
        "data": "synthetic",
        "config": {
            "workload": "dispatch: 4096 tokens x 7168 bf16, 256 experts, top-8 (sigmoid + Zipf(1.1)-biased routing), "
                        "per-token int8 quant + fp32 scales; then combine: 32768 bf16 rows x 7168 -> 4096 tokens",
            "tokens": T, "hidden": H, "experts": E, "top_k": K,
            "dispatch_bytes": disp_bytes, "combine_bytes": comb_bytes,
            "timing": "HIP graph replays (%d passes each) bracketed by HIP events on the launch stream; %d rotating "
                      "buffer sets" % (ROT, NBUF),
        },
    }
    if t_disp is not None and t_comb is not None:
        total_t = t_disp + t_comb
        line["value"] = (disp_bytes + comb_bytes) / total_t / 1e9
        line["ms_per_step"] = total_t * 1e3
        line["dispatch"] = dict(us=t_disp * 1e6, gb_per_s=disp_bytes / t_disp / 1e9, frac_hbm_peak=disp_bytes / t_disp / HBM_PEAK)
        line["combine"] = dict(us=t_comb * 1e6, gb_per_s=comb_bytes / t_comb / 1e9, frac_hbm_peak=comb_bytes / t_comb / HBM_PEAK)
        dom = "combine_gather" if kernels["combine_gather"]["us"] >= kernels["dispatch_permute_quant"]["us"] \
            else "dispatch_permute_quant"
        k = kernels[dom]
        # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by what the same
        # counter shows for a 256 MiB device copy (x2.000 and x1.000): profiles/dispatch_combine_c2_c4.md.
        measured_traffic = {"combine_gather": 539.0e6, "dispatch_permute_quant": 295.9e6}
        line["roofline"] = {"kernel": dom, "bound": "hbm", "achieved": k["achieved"], "peak": HBM_PEAK / 1e9,
                            "unit": "GB/s", "frac": k["frac"], "traffic": measured_traffic[dom], "us": k["us"],
                            "bytes": k["bytes"]}
    else:
        line["value"] = None
        line["ms_per_step"] = None
    line["kernels"] = kernels
    line.update(result)
    if cpu is not None:
        line["cpu_baseline"] = cpu
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
