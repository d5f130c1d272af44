#!/usr/bin/env python3
"""Benchmark of the MoE-layer forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2_mixtral] [--no-cpu-baseline]

A step is one forward pass of the layer over one batch of seeded synthetic tokens that already sit
in HBM.  Prints ONE JSON line: whole-layer tokens/s, the roofline figure of the dominant kernel
(the grouped up-projection, bf16 MFMA bound) measured with events on the library's own stream
inside the timed forwards, per-stage figures, a sampled parity check, and a CPU baseline (the
C restatement of the reference's CPU-style path, timed on a bounded token sample).
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3
PEAK_HBM_GBPS = 8000.0



def profiled_traffic(cfg_name):
    """HBM / fabric bytes per launch of the dominant kernel (the up product) from the tracked rocprofv3 --pmc summary of
    this workload, profiles/experts_bf16_<workload>_pmc.txt: the line `traffic_bytes_per_launch up <bytes>`
    (FETCH_SIZE x copy-kernel factor + WRITE_SIZE).  The counters cannot be read inside a timed run, so the figure
    belongs to the commit the summary was made at; None when there is no summary for the workload."""
    path = os.path.join(ROOT, "profiles", f"experts_bf16_{cfg_name}_pmc.txt")
    try:
        with open(path) as f:
            for line in f:
                parts = line.split()
                if len(parts) == 3 and parts[0] == "traffic_bytes_per_launch" and parts[1] == "up":
                    return float(parts[2]), os.path.relpath(path, ROOT)
    except OSError:
        pass
    return None, None



def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c2_mixtral")
    ap.add_argument("--seed", type=int, default=20251)
    ap.add_argument("--override", default="", help="replace dimensions of the named configuration, e.g. T=1024,K=8 "
                                                    "(experiments; the default line is the configuration as named)")
    ap.add_argument("--router", default="exact", choices=["exact", "fast"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-parity", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target CPU-baseline sample duration")
    ap.add_argument("--no-mfma-probe", action="store_true",
                    help="skip the matrix-core ceiling probe (two runs of about 1 s with no memory traffic)")
    ap.add_argument("--no-backward", action="store_true", help="skip the backward-pass figures")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain 256 MiB device copy (convert_kernel fp32->fp32) three times, so that "
                         "FETCH_SIZE / WRITE_SIZE of a profiled run can be scaled by a kernel of known traffic")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus above 1 is not supported (no collectives in this path)",
              file=sys.stderr)
        sys.exit(2)

    P = importlib.import_module("omega-ai_amd")
    L = importlib.import_module("omega-ai_amd._lib")
    C = P.configs
    cfg = C.CONFIGS[a.config]
    if a.override:
        import dataclasses
        kw = {k: int(v) for k, v in (item.split("=") for item in a.override.split(","))}
        cfg = dataclasses.replace(cfg, name=cfg.name + "[" + a.override + "]", **kw)
    ctx = P.Context(0)
    layer = P.MoELayer(cfg.d, cfg.H, cfg.E, cfg.K, renorm=cfg.renorm, nShared=cfg.Es, bias=cfg.has_gate_bias, ctx=ctx,
                       dtype=cfg.dtype, router_mode=a.router, T_max=cfg.T)
    layer.init_synthetic(a.seed, C, cfg)
    x = P.DeviceBuffer(ctx, (cfg.T, cfg.d), cfg.dtype)
    x.fill_normal(a.seed, C.STREAM_X, C.tensor_std(cfg, "x"))
    ctx.sync()

    if a.copy_calibration:
        n = 64 * 1024 * 1024
        src, dst = P.DeviceBuffer(ctx, (n,), "f32"), P.DeviceBuffer(ctx, (n,), "f32")
        for _ in range(3):
            ctx.check(ctx.lib.omega_hip_convert(ctx.handle, dst.ptr, L.DTYPE_F32, src.ptr, L.DTYPE_F32, n))
        ctx.sync()
        src.free()
        dst.free()
    for _ in range(a.warmup):
        layer.forward(x)
    ctx.sync()
    layer.set_profiling(True)
    t0 = time.perf_counter()
    for _ in range(a.steps):
        layer.forward(x)
    ctx.sync()
    t1 = time.perf_counter()
    stage_ms, n_prof = layer.get_profile()
    layer.set_profiling(False)
    ms_per_step = (t1 - t0) * 1e3 / a.steps
    tokens_per_s = cfg.T / (ms_per_step * 1e-3)

    b = 2 if cfg.dtype == "bf16" else 4
    rows = cfg.P + cfg.Es * cfg.T
    up_flops = 4.0 * cfg.d * cfg.H * rows
    down_flops = 2.0 * cfg.d * cfg.H * rows
    peak = PEAK_BF16_TFLOPS if cfg.dtype == "bf16" else PEAK_F32_TFLOPS
    up_tflops = up_flops / (stage_ms["experts_up"] * 1e-3) / 1e12
    down_tflops = down_flops / (stage_ms["experts_down"] * 1e-3) / 1e12
    # algorithmic bytes of the bandwidth-bound stages
    router_bytes = cfg.T * cfg.d * b + cfg.E * cfg.d * b + cfg.P * 8
    dispatch_bytes = 2 * cfg.P * cfg.d * b + cfg.P * 12
    combine_bytes = cfg.P * cfg.d * b + cfg.T * cfg.d * b + cfg.P * 8
    # bytes these kernels cannot avoid moving as the path is specified (not the algorithmic figures above): the gather
    # reads every token row once and writes it K times (+ once per batch for the shared experts' packed copy); the
    # combine reads the expert outputs as the fp32 rows the composition keeps them in
    # (bf16 layers whose up product fetches the rows of x itself write no gathered copy: the dispatch stage then moves
    #  index data only, and its byte fractions say nothing - they are left out)
    on_load = layer.gather_on_load()
    dispatch_real = cfg.T * cfg.d * b + cfg.P * cfg.d * b + (cfg.T * cfg.d * b if cfg.Es else 0) + cfg.P * 12
    combine_real = rows * cfg.d * 4 + cfg.T * cfg.d * b + cfg.P * 8
    # block form (out = x + layer(rmsnorm(x)), the widening next to the path): whole call and its pre-norm kernel
    outb = P.DeviceBuffer(ctx, (cfg.T, cfg.d), cfg.dtype)
    block_ms = layer.time_stage(L.STAGE_FORWARD_BLOCK, x, cfg.T, out=outb, warmup=2, iters=a.steps)
    rms_ms = layer.time_stage(L.STAGE_RMS, x, cfg.T, warmup=2, iters=20)
    outb.free()
    index_ms = layer.time_stage(L.STAGE_INDEX, x, cfg.T, warmup=2, iters=20)

    # what the matrix cores sustain on this device with nothing else going on: the nominal-clock rate with constant
    # operands and the rate under the power cap with random bf16 operands (the realistic ceiling for a GEMM)
    probe = None
    if cfg.dtype == "bf16" and not a.no_mfma_probe:
        import ctypes
        probe_lib = ctypes.CDLL(os.path.join(ROOT, "bench_probe.so"))   # built by __graft_entry__.build()
        probe_lib.bench_probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
        ctx.sync()
        v = ctypes.c_float()
        probe = {}
        for key, rnd in (("constant_operands_TFLOP/s", 0), ("random_operands_TFLOP/s", 1)):
            st = probe_lib.bench_probe_mfma(0, rnd, 400, ctypes.byref(v))
            if st != 0:
                raise RuntimeError(f"bench_probe_mfma: HIP error {st}")
            probe[key] = v.value
        probe["frac_of_random_operand_rate"] = up_tflops / probe["random_operands_TFLOP/s"]

    # backward pass (the widening behind the path): after a plain forward (h1 / h3 recomputed) and in training mode
    # (the forward pass keeps them); algorithmic work = input and weight gradients of the three products, 12*d*H per row
    backward = None
    if not a.no_backward:
        gbuf = P.DeviceBuffer(ctx, (cfg.T, cfg.d), cfg.dtype)
        gbuf.fill_normal(a.seed, 900, 1.0)
        dxb = P.DeviceBuffer(ctx, (cfg.T, cfg.d), cfg.dtype)
        outf = layer.forward(x)
        bw_ms = layer.time_backward(x, gbuf, cfg.T, dxb, warmup=2, iters=max(3, a.steps // 2))
        layer.set_training(True)
        fwd_train_ms = layer.time_stage(L.STAGE_FORWARD, x, cfg.T, out=outf, warmup=2, iters=max(3, a.steps // 2))
        layer.forward(x)
        bw_train_ms = layer.time_backward(x, gbuf, cfg.T, dxb, warmup=2, iters=max(3, a.steps // 2))
        layer.set_training(False)
        # optimiser step: AdamW on every parameter (learning rate 0: same traffic, weights unchanged), wall clock
        # around a synchronised batch of calls; 30 bytes move per expert parameter of a bf16 layer (fp32 master, two
        # moments and gradient read; master, moments and the bf16 weight written), 28 of an fp32 layer
        layer.updateAdamW(0.0, 1, weight_decay=0.0)
        ctx.sync()
        t_up = time.perf_counter()
        for i in range(3):
            layer.updateAdamW(0.0, 2 + i, weight_decay=0.0)
        ctx.sync()
        adamw_ms = (time.perf_counter() - t_up) / 3 * 1e3
        n_params = 3.0 * (cfg.E + cfg.Es) * cfg.H * cfg.d + cfg.E * cfg.d
        adamw_bytes = n_params * (30.0 if cfg.dtype == "bf16" else 28.0)
        bw_flops = 12.0 * cfg.d * cfg.H * rows
        backward = {"what": "omega_moe_backward: dx and all parameter gradients (fp32) for one dout",
                    "ms": bw_ms, "algorithmic_TFLOP/s": bw_flops / (bw_ms * 1e-3) / 1e12,
                    "training_mode": {"forward_ms": fwd_train_ms, "backward_ms": bw_train_ms,
                                      "algorithmic_TFLOP/s": bw_flops / (bw_train_ms * 1e-3) / 1e12,
                                      "frac_mfma": bw_flops / (bw_train_ms * 1e-3) / 1e12 / peak,
                                      "fwd+bwd_tokens/s": cfg.T / ((fwd_train_ms + bw_train_ms) * 1e-3)},
                    "adamw_update": {"ms": adamw_ms, "parameters": n_params, "bound": "hbm",
                                     "achieved_GB/s": adamw_bytes / (adamw_ms * 1e-3) / 1e9, "frac_hbm": adamw_bytes / (adamw_ms * 1e-3) / 8e12}}
        gbuf.free()
        dxb.free()

    traffic, traffic_src = profiled_traffic(C.CONFIGS[a.config].name if not a.override else "")
    res = {
        "metric": "MoE-layer fwd tokens/s (Mixtral shape, bf16); MFMA util %; dispatch GB/s",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": cfg.dtype, "data": "synthetic (seeded counter-based normal generator, generated in HBM)",
        "config": {"workload": f"{cfg.name}: T={cfg.T} ({cfg.batch}x{cfg.seq}) d={cfg.d} E={cfg.E} K={cfg.K} H={cfg.H} "
                               f"Es={cfg.Es} renorm={int(cfg.renorm)} {cfg.dtype}, fp32 accumulate",
                   "router_mode": a.router, "seed": a.seed},
        "roofline": {"bound": "mfma", "kernel": ("experts_up4_kernel" if cfg.dtype == "bf16" else "experts_f32_kernel<true>") + " (up product): a = silu(xg W1^T) * (xg W3^T)",
                     "achieved": up_tflops, "peak": peak, "unit": "TFLOP/s", "frac": up_tflops / peak,
                     "algorithmic_flops_per_launch": up_flops, "avg_launch_ms": stage_ms["experts_up"],
                     "traffic": traffic, "traffic_source": traffic_src,
                     "mfma_only_probe": probe},
        "block_form": {"what": "out = x + layer(rmsnorm(x)) in one call (omega_moe_forward_block)", "ms_per_step": block_ms,
                       "tokens/s": cfg.T / (block_ms * 1e-3), "prenorm_kernel_ms": rms_ms},
        "backward": backward,
        "stages": {
            "avg_ms": stage_ms, "profiled_forwards": n_prof,
            "experts_down": {"TFLOP/s": down_tflops, "frac_mfma": down_tflops / peak},
            "experts_total_frac_mfma": (up_flops + down_flops) / ((stage_ms["experts_up"] + stage_ms["experts_down"]) * 1e-3) / 1e12 / peak,
            "router": {"GB/s": router_bytes / (stage_ms["router"] * 1e-3) / 1e9, "frac_hbm": router_bytes / (stage_ms["router"] * 1e-3) / 1e9 / PEAK_HBM_GBPS},
            "dispatch": {"rows": "fetched from x by the loads of the up product (no gathered copy)" if on_load
                                 else "gathered copy written by the dispatch launch",
                         "GB/s": None if on_load else dispatch_bytes / (stage_ms["dispatch"] * 1e-3) / 1e9,
                         "frac_hbm": None if on_load else dispatch_bytes / (stage_ms["dispatch"] * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                         "frac_hbm_real_traffic": None if on_load else dispatch_real / (stage_ms["dispatch"] * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                         "index_only_ms": index_ms},
            "combine": {"GB/s": combine_bytes / (stage_ms["combine"] * 1e-3) / 1e9,
                        "frac_hbm": combine_bytes / (stage_ms["combine"] * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                        "frac_hbm_real_traffic": combine_real / (stage_ms["combine"] * 1e-3) / 1e9 / PEAK_HBM_GBPS},
        },
    }

    need_host = not (a.no_parity and a.no_cpu_baseline)
    if need_host:
        from oracle import oracle as O
        from oracle import oracle_np as N
        G = cfg.E + cfg.Es
        xh = x.to_numpy()
        Wg = layer._download_weight(L.W_GATE, 0, (cfg.E, cfg.d))
        bg = C.zipf_gate_bias(cfg, a.seed)
        W1 = np.empty((G, cfg.H, cfg.d), np.float32)
        W3 = np.empty((G, cfg.H, cfg.d), np.float32)
        W2 = np.empty((G, cfg.d, cfg.H), np.float32)
        for g in range(G):
            W1[g] = layer._download_weight(L.W_W1, g, (cfg.H, cfg.d))
            W3[g] = layer._download_weight(L.W_W3, g, (cfg.H, cfg.d))
            W2[g] = layer._download_weight(L.W_W2, g, (cfg.d, cfg.H))
        bf = cfg.dtype == "bf16"
        if not a.no_parity:
            out = layer.forward(x).to_numpy()
            r = layer.routing()
            p = O.softmax(O.gate(xh, Wg, bg))
            ids, w = O.topk(p, cfg.K, cfg.renorm)
            counts, offsets, dst, src = O.dispatch(ids, cfg.E)
            # a token of every row tile of every expert (first row of the tile, last row of the expert), so that the
            # sample touches every row tile the grouped products schedule, plus 16 evenly spaced tokens
            bm = 256 if bf else 64
            pick = set(np.linspace(0, cfg.T - 1, 16).astype(np.int64).tolist())
            for e in range(cfg.E):
                n, l0 = int(counts[e]), int(offsets[e])
                if n:
                    Mg, nblk = -(-n // bm), -(-n // 32)
                    qb, nhi = divmod(nblk, Mg)
                    pick.update(int(src[l0 + 32 * (mt * qb + min(mt, nhi))]) for mt in range(Mg))
                    pick.add(int(src[l0 + n - 1]))
            if cfg.Es:
                pick.update(range(0, cfg.T, bm))
            tok = np.array(sorted(pick), np.int32)
            from concurrent.futures import ThreadPoolExecutor
            parts = [p for p in np.array_split(tok, min(8, len(tok))) if len(p)]
            with ThreadPoolExecutor(len(parts)) as ex:
                ref = np.concatenate(list(ex.map(
                    lambda part: O.moe_tokens(xh, ids, w, W1, W3, W2, cfg.E, cfg.Es, part, bf16=bf), parts)))
            res["parity"] = {
                "ids_bit_exact": bool(np.array_equal(r["ids"], ids)), "weights_bit_exact": bool(np.array_equal(r["w"], w)),
                "counts_bit_exact": bool(np.array_equal(r["counts"], counts)),
                "perm_bit_exact": bool(np.array_equal(r["dst"], dst) and np.array_equal(r["src_row"], src)),
                "out_rel_l2_sampled_tokens": N.rel_l2(out[tok], ref), "sampled_tokens": int(len(tok)),
                "tolerance": 1e-2 if bf else 1e-5}
        if not a.no_cpu_baseline:
            n_threads = min(16, os.cpu_count() or 1)
            Ts, secs = min(16, cfg.T), 0.0
            while True:
                secs, _ = O.cpu_baseline_forward(np.ascontiguousarray(xh[:Ts]), Wg, bg, W1, W3, W2, cfg.K, cfg.renorm,
                                                 cfg.Es, n_threads)
                if secs >= a.cpu_seconds / 3 or Ts >= cfg.T:
                    break
                Ts = int(min(cfg.T, max(Ts * 2, Ts * a.cpu_seconds / max(secs, 1e-3))))
            res["cpu_baseline"] = {
                "value": Ts / secs, "unit": "tokens/s", "cores": min(n_threads, G), "kind": "port",
                "sample": f"C restatement (no JDK) of the reference's CPU-style path (column-major j8->p->i sgemm, "
                          f"one task per expert, {n_threads}-thread pool): first {Ts} tokens of the same batch, all "
                          f"{G} experts' weights, fp32 arithmetic on the bf16-rounded values, {secs:.2f} s",
                "host_cpus": os.cpu_count()}
    print(json.dumps(res))


if __name__ == "__main__":
    main()
