#!/usr/bin/env python3
"""Benchmark of the routed-expert MoE layer on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W]
                  [--workload headline|prefill|decode|verify|q4k_prefill|q4k_decode|stack|ggmix_decode|ggmix_verify|
                              v2_prefill|v2_decode|v2_verify]

One step = one pass of the MoE layer (moe_forward) over one batch of synthetic input that is
already resident in HBM.  Prints ONE JSON line: whole-layer throughput, the roofline figure of the
dominant kernel (timed live with HIP events on the launch stream) and the CPU oracle timed on the
host cores on a bounded sample of the same workload.

`headline` (the default) is the prefill chunk T=16384 as the primary figure, with the decode T=1
figure of the same layer shape measured in the same run and reported under "decode_T1".
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA
D, MID, E, K = 3072, 768, 512, 10
LIB_OPTIONS = []              # (option id, value) pairs of --opt, applied to every context
GG_MIX_TYPES = None           # --gg-types: ggml types (gate/up, down, shared expert) of the ggmix_* workloads
CPU_BUDGET_S = 12.0            # the cpu_baseline leg stops starting new work after this long
# Counters cannot be read from inside this process: the HBM bytes per launch of the dominant kernel (read + written)
# come from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summaries under profiles/ (the table's "total MB" column of
# the named kernel's line); a workload or shape without such a summary reports null.
PMC_TRAFFIC = {("prefill", "q4cp", 16384): ("prefill_q4cp_T16384_hbm_traffic.txt", "k_moe_gemm_q4cp<true", "max"),
               ("decode", "q4cp", 1): ("decode_q4cp_T1_hbm_traffic.txt", "k_dec_gu", "max"),
               ("verify", "q4cp", 20): ("verify_q4cp_T20_hbm_traffic.txt", "k_dec_gu", "max"),
               ("decode", "q4k", 1): ("decode_q4k_T1_hbm_traffic.txt", "k_dec4k_gu", "max"),
               ("prefill", "q4k", 8192): ("prefill_q4k_T8192_hbm_traffic.txt", "k_moe_gemm_q4cp<true", "max")}


_timing_capi = False


def timing_capi():
    """A second binding of the C ABI, on the library's timing twin (the same sources built with -DMOE_TIMING_HOOKS, the
    only build in which a stage's launches can be left out), or None when that library is not there.  Used to time the
    dominant launch of a small-batch call as the difference of two step loops; the step loop that gives `value` runs
    on the default library."""
    global _timing_capi
    if _timing_capi is False:
        from gfx1151_engine_amd import LIB_TIMING, capi
        path = os.environ.get("MI355MOE_LIB_TIMING") or (None if os.environ.get("MI355MOE_LIB") else LIB_TIMING)
        _timing_capi = capi.second_binding(path) if path and os.path.exists(path) else None
    return _timing_capi


def pmc_traffic(kind, fmt, T):
    """HBM bytes per launch of the workload's dominant kernel from its committed counter summary, or None."""
    ent = PMC_TRAFFIC.get((kind, fmt, T))
    if not ent:
        return None
    path = os.path.join(ROOT, "profiles", ent[0])
    try:
        vals = [float(ln.split()[-1]) for ln in open(path) if ln.startswith(ent[1]) and len(ln.split()) >= 7]
    except (OSError, ValueError):
        return None
    return max(vals) * 1e6 if vals else None  # routed and shared-expert launches of one kernel: the larger grid


def cpu_leg(kind, layer, xs, ids, cnt, m, T, eb, budget=CPU_BUDGET_S):
    """The CPU restatement of src/ref.cpp Model::moe (OpenMP over rows) on a bounded sample of the
    same workload, and the GPU result's distance from it on that sample."""
    import numpy as np
    import torch
    from oracle import oracle as O
    ol = O.layer_from_device(layer)
    y = torch.empty((T, D), dtype=torch.float32, device="cuda")
    if kind == "prefill":
        # tokens routed to the hottest expert first, then tokens in batch order, in chunks of 256
        hot = int(np.argmax(cnt))
        order = np.concatenate([np.where((ids == hot).any(1))[0][:64], np.arange(T)])
        _, first = np.unique(order, return_index=True)
        order = order[np.sort(first)]
        m.forward(0, xs[0], y)
        yg_all = y.cpu().numpy()
        xh = xs[0].cpu().numpy()
        done, cpu_s, err = 0, 0.0, 0.0
        while cpu_s < budget and done < len(order):
            toks = order[done:done + 256]
            t0 = time.perf_counter()
            yo, _, _ = O.moe_layer(ol, xh[toks])
            cpu_s += time.perf_counter() - t0
            err = max(err, float(np.abs(yg_all[toks].astype(np.float64) - yo).max() / np.abs(yo).max()))
            done += len(toks)
        out = {"value": round(done / cpu_s, 3), "unit": "tok/s",
               "sample": f"{done} of the batch's {T} tokens (64 of the hottest expert's first), chunks of 256"}
    else:
        done, cpu_s, err, nbytes = 0, 0.0, 0.0, 0
        while cpu_s < budget and done < 4096:
            xg = xs[done % len(xs)]
            xh = xg.cpu().numpy()
            t0 = time.perf_counter()
            yo, io, _ = O.moe_layer(ol, xh)
            cpu_s += time.perf_counter() - t0
            if done < len(xs):
                m.forward(0, xg, y)
                err = max(err, float(np.abs(y.cpu().numpy().astype(np.float64) - yo).max() / np.abs(yo).max()))
            nbytes += (int(np.unique(io[:, :K]).size) + 1) * eb + E * D * 4 + D * 4 + T * 2 * D * 4
            done += 1
        out = {"value": round(nbytes / cpu_s / 1e9, 4), "unit": "GB/s",
               "sample": f"{done} steps of {T} token(s), same inputs as the GPU steps"}
    out.update({"cores": O.num_threads(), "kind": "port", "seconds": round(cpu_s, 3),
                "what": "OpenMP restatement of src/ref.cpp Model::moe (fp64 dot products), weights dequantised row by row",
                "max_abs_rel_vs_gpu": err})
    return out


def measure(wl, steps, warmup, tokens=0, nlayers_arg=48, cpu=True, opts=(), cpu_budget=CPU_BUDGET_S, codebook="zp8"):
    import numpy as np
    import torch
    from gfx1151_engine_amd import capi, workloads as W
    from gfx1151_engine_amd import synth as S
    d, mid, k = D, MID, K
    # ggmix_*: GGUF layer in the reference checkpoints' type mix (Q5_K gate/up, Q8_0 down, Q8_0 shared expert) on the
    # general GEMV kernels
    # v2_*: hgn v2 layer (Hadamard-rotated i4r routed experts, q4cp shared expert)
    ggmix = wl.startswith("ggmix_")
    fmt = "q4k" if wl.startswith("q4k") or ggmix else "i4r" if wl.startswith("v2_") else "q4cp"
    gg_types = (GG_MIX_TYPES or (13, 8, 8)) if ggmix else (12, 12, 12)
    kind = wl.replace("q4k_", "").replace("ggmix_", "").replace("v2_", "")
    T = tokens or {"prefill": 16384 if fmt in ("q4cp", "i4r") else 8192, "decode": 1, "verify": 20, "stack": 1}[kind]
    nlayers = nlayers_arg if kind == "stack" else 1

    layers = [W.DeviceLayer(1000 + l, d, mid, E, k, fmt, gg_types=gg_types, codebook=codebook) for l in range(nlayers)]
    universal = fmt == "q4cp" and codebook == "universal"
    g = torch.Generator(device="cuda")
    g.manual_seed(99)
    extra = {}
    if kind == "prefill":
        x = torch.randn((T, d), device="cuda", generator=g).to(torch.bfloat16).to(torch.float32)
        bias, beta = W.calibrate_zipf(layers[0].router, x, k)
        layers[0].bias = bias
        xs = [x]
        extra["zipf_beta"] = round(beta, 4)
    elif kind == "verify":
        xs = [W.verify_batch(layers[0].router, d, T, seed=5 + i) for i in range(64)]
    else:
        # decode: rotate 64 different tokens so that no cache level can hold the experts of a step
        xs = [torch.randn((T, d), device="cuda", generator=g) for _ in range(64)]
    m = capi.Moe(d, mid, E, k, layers=nlayers, max_tokens=T)
    for l, L in enumerate(layers):
        L.register(m, l)
    for o, v in list(LIB_OPTIONS) + list(opts):
        m.set_option(o, v)
    y = torch.empty((T, d), dtype=torch.float32, device="cuda")

    def step(i):
        if kind == "stack":
            for l in range(nlayers):
                m.forward(l, xs[(i * nlayers + l) % len(xs)], y)
        else:
            m.forward(0, xs[i % len(xs)], y)

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    # the path the timed calls take: batches over 32 tokens on the grouped GEMM (a batch walked through the in-place
    # kernels 32 rows at a time would return right results and a meaningless figure)
    step(0)
    want = capi.PATH_BATCH if T > 32 else capi.PATH_SMALL
    if m.last_path() != want:
        raise SystemExit(f"bench.py: workload {kind!r} at {T} tokens took path {m.last_path()}, expected {want} (moe_last_path)")
    torch.cuda.synchronize()
    # whole-job timing: K steps between two synchronisations, HIP events on the launch stream
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        step(warmup + i)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms = e0.elapsed_time(e1) / steps

    # per-stage timing (HIP events recorded by the library between its kernels, same stream)
    m.profile(True)
    stage = {}
    nprof = max(5, min(steps, 20))
    for i in range(nprof):
        m.forward(i % nlayers, xs[i % len(xs)], y)
        for kk, v in m.profile_read().items():
            stage[kk] = stage.get(kk, 0.0) + v / nprof
    m.profile(False)
    # Batches of at most 32 tokens: a kernel takes about as long as an event pair's own dispatch latency, so the
    # dominant kernel (gate/up) is timed as the difference between the step loop above and the same loop with that
    # stage's launch left out (MOE_OPT_TIMING_SKIP_STAGE): its cost inside the pipelined stream, on the same
    # rotating inputs (so no cache level holds the experts).  Three alternations, median.
    up_marginal_ms = None
    if T <= 32:
        ct = timing_capi()
        if ct is not None:
            # a context of the timing twin over the same device weights (its own scratch); the loops below run on it
            mt = ct.Moe(d, mid, E, k, layers=nlayers, max_tokens=T)
            for l, L in enumerate(layers):
                L.register(mt, l)
            for o, v in list(LIB_OPTIONS) + list(opts):
                mt.set_option(o, v)

            def step_t(i):
                if kind == "stack":
                    for l in range(nlayers):
                        mt.forward(l, xs[(i * nlayers + l) % len(xs)], y)
                else:
                    mt.forward(0, xs[i % len(xs)], y)

            def loop_ms():
                f0, f1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                f0.record()
                for i in range(steps):
                    step_t(warmup + i)
                f1.record()
                torch.cuda.synchronize()
                return f0.elapsed_time(f1) / steps
            for i in range(warmup):
                step_t(i)
            diffs = []
            for _ in range(3):
                full = loop_ms()
                mt.set_option(5, 3)   # MOE_OPT_TIMING_SKIP_STAGE = 1 + MOE_PROF_UP
                part = loop_ms()
                mt.set_option(5, 0)
                diffs.append(full - part)
            up_marginal_ms = sorted(diffs)[1] / nlayers
            mt.close()

    # A pair of stage events costs a few microseconds more than the kernels between them take when they run
    # back to back (the event makes the next dispatch wait).  The mean surplus per stage is reported for
    # information; the roofline figures below use the raw event times (the conservative side: at decode sizes
    # rocprofv3's kernel durations are 2-4 us shorter than the event intervals).
    live = [v for v in stage.values() if v > 0]
    stage_overhead = max(0.0, (sum(live) - ms) / max(1, len(live)))

    # routing statistics of the last step (for the algorithmic byte / flop counts)
    ids, _ = m.last_routing(T)
    ids = ids[:, :k].cpu().numpy()
    eb = layers[0].expert_bytes()
    uniq = int(np.unique(ids).size)
    cnt = np.bincount(ids.reshape(-1), minlength=E)
    pairs = T * k
    res = {"n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 5),
           "host_ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "data": "synthetic", "stage_ms": {kk: round(v, 5) for kk, v in stage.items()},
           "stage_event_overhead_ms": round(stage_overhead, 5)}
    cfg = {"workload": wl, "tokens": T, "d_model": d, "moe_mid": mid, "experts": E, "topk": k, "shared_experts": 1,
           "format": ("q4cp g32, the reference converter's universal expert codebook (table look-up, f32 GEMV kernels)"
                      if universal else "q4cp g32 zero-point 8") if fmt == "q4cp" else
           "hgn v2 i4r g128, Hadamard-rotated (q4cp shared expert)" if fmt == "i4r" else
           (("GGUF ggml types %d gate/up, %d down, %d shared expert" % gg_types if GG_MIX_TYPES else
             "GGUF Q5_K gate/up, Q8_0 down, Q8_0 shared expert") if ggmix else "GGUF Q4_K"),
           "layers": nlayers, **extra}
    if kind == "prefill":
        flop_tok = k * 6 * d * mid + 6 * d * mid + 2 * d * E + 2 * d
        # the timed gate/up launch: the routed experts' pairs; the shared expert's tiles are in the same launch only
        # with MOE_OPT_SHARED_ASIDE = 0 or MOE_OPT_FUSED_COMBINE = 1 (by default its GEMMs run on the library's side
        # stream next to the router launch and are over before this launch starts)
        od = dict(list(LIB_OPTIONS) + list(opts))
        shared_in_launch = od.get(4, 1) == 0 or od.get(3, 0) != 0
        up_flop = (pairs + (T if shared_in_launch else 0)) * 2 * (2 * mid) * d
        up_s = stage["up"] * 1e-3
        res.update({"metric": "moe_layer_prefill_tokens_per_s", "unit": "tok/s", "value": round(T / (ms * 1e-3), 1),
                    "dtype": "f16",
                    "layer_tflops": round(flop_tok * T / (ms * 1e-3) / 1e12, 2),
                    "layer_mfma_frac": round(flop_tok * T / (ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                    "roofline": {"bound": "mfma", "kernel": ("k_moe_gemm (gate | up unfused) + the slot-wise rotations and SwiGLU, "
                                                              if fmt == "i4r" else "k_moe_gemm (gate/up + SwiGLU), ") +
                                 ("routed + shared expert tiles" if shared_in_launch else "routed experts' tiles"),
                                 "achieved": round(up_flop / up_s / 1e12, 2), "peak": MFMA_F16_PEAK_TFLOPS,
                                 "unit": "TFLOP/s", "frac": round(up_flop / up_s / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                                 "timing": "HIP events around the launch (moe_profile_enable), same stream",
                                 "traffic": None if shared_in_launch or universal else pmc_traffic(kind, fmt, T)}})
        # rows the grouped GEMM computes for the routed pairs: tiles of 128, the last tile of an expert padded
        # to a multiple of 32 rows
        rem = cnt % 128
        padded = (cnt // 128) * 128 + (rem + 31) // 32 * 32
        cfg.update({"hottest_over_mean": round(float(cnt.max() / cnt.mean()), 2), "empty_experts": int((cnt == 0).sum()),
                    "tile_row_fill": round(float(cnt.sum() / max(1, padded.sum())), 4)})
    else:
        # algorithmic bytes of a step: unique experts + shared expert + fp32 router + gate vector + x/y
        if kind == "stack":
            uniq = k
        step_bytes = nlayers * (uniq * eb + layers[0].shared_bytes() + E * d * 4 + d * 4 + T * 2 * d * 4)
        if fmt == "q4cp":
            gu_bytes = (uniq + 1) * 2 * mid * (d // 2 + S.q4cp_scale_stride(d))
        elif fmt == "i4r":
            gu_bytes = uniq * 2 * mid * (d // 2 + d // 128 * 2) + 2 * mid * (d // 2 + S.q4cp_scale_stride(d))
        else:
            gu_bytes = 2 * mid * (uniq * W.gg_row_bytes(gg_types[0], d) + W.gg_row_bytes(gg_types[2], d))
        marginal = up_marginal_ms is not None
        if not marginal:  # (no timing twin of the library: the event pair around the launch, an upper bound)
            up_marginal_ms = stage["up"]
        up_s = up_marginal_ms * 1e-3
        od = dict(list(LIB_OPTIONS) + list(opts))
        int_dec = od.get(1, 1) != 0 and not universal  # (a table codebook takes look-up / f32 kernels)
        # the arithmetic of the GEMV kernels: integer dot products of the 4-bit codes with the activations' 4-bit
        # (q4cp: v_dot8_i32_i4, four planes) or 8-bit (Q4_K: v_dot4_i32_i8, two planes) digit planes, f32 scales;
        # or plain f32 FMAs (MOE_OPT_INT_DECODE = 0, and the general GGUF kernels)
        res.update({"metric": "moe_layer_decode_hbm_GB_per_s", "unit": "GB/s",
                    "value": round(step_bytes / (ms * 1e-3) / 1e9, 1),
                    "dtype": "f32" if not int_dec else ("i4" if fmt in ("q4cp", "i4r") else "i8"),
                    "up_kernel_ms": round(up_marginal_ms, 5),
                    "hbm_frac": round(step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                    "tokens_per_s": round(T / (ms * 1e-3), 1),
                    "roofline": {"bound": "hbm", "kernel": ("gate | up GEMV in the rotated domain (sums left unfused)"
                                                             if fmt == "i4r" else "gate/up GEMV + SwiGLU"),
                                 "achieved": round(gu_bytes / up_s / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                 "frac": round(gu_bytes / up_s / 1e9 / HBM_PEAK_GBS, 4),
                                 "timing": ("step loop minus the same loop without this launch (on the library's timing "
                                            "twin, same kernels), HIP events around the loops (an event pair around the "
                                            "single launch reads %.2f us: the pair's dispatch latency is of the kernel's "
                                            "size)" % (stage["up"] * 1e3)) if marginal else
                                           "HIP events around the launch (moe_profile_enable), same stream",
                                 "traffic": pmc_traffic(kind, fmt, T) if int_dec else None}})
        cfg.update({"unique_experts": uniq, "step_bytes": int(step_bytes)})
    res["config"] = cfg
    if cpu:
        res["cpu_baseline"] = cpu_leg(kind, layers[0], xs, ids, cnt, m, T, eb, cpu_budget)
    m.close()
    return res


def measure_load(fmt, steps, nlayers):
    """Checkpoint file -> HBM: writes `nlayers` synthetic full-size layers to a temporary .hgn / GGUF file,
    then times moe_load_layers (file mapping -> one H2D copy per tensor -> registration).  Host-side,
    PCIe-bound set-up work: reported beside the hot path, never as its throughput."""
    import tempfile
    import torch
    from gfx1151_engine_amd import capi, files, workloads as W
    d, mid, k = D, MID, K
    tmp = tempfile.mkdtemp(prefix="moe_load_")
    path = os.path.join(tmp, "layers.hgn" if fmt == "q4cp" else "layers.gguf")
    tens = []
    for l in range(nlayers):
        L = W.DeviceLayer(2000 + l, d, mid, E, k, fmt)
        h = lambda t: t.cpu().numpy()

        class HL:  # the attribute names files.*_layer_tensors read
            pass
        hl = HL()
        hl.d, hl.mid, hl.E = d, mid, E
        hl.router = h(L.router)
        hl.shared = [h(L.sh[0]), h(L.sh[1]), h(L.sh[2]), h(L.sh_sg)]
        hl.down = h(L.down)
        if fmt == "q4cp":
            hl.gate_up = h(L.gate_up)
            tens += files.hgn_layer_tensors(l, hl)
        else:
            hl.gate, hl.up = h(L.gate), h(L.up)
            hl.shared[3] = hl.shared[3].reshape(-1)
            tens += files.gguf_layer_tensors(l, hl)
        del L
        torch.cuda.empty_cache()
    (files.write_hgn if fmt == "q4cp" else files.write_gguf)(path, tens)
    del tens
    nbytes = os.path.getsize(path)
    times = []
    try:
        for i in range(steps + 1):  # the first pass also pages the file in: not timed
            f = capi.ModelFile(path)
            cfg = f.config(0)
            m = capi.Moe(cfg.d, cfg.mid, cfg.experts, k, layers=cfg.layers, max_tokens=1)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            w = f.load_layers(m, 0, 0, cfg.layers)
            torch.cuda.synchronize()
            if i:
                times.append(time.perf_counter() - t0)
            wb = w.nbytes
            f.close()
            m.close()
            w.free()
    finally:
        os.remove(path)
        os.rmdir(tmp)
    ms = 1e3 * sum(times) / len(times)
    return {"metric": "moe_file_load_GB_per_s", "value": round(wb / (ms * 1e-3) / 1e9, 2), "unit": "GB/s", "n_gpus": 1,
            "steps": steps, "warmup": 1, "ms_per_step": round(ms, 3), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": "load_" + fmt, "layers": nlayers, "file_bytes": nbytes, "device_bytes": int(wb),
                       "format": ".hgn (HGN1)" if fmt == "q4cp" else "GGUF v3", "path": "page cache -> pinned staging (2 x 32 MiB, 6 threads) -> H2D"},
            "roofline": None, "cpu_baseline": None}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="headline")
    ap.add_argument("--tokens", type=int, default=0, help="override the batch size of the workload")
    ap.add_argument("--opt", action="append", default=[], metavar="ID=VALUE",
                    help="moe_set_option(ID, VALUE) on the context before the run (A/B runs of the library's switches)")
    ap.add_argument("--layers", type=int, default=48, help="stack workload: number of resident layers")
    ap.add_argument("--codebook", default="zp8", choices=("zp8", "universal"),
                    help="q4cp workloads: the benchmark's zero-point-8 grid, or the non-uniform 16-entry table that the "
                         "reference's converter writes into its checkpoints")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--gg-types", default="", metavar="GU,DN,SH",
                    help="ggmix_* workloads: ggml types of gate/up, down and the shared expert (default 13,8,8)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 256 MiB device copies (a kernel of known HBM traffic to scale "
                         "rocprofv3's FETCH_SIZE / WRITE_SIZE counters by)")
    a = ap.parse_args()
    if a.gg_types:
        global GG_MIX_TYPES
        GG_MIX_TYPES = tuple(int(v) for v in a.gg_types.split(","))
        if len(GG_MIX_TYPES) != 3:
            ap.error("--gg-types takes three ggml type numbers")
    LIB_OPTIONS.extend(tuple(int(v) for v in o.split("=")) for o in a.opt)
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU (the path has no multi-GPU part); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from gfx1151_engine_amd import capi
    capi.lib()  # raises if the HIP library is missing: there is no other path
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    if a.copy_calibration:
        src = torch.full((1 << 28,), 7, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if a.workload == "headline":
        res = measure("prefill", a.steps, a.warmup, a.tokens, cpu=not a.no_cpu)
        torch.cuda.empty_cache()
        # the other configurations of the benchmark, measured in the same run and reported as sub-records
        keys = ("metric", "value", "unit", "hbm_frac", "layer_mfma_frac", "ms_per_step", "steps", "stage_ms",
                "up_kernel_ms", "dtype", "roofline", "config", "cpu_baseline")
        nd, wd = max(a.steps, 64) * 4, max(a.warmup, 8)

        def sub(name, wl, steps, warmup, **kw):
            torch.cuda.empty_cache()
            r = measure(wl, steps, warmup, cpu=not a.no_cpu, cpu_budget=5.0, **kw)
            res[name] = {kk: r[kk] for kk in keys if kk in r}
        sub("decode_T1", "decode", nd, wd)
        sub("decode_T1_f32_kernels", "decode", nd, wd, opts=((1, 0),))   # MOE_OPT_INT_DECODE = 0
        sub("verify_T20", "verify", 128, wd)
        sub("stack48_T1", "stack", 16, 2)
        sub("q4k_prefill_T8192", "q4k_prefill", a.steps, a.warmup)
        sub("q4k_decode_T1", "q4k_decode", nd, wd)
        # the same q4cp shapes with the 16-entry table of the reference's converter (not affine: the grouped GEMM
        # dequantises through a table, the decode kernels look codes up instead of taking integer dots)
        sub("universal_codebook_prefill_T16384", "prefill", a.steps, a.warmup, codebook="universal")
        sub("universal_codebook_decode_T1", "decode", nd, wd, codebook="universal")
        # a GGUF layer in the type mix of the reference's checkpoints, and an hgn v2 layer (rotated i4r experts)
        sub("gguf_q5k_q8_0_prefill_T8192", "ggmix_prefill", a.steps, a.warmup)
        sub("gguf_q5k_q8_0_decode_T1", "ggmix_decode", nd, wd)
        sub("hgn_v2_prefill_T16384", "v2_prefill", a.steps, a.warmup)
        sub("hgn_v2_decode_T1", "v2_decode", nd, wd)
        sub("universal_codebook_verify_T20", "verify", 128, wd, codebook="universal")
        # the sub-records' key figures once more as top-level scalars, in front of the records themselves (a reader
        # that keeps only the head of the line still has every configuration's number)
        flat = {}
        for name in [n for n, v in res.items() if isinstance(v, dict) and "ms_per_step" in v]:
            r = res[name]
            flat[name + "_ms"] = r["ms_per_step"]
            if "hbm_frac" in r:
                flat[name + "_hbm_frac"] = r["hbm_frac"]
            if "layer_mfma_frac" in r:
                flat[name + "_layer_mfma_frac"] = r["layer_mfma_frac"]
            if r.get("roofline"):
                flat[name + "_kernel_frac"] = r["roofline"]["frac"]
        subs = {n: res.pop(n) for n in list(res) if isinstance(res[n], dict) and "ms_per_step" in res[n]}
        res.update(flat)
        res.update(subs)
    elif a.workload in ("load", "q4k_load"):
        res = measure_load("q4k" if a.workload.startswith("q4k") else "q4cp", min(a.steps, 5), min(a.layers, 2))
    else:
        res = measure(a.workload, a.steps, a.warmup, a.tokens, a.layers, cpu=not a.no_cpu, codebook=a.codebook)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
