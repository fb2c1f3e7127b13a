#!/usr/bin/env python3
"""Benchmark of the per-rank Odysseus hot path on one MI355X.

A "step" is one causal attention forward + backward over one rank's share of a
Llama-2-7B layer: 4 heads x 128, L = 32768, bf16, batch 1 (synthetic N(0,1)
inputs, already resident in HBM).  `value` is the algorithmic TFLOP/s of that step
(3.5 * 4 * L^2 * D * H / 2 FLOPs).  The same JSON line carries:

  roofline      the dominant kernel's algorithmic FLOP rate against the bf16 dense
                MFMA peak, its duration measured with HIP events on the launch stream
  kernels       the same for every attention kernel of the step
  step_ms       median / min / max of the K timed steps (HIP events around each step)
  mfma_sustained  what a loop of nothing but MFMAs sustains with constant and with random operands
  tile_cost_ladder  a synthetic kernel of the forward kernel's shape with the ingredients of a tile added one at a
                time (vector work, LDS operand reads, direct loads), ns per 64-key turn, beside the forward kernel
  configs       the other attention configurations (L = 131072; GQA 4:1 at L = 65536; the ring
                step over 8 key blocks of 16384; one rank of a zigzag ring of 8): ms, TFLOP/s, % of peak,
                forward / backward split
  layer         the other pieces of the rank's layer share (QKV / O / MLP GEMMs with
                torch.matmul on the same tensors as a same-box yardstick, RoPE, RMSNorm, SwiGLU)
                and the resulting tokens/s as a sum of pieces
  layer_end_to_end  the same share run through the modules and autograd
  cpu_baseline  the CPU oracle timed on this host's cores: the whole step, and the layer's products once

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-layer] [--no-configs]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, published
PEAK_FP32_TFLOPS = 157.3    # MI355X dense fp32 MFMA, published

# the rank shard the metric is quoted on
L, H, HKV, D = 32768, 4, 4, 128
D_MODEL, I_MLP, T_MLP = 4096, 11008, 4096


def attn_flops(Lq, Lk, h, d, causal=True):
    fwd = 4.0 * Lq * Lk * d * h * (0.5 if causal else 1.0)
    return fwd, 2.5 * fwd


def time_gpu(fn, iters, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / iters


def time_events(fn, iters, warmup):
    """Per-call durations (ms) from HIP events recorded on the current stream around every call."""
    import torch
    for _ in range(warmup):
        fn()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    torch.cuda.synchronize()
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return sorted(a.elapsed_time(b) for a, b in evs)


def spread(ms_sorted):
    n = len(ms_sorted)
    med = ms_sorted[n // 2] if n % 2 else 0.5 * (ms_sorted[n // 2 - 1] + ms_sorted[n // 2])
    return {"median": round(med, 4), "min": round(ms_sorted[0], 4), "max": round(ms_sorted[-1], 4)}


def kernel_ms(_lib, fn, iters, warmup):
    """Average duration per call of the library's own kernels (HIP events on the launch stream),
    summed over the kernels one call launches: (ms, {kernel: ms})."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    _lib.profile_collect()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    prof = _lib.profile_collect()
    _lib.profile_enable(False)
    per = {n: t / iters for n, (_, t, _) in prof.items()}
    return sum(per.values()), per


def measured_traffic():
    """HBM bytes per launch of the attention kernels at this workload, as measured with the
    FETCH_SIZE / WRITE_SIZE counters and recorded (as a JSON block) in the profile summary."""
    import re
    f = ROOT / "profiles" / "attention_L32768_hbm_traffic.md"
    if not f.exists():
        return {}
    m = re.search(r"```json\s*(\{.*?\})\s*```", f.read_text(), re.S)
    return json.loads(m.group(1)) if m else {}


_PROBES = None


def probes():
    """bench.py's own measurement kernels (odysseus_transformer_amd/lib/libodysseus_bench.so, built beside the product
    library from csrc/bench/probes.hip): not part of the product's ABI."""
    global _PROBES
    if _PROBES is None:
        import ctypes as C
        path = ROOT / "odysseus_transformer_amd" / "lib" / "libodysseus_bench.so"
        if not path.exists():
            from odysseus_transformer_amd import build
            build.build(verbose=False)
        lib = C.CDLL(str(path))
        lib.ody_bench_mfma_probe.restype = C.c_int
        lib.ody_bench_mfma_probe.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]
        lib.ody_bench_pipeline_probe.restype = C.c_int
        lib.ody_bench_pipeline_probe.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]
        _PROBES = lib
    return _PROBES


def _probe(name, *args):
    rc = getattr(probes(), name)(*args)
    if rc != 0:
        raise RuntimeError(f"{name} failed with status {rc}")


def mfma_sustained(_lib, dev):
    """What the matrix pipe sustains in a loop of nothing but MFMAs on register operands: with constant operands (the
    published peak is reached) and with random ones (what real data allows), for the 32x32x16 instruction that the
    kernels of this library use and for the 16x16x32 one."""
    import torch
    blocks, iters = 256, 8000            # one block of 4 wavefronts per CU; ~5 ms at the rates seen
    sink = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
    res = {}
    g = torch.Generator().manual_seed(7)
    st = torch.cuda.current_stream().cuda_stream
    for name, data in (("constant_operands", torch.ones(1 << 19)), ("random_operands", torch.randn(1 << 19, generator=g))):
        ops_ = data.to(torch.bfloat16).to(dev)
        for shape, tag in ((0, ""), (1, "_16x16x32")):
            best = None
            for rep in range(3):
                _probe("ody_bench_mfma_probe", ops_.data_ptr(), sink.data_ptr(), blocks, 200, shape, st)
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                _probe("ody_bench_mfma_probe", ops_.data_ptr(), sink.data_ptr(), blocks, iters, shape, st)
                e1.record()
                torch.cuda.synchronize()
                best = e0.elapsed_time(e1) if best is None else min(best, e0.elapsed_time(e1))
            # per iteration and wavefront: 16 MFMAs of 32768 FLOP, or 64 of 16384 (the 128 x 128 tile with k = 32)
            flop = blocks * 4 * iters * (16 * 32768.0 if shape == 0 else 64 * 16384.0)
            res[name + tag + "_tflops"] = round(flop / (best * 1e-3) / 1e12, 1)
    return res


def tile_cost_ladder(_lib, dev, fwd_ms):
    """What the ingredients of an attention tile cost on top of its MFMAs, measured with a synthetic kernel that has
    the forward kernel's shape (8 wavefronts, two per SIMD, one workgroup per CU, a barrier per 64-key turn, 32 MFMAs
    per wavefront and turn) and adds them one at a time -- and the forward kernel itself in the same unit."""
    import torch
    blocks, turns = 1024, 2000                   # 4 workgroups per CU in sequence; ~10 ms per rung
    sink = torch.empty(blocks * 512, dtype=torch.float32, device=dev)
    g = torch.Generator().manual_seed(7)
    ops_ = torch.randn(1 << 19, generator=g).to(torch.bfloat16).to(dev)
    src = torch.randn(32 << 20, generator=g).to(torch.bfloat16).to(dev)     # 64 MiB
    st = torch.cuda.current_stream().cuda_stream
    rungs = (("mfma_only", 0), ("plus_vector_work", 1), ("plus_lds_operand_reads", 3), ("plus_direct_loads_only", 5),
             ("plus_lds_reads_and_direct_loads", 7))
    res = {}
    for name, what in rungs:
        best = None
        for rep in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            _probe("ody_bench_pipeline_probe", ops_.data_ptr(), src.data_ptr(), sink.data_ptr(), blocks, turns, what, st)
            e1.record()
            torch.cuda.synchronize()
            if rep:
                best = e0.elapsed_time(e1) if best is None else min(best, e0.elapsed_time(e1))
        res[name] = {"ns_per_turn": round(best * 1e6 / (blocks / 256 * turns), 1),
                     "tflops": round(blocks * 8 * turns * 32 * 32768.0 / (best * 1e-3) / 1e12, 1)}
    # the forward kernel: 64 MFMAs per SIMD and turn as well; turns = executed MFMAs / (1024 SIMDs * 64)
    nqb = L // 256
    tiles = sum(min(L // 64, (qb * 256 + 255) // 64 + 1) for qb in range(nqb)) * H     # 64-key tiles x 256-query blocks
    mfmas = (tiles * 8 - nqb * H * 12) * 32        # 12 (wavefront, tile) pairs of a diagonal block lie above the diagonal
    res["attn_fwd_w8"] = {"ns_per_turn": round(fwd_ms * 1e6 / (mfmas / (1024 * 64)), 1),
                          "tflops_executed": round(mfmas * 32768.0 / (fwd_ms * 1e-3) / 1e12, 1)}
    return res


def cpu_baseline():
    """The oracle (plain PyTorch, fp32) on the host cores: the whole benchmark step -- causal
    attention fwd+bwd at 4 heads x 128, L = 32768 -- once (about 10 s on 16 cores), the three
    products (forward, dgrad, wgrad) of the rank's four linears once, and the fp32 layer."""
    import torch
    sys.path.insert(0, str(ROOT / "oracle"))
    import odysseus_oracle as oracle
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(2000)
    q, k, v, do = (torch.randn(1, L, H, D, generator=g) for _ in range(4))
    t0 = time.perf_counter()
    o, lse = oracle.attention_fwd(q, k, v, causal=True)
    oracle.attention_bwd(q, k, v, o, lse, do, causal=True)
    dt = time.perf_counter() - t0
    del q, k, v, do, o, lse
    f, b = attn_flops(L, L, H, D)
    gemms = {}
    for tag, (M, N, K) in (("qkv_proj", (L, (H + 2 * HKV) * D, D_MODEL)), ("o_proj", (L, D_MODEL, H * D)),
                           ("gate_up_proj", (T_MLP, 2 * I_MLP, D_MODEL)), ("down_proj", (T_MLP, D_MODEL, I_MLP))):
        x, w, dy = torch.randn(M, K, generator=g), torch.randn(N, K, generator=g) * 0.02, torch.randn(M, N, generator=g)
        t0 = time.perf_counter()
        oracle.linear_fwd(x, w)
        oracle.linear_bwd(x, w, dy)
        tg = time.perf_counter() - t0
        gemms[tag] = {"fwd_dgrad_wgrad_s": round(tg, 3), "tflops": round(6.0 * M * N * K / tg / 1e12, 3)}
        del x, w, dy
    # the fp32 configuration as a whole on the same cores: one decoder layer forward + backward,
    # d=512, 8 heads x 64, i=1376, L=2048 (3 warm-up runs, 10 timed)
    Lc, dc, Hc, Dc, ic = 2048, 512, 8, 64, 1376
    w = {"ln1": torch.ones(dc), "ln2": torch.ones(dc),
         "w_qkv": torch.randn(3 * Hc * Dc, dc, generator=g) * 0.02, "w_o": torch.randn(dc, Hc * Dc, generator=g) * 0.02,
         "w_gate_up": torch.randn(2 * ic, dc, generator=g) * 0.02, "w_down": torch.randn(dc, ic, generator=g) * 0.02}
    x, dy = torch.randn(1, Lc, dc, generator=g), torch.randn(1, Lc, dc, generator=g)
    for _ in range(3):
        oracle.decoder_layer_fwd_bwd(x, w, dy, Hc, Hc, Dc)
    t0 = time.perf_counter()
    for _ in range(10):
        oracle.decoder_layer_fwd_bwd(x, w, dy, Hc, Hc, Dc)
    layer_ms = (time.perf_counter() - t0) / 10 * 1e3
    return {"value": (f + b) / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"the whole step once: causal attention fwd+bwd, {H} heads x {D}, L={L}, fp32, {dt:.2f} s wall",
            "step_s": round(dt, 3), "linears_once": gemms,
            "fp32_layer_L2048_d512_ms": round(layer_ms, 2)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=15)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-layer", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="skip the L = 131072, GQA and ring configurations")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain device copy of the packed qkv buffer (100 MiB read + 100 MiB "
                         "written): the known-size kernel that calibrates the HBM byte counters of a "
                         "rocprofv3 --pmc run of this script")
    ap.add_argument("--power", action="store_true",
                    help="also read package power and engine clock from rocm-smi while the step, a GEMM, the MFMA "
                         "probe and a plain copy each run in a loop for a few seconds (slow: rocm-smi takes seconds "
                         "per reading)")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU's share of the layer on ONE GPU; collectives and multi-GPU runs are "
              "not part of this build (--gpus must be 1).", file=sys.stderr)
        sys.exit(2)

    import torch
    from odysseus_transformer_amd import _lib, ops
    _lib.load()
    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    prop = torch.cuda.get_device_properties(0)
    dt = torch.bfloat16

    def rn(shape, seed, std=1.0):
        g = torch.Generator().manual_seed(seed)
        return (torch.randn(shape, generator=g) * std).to(dt).to(dev)

    # ---- the step: attention fwd + bwd on q/k/v slices of a packed projection buffer
    qkv = rn((1, L, H + 2 * HKV, D), 2001)
    q, k, v = qkv[:, :, :H], qkv[:, :, H:H + HKV], qkv[:, :, H + HKV:]
    do = rn((1, L, H, D), 2002)
    dqkv = torch.empty_like(qkv)
    state = {}

    def step():
        o, lse = ops.attn_fwd(q, k, v, causal=True)
        ops.attn_bwd(q, k, v, o, lse, do, causal=True, dq=dqkv[:, :, :H], dk=dqkv[:, :, H:H + HKV],
                     dv=dqkv[:, :, H + HKV:])
        state["o"] = o

    # Kept dS is opt-in (it spends B * Hq * L * L bytes of scratch: 4 GiB here, 64 GiB at L = 131072): the benchmark
    # opts in, with a quarter of the device's memory as its budget, and also times the step without it below.
    ds_budget = prop.total_memory // 4
    ops.set_keep_ds_max_bytes(ds_budget)
    ds_bytes = _lib.load().ody_attn_bwd_ds_bytes(1, L, L, H, HKV, D, _lib.ODY_BF16, 1)
    for _ in range(a.warmup):
        step()
    if a.copy_probe:
        dqkv.copy_(qkv)
    # ---- the timed region: exactly K steps between two synchronisations, nothing else on the device
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / a.steps
    # ---- the same K steps again with every kernel between its own pair of HIP events on the launch stream
    # (the events serialise the launches, so these steps run a few percent longer than the timed ones)
    _lib.profile_enable(True)
    _lib.profile_collect()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    torch.cuda.synchronize()
    sec_profiled = (time.perf_counter() - t0) / a.steps
    prof = _lib.profile_collect()
    _lib.profile_enable(False)
    step_spread = spread(time_events(step, a.steps, 0))   # and once more, every step between its own pair of events
    # ---- the same step on the recomputing backward (no dS scratch: what ops.attn_bwd does unless asked otherwise)
    ops.set_keep_ds_max_bytes(0)
    sec_recompute = time_gpu(step, a.steps, 3)
    ops.set_keep_ds_max_bytes(ds_budget)

    f_fwd, f_bwd = attn_flops(L, L, H, D)
    # algorithmic FLOPs per launch: the backward's 5 tile products are S, dP, dV, dK (in the
    # dK/dV kernel) and dQ (in the dQ kernel); the S and dP the dQ kernel recomputes are not counted
    # (with kept dS -- ops.attn_bwd's default where the scratch fits -- the dQ kernel is the one product, over
    # the dS tiles that the dK/dV kernel stored: 2 bytes per visible pair each way)
    dq_kernel = "attn_bwd_dq_kept" if "attn_bwd_dq_kept" in prof else "attn_bwd_dq_pipe"
    algo = {"attn_fwd_w8": f_fwd, "attn_bwd_dkdv_pipe": f_bwd * 4 / 5, dq_kernel: f_bwd * 1 / 5}
    missing = [n for n in algo if n not in prof]
    if missing:
        raise SystemExit(f"bench.py: the library ran no kernel named {missing}; it reported {sorted(prof)}")
    kernels = {}
    for name, (n, total_ms, min_ms) in prof.items():
        avg = total_ms / n
        kernels[name] = {"launches": n, "avg_ms": round(avg, 4), "min_ms": round(min_ms, 4)}
        if name in algo:
            kernels[name]["tflops"] = round(algo[name] / (avg * 1e-3) / 1e12, 1)
        if name in ("attn_images", "attn_bwd_prepass"):
            # memory-bound passes: algorithmic bytes (one 64-row image pass reads and writes L*H*D bf16; the
            # query-side pre-pass reads Q, dO, O and lse and writes two images, delta and the start values)
            # against the HBM peak and against a device copy that moves the same number of bytes
            e = 2
            nbytes = 2 * L * H * D * e if name == "attn_images" else (3 + 2) * L * H * D * e + 2 * L * H * 4 + (L // 64) * H * 1024
            src = torch.empty(nbytes // 2, dtype=torch.uint8, device=dev)
            dst = torch.empty_like(src)
            ty = spread(time_events(lambda: dst.copy_(src), 20, 3))["median"]
            del src, dst
            kernels[name].update({"algorithmic_bytes": nbytes, "frac_of_hbm_peak": round(nbytes / (avg * 1e-3) / 1e9 / PEAK_HBM_GBS, 3),
                                  "copy_yardstick_ms": round(ty, 4), "ours_over_yardstick": round(ty / avg, 3)})
        if name == "attn_bwd_dq_kept":   # bound by HBM: the kept dS, read once
            ds_bytes = _lib.load().ody_attn_bwd_ds_bytes(1, L, L, H, HKV, D, _lib.ODY_BF16, 1)
            kernels[name]["hbm_read_gbps"] = round(ds_bytes / (avg * 1e-3) / 1e9, 1)
            kernels[name]["frac_of_hbm_peak"] = round(ds_bytes / (avg * 1e-3) / 1e9 / PEAK_HBM_GBS, 3)
    dom = max(algo, key=lambda n: prof[n][1] / prof[n][0])
    dom_avg = prof[dom][1] / prof[dom][0]
    achieved = algo[dom] / (dom_avg * 1e-3) / 1e12
    # the dK/dV kernel was measured both ways: keeping dS (4.3 GB more written) and on the recomputing path
    traffic = measured_traffic().get(dom + "_recompute" if dom == "attn_bwd_dkdv_pipe" and dq_kernel == "attn_bwd_dq_pipe" else dom)
    value = (f_fwd + f_bwd) / sec / 1e12

    info = _lib.device_info()
    device = {"name": prop.name, "cus": info["compute_units"], "clock_mhz": info["clock_khz"] / 1000.0,
              "lds_bytes_per_cu": info["lds_bytes_per_cu"],
              # 4 SIMDs x one 32x32x16 bf16 MFMA (32768 FLOP) per 32 cycles = 4096 FLOP per clock per CU
              "bf16_peak_from_cus_and_clock_tflops": round(info["compute_units"] * info["clock_khz"] * 1e3 * 4096 / 1e12, 1)}
    # kernels of the forward: the V image (one of the step's two image launches; the other is the backward's K
    # image), the main kernel and its follow-up over flagged query blocks; everything else belongs to the backward
    fwd_ms = (prof["attn_fwd_w8"][1] + prof.get("attn_fwd_mfma", (0, 0.0, 0))[1] +
              prof.get("attn_images", (0, 0.0, 0))[1] / 2) / a.steps
    bwd_ms = sum(t for n, (_, t, _) in prof.items()) / a.steps - fwd_ms

    out = {
        "metric": "attention fwd+bwd TFLOP/s (% bf16 MFMA peak) + decoder-layer tokens/s, 1 GPU",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(sec * 1e3, 4), "ms_per_step_with_kernel_events": round(sec_profiled * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "causal attention fwd+bwd, Llama-2-7B rank shard at N=8: 4 heads x 128, L=32768, "
                               "batch 1 (attention part of the 32768-token bf16 configuration)",
                   "heads": H, "kv_heads": HKV, "head_dim": D, "seq_len": L, "flops_per_step": f_fwd + f_bwd,
                   "seeds": {"qkv": 2001, "dout": 2002},
                   "backward": "kept dS" if dq_kernel == "attn_bwd_dq_kept" else "recomputing",
                   "ds_scratch_bytes": ds_bytes if dq_kernel == "attn_bwd_dq_kept" else 0,
                   "keep_ds_budget_bytes": ds_budget},
        "ms_per_step_recompute": round(sec_recompute * 1e3, 4),
        "value_recompute": round((f_fwd + f_bwd) / sec_recompute / 1e12, 2),
        "step_ms": step_spread, "fwd_ms": round(fwd_ms, 4), "bwd_ms": round(bwd_ms, 4),
        "fwd_tflops": round(f_fwd / (fwd_ms * 1e-3) / 1e12, 1), "bwd_tflops": round(f_bwd / (bwd_ms * 1e-3) / 1e12, 1),
        "pct_of_bf16_peak": round(100.0 * value / PEAK_BF16_TFLOPS, 2),
        "device": device,
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": traffic,
                     "avg_ms": round(dom_avg, 4), "algorithmic_flops_per_launch": algo[dom]},
        "kernels": kernels,
    }

    # context for the roofline: the rate a register-only MFMA loop sustains on this box
    out["mfma_sustained"] = mfma_sustained(_lib, dev)
    # boxes differ by ~10 % in what they sustain at the power limit; this ratio does not
    out["value_over_mfma_sustained_random"] = round(value / out["mfma_sustained"]["random_operands_tflops"], 3)
    out["tile_cost_ladder"] = tile_cost_ladder(_lib, dev, kernels["attn_fwd_w8"]["avg_ms"])
    if a.power:
        out["power"] = power_under_load(_lib, ops, dev, step)
    del qkv, q, k, v, do, dqkv
    state.clear()
    torch.cuda.empty_cache()
    if not a.no_configs:
        out["configs"] = other_configs(_lib, ops, rn, dev)
    if not a.no_layer:
        out["layer"] = layer_share(_lib, ops, rn, dev, sec)
        out["layer_end_to_end"] = layer_end_to_end(_lib, rn, dev, out["layer"])
        out["fp32"] = fp32_configuration(_lib, ops, dev)
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


FWD_KERNELS = ("attn_fwd_w8", "attn_fwd_mfma", "lse_merge", "cast_from_f32")


def other_configs(_lib, ops, rn, dev):
    """The remaining attention configurations, each timed like the main step: a few whole steps between HIP
    events, and the library's kernels by their own events for the forward / backward split."""
    import torch
    res = {}

    def record(tag, step, flops_fwd, flops_bwd, iters, n_images_fwd, n_images, note):
        ms = time_events(step, iters, 2)
        _, per = kernel_ms(_lib, step, iters, 0)
        img = per.get("attn_images", 0.0)
        fwd = sum(t for n, t in per.items() if n in FWD_KERNELS) + img * n_images_fwd / max(n_images, 1)
        bwd = sum(per.values()) - fwd
        med = spread(ms)["median"]
        tf = (flops_fwd + flops_bwd) / (med * 1e-3) / 1e12
        res[tag] = {"workload": note, "step_ms": spread(ms), "tflops": round(tf, 1),
                    "pct_of_bf16_peak": round(100 * tf / PEAK_BF16_TFLOPS, 2), "flops_per_step": flops_fwd + flops_bwd,
                    "fwd_kernel_ms": round(fwd, 4), "bwd_kernel_ms": round(bwd, 4),
                    "fwd_tflops": round(flops_fwd / (fwd * 1e-3) / 1e12, 1),
                    "bwd_tflops": round(flops_bwd / (bwd * 1e-3) / 1e12, 1),
                    "kernels_ms": {n: round(t, 4) for n, t in sorted(per.items())}}

    def plain(tag, Lc, Hq, Hkv, seed, iters, note):
        q, do = rn((1, Lc, Hq, D), seed), rn((1, Lc, Hq, D), seed + 3)
        k, v = rn((1, Lc, Hkv, D), seed + 1), rn((1, Lc, Hkv, D), seed + 2)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)

        def step():
            o, lse = ops.attn_fwd(q, k, v, causal=True)
            ops.attn_bwd(q, k, v, o, lse, do, causal=True, dq=dq, dk=dk, dv=dv)

        f, b = attn_flops(Lc, Lc, Hq, D)
        record(tag, step, f, b, iters, 1, 2, note)

    plain("cfg3_L131072", 131072, 4, 4, 3000, 3, "causal attention fwd+bwd, 4 heads x 128, L=131072")
    torch.cuda.empty_cache()
    plain("cfg4_L65536_gqa4", 65536, 4, 1, 4000, 5, "causal attention fwd+bwd, 4 query heads on 1 kv head x 128, L=65536")
    torch.cuda.empty_cache()

    # the ring step: local queries against 8 key blocks, block 0 the causal diagonal, through autograd
    Lq, NB = 16384, 8
    q = rn((1, Lq, H, D), 5000).requires_grad_(True)
    ks = [rn((1, Lq, H, D), 5001 + 2 * b).requires_grad_(True) for b in range(NB)]
    vs = [rn((1, Lq, H, D), 5002 + 2 * b).requires_grad_(True) for b in range(NB)]
    do = rn((1, Lq, H, D), 5100)

    def ring_step():
        for t in [q] + ks + vs:
            t.grad = None
        out, _ = ops.ring_blocks_attn(q, ks, vs, causal_block=0)
        out.backward(do)

    f_full, b_full = attn_flops(Lq, Lq, H, D, causal=False)
    f_diag, b_diag = attn_flops(Lq, Lq, H, D, causal=True)
    record("cfg5_ring_8x16384", ring_step, 7 * f_full + f_diag, 7 * b_full + b_diag, 5, NB, 2 * NB,
           "ring step through autograd: 16384 queries x 4 heads x 128 against 8 key blocks of 16384 "
           "(block 0 causal), LSE merge after each, backward over all 8")
    del q, ks, vs, do
    torch.cuda.empty_cache()

    # one rank of a zigzag ring of 8 (rank 3): its two chunks of 8192 queries against the 8 blocks it would receive,
    # through autograd; 3 steps see the first chunk of a block with all queries, 4 the whole block with the second chunk
    c, NR, rank = 8192, 8, 3
    q = rn((1, 2 * c, H, D), 6000).requires_grad_(True)
    ks = [rn((1, 2 * c, H, D), 6001 + 2 * b).requires_grad_(True) for b in range(NR)]
    vs = [rn((1, 2 * c, H, D), 6002 + 2 * b).requires_grad_(True) for b in range(NR)]
    do = rn((1, 2 * c, H, D), 6100)

    def zigzag_step():
        for t in [q] + ks + vs:
            t.grad = None
        out, _ = ops.zigzag_ring_rank_attn(q, ks, vs, rank, NR)
        out.backward(do)

    f_c, b_c = attn_flops(2 * c, 2 * c, H, D, causal=True)        # step 0
    f_r, b_r = attn_flops(2 * c, c, H, D, causal=False)           # every other step: 2c x c or c x 2c score elements
    record("zigzag_ring_rank3_of_8", zigzag_step, f_c + (NR - 1) * f_r, b_c + (NR - 1) * b_r, 5, NR, 2 * NR,
           "one rank of a zigzag ring of 8 through autograd: chunks 3 and 12 of a 131072-token sequence (2 x 8192 queries, "
           "4 heads x 128) against the 8 blocks it receives, LSE merge after each, backward over all 8")
    return res


def layer_end_to_end(_lib, rn, dev, pieces):
    """One rank's share of a layer run through the modules and autograd instead of summed from separately
    timed pieces: LlamaFlashAttention2TPSP on the gathered 32768 tokens (packed QKV projection, RoPE, attention,
    output projection; forward + backward), and on the 4096-token shard RMSNorm -> LlamaMLPZeRO plus the other
    RMSNorm and both residual adds.  Host overhead, workspace handling and autograd bookkeeping are inside."""
    import types
    import torch
    from odysseus_transformer_amd.decoder.odysseus import LlamaFlashAttention2TPSP, LlamaMLPZeRO, LlamaRMSNorm
    from odysseus_transformer_amd.utils import globals as arena
    cfg = types.SimpleNamespace(hidden_size=D_MODEL, num_attention_heads=H, num_key_value_heads=HKV, head_dim=D,
                                intermediate_size=I_MLP, hidden_act="silu", attention_dropout=0.0, rms_norm_eps=1e-6,
                                rope_theta=10000.0, max_position_embeddings=1 << 20, pretraining_tp=1,
                                num_hidden_layers=1)
    dt = torch.bfloat16
    if arena._Arena.instance is None:
        arena._set_global_memory_buffer(dev)
    attn = LlamaFlashAttention2TPSP(cfg, 0).to(dt).to(dev)
    mlp = LlamaMLPZeRO(cfg).to(dt).to(dev)
    n1, n2 = LlamaRMSNorm(D_MODEL).to(dt).to(dev), LlamaRMSNorm(D_MODEL).to(dt).to(dev)
    with torch.no_grad():
        for i, w in enumerate(list(attn.parameters()) + list(mlp.parameters())):
            w.copy_(rn(tuple(w.shape), 9000 + i, 0.02))
    x_full = rn((1, L, D_MODEL), 9100).requires_grad_(True)     # the gathered, normalised activation
    dy_full = rn((1, L, D_MODEL), 9101)
    x_loc = rn((1, T_MLP, D_MODEL), 9102).requires_grad_(True)
    dy_loc = rn((1, T_MLP, D_MODEL), 9103)
    pos = torch.arange(L, device=dev)[None]
    params = list(attn.parameters()) + list(mlp.parameters()) + list(n1.parameters()) + list(n2.parameters())

    def attn_part():
        attn(x_full, position_ids=pos)[0].backward(dy_full)

    from odysseus_transformer_amd import ops as _ops

    def shard_part():
        a = n1(x_loc)                      # the norm in front of the attention block (its output is what gets gathered)
        h = x_loc + a                      # stands in for the residual add after the reduce-scatter of the attention block
        # second norm, SwiGLU MLP and the second residual add with the elementwise steps in the products' epilogues
        n, skip = _ops.rmsnorm_fork(h, n2.weight, n2.variance_epsilon)
        mlp(n, residual=skip).backward(dy_loc)

    def whole():
        for t in params + [x_full, x_loc]:
            t.grad = None
        attn_part()
        shard_part()

    ms = time_events(whole, 10, 3)
    ms_attn = time_events(lambda: ([setattr(t, "grad", None) for t in params + [x_full]], attn_part()), 10, 1)
    ms_shard = time_events(lambda: ([setattr(t, "grad", None) for t in params + [x_loc]], shard_part()), 10, 1)
    med = spread(ms)["median"]
    arena._destroy_global_memory_buffer()
    return {"workload": "LlamaFlashAttention2TPSP (32768 gathered tokens, 4 x 128 heads) + RMSNorm / LlamaMLPZeRO / "
                        "residual adds on the 4096-token shard, forward + backward through autograd",
            "ms": spread(ms), "attention_block_ms": spread(ms_attn), "shard_part_ms": spread(ms_shard),
            "layer_tokens_per_s_per_gpu": round(T_MLP / (med * 1e-3), 1),
            "sum_of_pieces_tokens_per_s_per_gpu": pieces["layer_tokens_per_s_per_gpu"],
            "scratch": "attention, split-K and norm workspaces drawn from the GlobalMemoryBuffer arena",
            "fusions": "SwiGLU forward / backward, both residual adds and the rotary embedding run in GEMM epilogues, the "
                       "rotary backward in the attention backward's epilogues, the gradient sum at the fork of the "
                       "residual stream inside the RMSNorm backward"}


def layer_share(_lib, ops, rn, dev, attn_sec):
    """Times the rest of the rank's share of the layer: the TP-split QKV / O linears over
    the gathered 32768 tokens, RoPE, and the sequence shard's RMSNorm + SwiGLU MLP over
    4096 tokens, each forward and backward (fwd, dgrad, wgrad)."""
    import torch
    res = {}

    def gemm3(tag, M, N, K):
        """The three products of one linear, 20 calls each: the library's kernels by their own HIP events, and
        torch.matmul on the same tensors by events on the same stream as a same-box yardstick (measurement
        only: it is not on any product path)."""
        x, w, dy = rn((M, K), 1), rn((N, K), 2, 0.02), rn((M, N), 3)
        fl = 2.0 * M * N * K
        mine, yard, kern = [], [], {}
        for name, ours, theirs in (("fwd", lambda: ops.gemm(ops.GEMM_NT, x, w), lambda: torch.matmul(x, w.t())),
                                   ("dgrad", lambda: ops.gemm(ops.GEMM_NN, dy, w), lambda: torch.matmul(dy, w)),
                                   ("wgrad", lambda: ops.gemm(ops.GEMM_TN, dy, x), lambda: torch.matmul(dy.t(), x))):
            t, per = kernel_ms(_lib, ours, 20, 3)
            mine.append(t * 1e-3)
            kern[name] = sorted(per)
            yard.append(spread(time_events(theirs, 20, 3))["median"] * 1e-3)
        res[tag] = {"M": M, "N": N, "K": K, "fwd_ms": round(mine[0] * 1e3, 4), "dgrad_ms": round(mine[1] * 1e3, 4),
                    "wgrad_ms": round(mine[2] * 1e3, 4), "tflops": [round(fl / t / 1e12, 1) for t in mine],
                    "frac_of_bf16_peak": [round(fl / t / 1e12 / PEAK_BF16_TFLOPS, 3) for t in mine],
                    "kernels": kern,
                    "yardstick": {"what": "torch.matmul on the same tensors (hipBLASLt), median of 20 by HIP events",
                                  "ms": [round(t * 1e3, 4) for t in yard],
                                  "tflops": [round(fl / t / 1e12, 1) for t in yard],
                                  "ours_over_yardstick": [round(ty / tm, 3) for tm, ty in zip(mine, yard)]}}
        del x, w, dy
        return sum(mine)

    def membound(tag, fn, nbytes):
        # wall clock per call (what the layer total uses; for kernels this short it includes the host's
        # launch cost) and the kernels' own duration from HIP events on the launch stream (the HBM rate)
        t = time_gpu(fn, 10, 3)
        _lib.profile_enable(True)
        _lib.profile_collect()
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        prof = _lib.profile_collect()
        _lib.profile_enable(False)
        tk = sum(total_ms for (_, total_ms, _) in prof.values()) / 10 * 1e-3
        # same-box yardstick: a device copy that moves the same number of bytes (half read, half written), one
        # launch between two HIP events like the kernels above (measurement only, on no product path)
        src = torch.empty(nbytes // 2, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        ty = spread(time_events(lambda: dst.copy_(src), 20, 3))["median"] * 1e-3
        del src, dst
        res[tag] = {"ms": round(t * 1e3, 4), "kernel_ms": round(tk * 1e3, 4), "kernels": sorted(prof),
                    "algorithmic_GBs": round(nbytes / tk / 1e9, 1),
                    "frac_of_hbm_peak": round(nbytes / tk / 1e9 / PEAK_HBM_GBS, 3),
                    "copy_yardstick": {"ms": round(ty * 1e3, 4), "GBs": round(nbytes / ty / 1e9, 1),
                                       "frac_of_hbm_peak": round(nbytes / ty / 1e9 / PEAK_HBM_GBS, 3),
                                       "ours_over_yardstick": round(ty / tk, 3)}}
        return t

    t_attn_half = attn_sec
    t_attn_half += gemm3("qkv_proj", L, (H + 2 * HKV) * D, D_MODEL)
    t_attn_half += gemm3("o_proj", L, D_MODEL, H * D)
    qkv = rn((1, L, H + 2 * HKV, D), 5)
    e = 2
    rope_bytes = 2 * L * (H + HKV) * D * e
    t_attn_half += 2 * membound("rope", lambda: ops.rope_(qkv, H + HKV), rope_bytes)
    del qkv
    # the same rotation inside the QKV projection's epilogue (what the modules run): table + fused product, by kernel events
    xq, wq = rn((L, D_MODEL), 8), rn(((H + 2 * HKV) * D, D_MODEL), 9, std=0.02)
    _lib.profile_enable(True)
    _lib.profile_collect()
    for _ in range(10):
        ops.linear_rope(xq, wq, ops.rope_table(None, L, D, 10000.0, device=dev), H + HKV, D)
    torch.cuda.synchronize()
    prof = _lib.profile_collect()
    _lib.profile_enable(False)
    res["qkv_proj_with_rope"] = {"kernels_ms": {k: round(v[1] / 10, 4) for k, v in sorted(prof.items())},
                                 "fwd_tflops": round(2.0 * L * (H + 2 * HKV) * D * D_MODEL / (prof["gemm_bf16_nt_rope"][1] / 10 * 1e-3) / 1e12, 1)}
    del xq, wq

    t_mlp_half = gemm3("gate_up_proj", T_MLP, 2 * I_MLP, D_MODEL)
    t_mlp_half += gemm3("down_proj", T_MLP, D_MODEL, I_MLP)
    gu, dh = rn((T_MLP, 2 * I_MLP), 6), rn((T_MLP, I_MLP), 7)
    t_mlp_half += membound("swiglu_fwd", lambda: ops.swiglu_fwd(gu), 3 * T_MLP * I_MLP * e)
    t_mlp_half += membound("swiglu_bwd", lambda: ops.swiglu_bwd(gu, dh), 5 * T_MLP * I_MLP * e)
    del gu, dh
    x, w, dy = rn((T_MLP, D_MODEL), 8), rn((D_MODEL,), 9), rn((T_MLP, D_MODEL), 10)
    _, rstd = ops.rmsnorm_fwd(x, w)
    t_n = membound("rmsnorm_fwd", lambda: ops.rmsnorm_fwd(x, w), 2 * T_MLP * D_MODEL * e)
    t_n += membound("rmsnorm_bwd", lambda: ops.rmsnorm_bwd(x, w, rstd, dy), 3 * T_MLP * D_MODEL * e)
    t_mlp_half += 2 * t_n  # both norms of the layer act on the sequence shard
    del x, w, dy
    # the same memory-bound kernels at 8x the rows: at the layer's own sizes they run 15-40 us, where launch
    # and ramp-up are a visible share; these show what the kernels reach once the chip is filled for longer
    big = {}
    T8 = 8 * T_MLP
    x, w, dy = rn((T8, D_MODEL), 8), rn((D_MODEL,), 9), rn((T8, D_MODEL), 10)
    _, rstd = ops.rmsnorm_fwd(x, w)
    keep = dict(res)
    membound("rmsnorm_fwd", lambda: ops.rmsnorm_fwd(x, w), 2 * T8 * D_MODEL * e)
    membound("rmsnorm_bwd", lambda: ops.rmsnorm_bwd(x, w, rstd, dy), 3 * T8 * D_MODEL * e)
    del x, w, dy
    qkv = rn((1, 4 * L, H + 2 * HKV, D), 5)
    membound("rope", lambda: ops.rope_(qkv, H + HKV), 2 * 4 * L * (H + HKV) * D * e)
    del qkv
    for k in ("rmsnorm_fwd", "rmsnorm_bwd", "rope"):
        big[k] = {n: res[k][n] for n in ("kernel_ms", "algorithmic_GBs", "frac_of_hbm_peak", "copy_yardstick")}
    res.clear()
    res.update(keep)
    res["memory_bound_at_8x_rows"] = {"rows": {"rmsnorm": T8, "rope": 4 * L}, **big}
    res["attn_half_ms"] = round(t_attn_half * 1e3, 3)
    res["mlp_half_ms"] = round(t_mlp_half * 1e3, 3)
    res["attn_half_tokens_per_s"] = round(L / t_attn_half, 1)
    res["mlp_half_tokens_per_s"] = round(T_MLP / t_mlp_half, 1)
    # one rank advances its 4096-token shard of the 32768-token layer in attn_half + mlp_half
    res["layer_tokens_per_s_per_gpu"] = round(T_MLP / (t_attn_half + t_mlp_half), 1)
    return res


def power_under_load(_lib, ops, dev, attention_step):
    """Package power (W) and engine clock (MHz) as rocm-smi reports them while one workload at a time keeps
    the queue full: the matrix kernels run at the package power limit, and the clock is what gives."""
    import subprocess
    import torch

    def reading():
        txt = subprocess.run(["/opt/rocm/bin/rocm-smi", "-a", "--json"], capture_output=True, text=True).stdout
        card = json.loads(txt[txt.index("{"):])["card0"]
        return {"socket_power_w": card.get("current_socket_power (W)"), "sclk": card.get("sclk clock speed:"),
                "power_limit_w": card.get("Max Graphics Package Power (W)"),
                "junction_c": card.get("Temperature (Sensor junction) (C)")}

    def under(fn, secs=4.0):
        fn()
        torch.cuda.synchronize()
        t0, got = time.time(), None
        while time.time() - t0 < secs or got is None:
            for _ in range(20):
                fn()
            if time.time() - t0 > 1.5 and got is None:
                got = reading()          # taken while 20 launches are still queued
        torch.cuda.synchronize()
        return got

    st = torch.cuda.current_stream().cuda_stream
    rand = torch.randn(1 << 20, device=dev).bfloat16()
    ones = torch.ones(1 << 20, device=dev).bfloat16()
    sink = torch.empty(4096 * 256, device=dev)
    a = torch.randn((8192, 8192), device=dev).bfloat16()
    b = torch.randn((8192, 8192), device=dev).bfloat16()
    src = torch.randn(1 << 28, device=dev).bfloat16()
    dst = torch.empty_like(src)
    return {
        "attention_step": under(attention_step),
        "gemm_nt_8192": under(lambda: ops.gemm(ops.GEMM_NT, a, b)),
        "mfma_probe_random_operands": under(lambda: _probe("ody_bench_mfma_probe", rand.data_ptr(), sink.data_ptr(), 4096,
                                                              2000, 0, st)),
        "mfma_probe_constant_operands": under(lambda: _probe("ody_bench_mfma_probe", ones.data_ptr(), sink.data_ptr(),
                                                                4096, 2000, 0, st)),
        "copy_512MiB": under(lambda: dst.copy_(src)),
    }


def fp32_configuration(_lib, ops, dev):
    """The fp32 parity configuration on the GPU (d=512, 8 heads x 64, i=1376, L=2048: one decoder layer forward +
    backward), and the fp32 kernels at a size that fills the chip, against the 157.3 TFLOP/s fp32 matrix peak."""
    import types
    import torch
    from odysseus_transformer_amd.decoder.odysseus import OdysseusDecoderLayer
    res = {}
    Lc, d, Hc, Dc, ic = 2048, 512, 8, 64, 1376
    cfg = types.SimpleNamespace(hidden_size=d, num_attention_heads=Hc, num_key_value_heads=Hc, head_dim=Dc,
                                intermediate_size=ic, hidden_act="silu", attention_dropout=0.0, rms_norm_eps=1e-6,
                                rope_theta=10000.0, max_position_embeddings=1 << 20, pretraining_tp=1,
                                num_hidden_layers=1)
    layer = OdysseusDecoderLayer(cfg).to(dev)
    g = torch.Generator().manual_seed(0)
    with torch.no_grad():
        for w in layer.parameters():
            if w.dim() > 1:
                w.copy_((torch.randn(w.shape, generator=g) * 0.02).to(dev))
    x = torch.randn((1, Lc, d), generator=g).to(dev).requires_grad_(True)
    dy = torch.randn((1, Lc, d), generator=g).to(dev)
    pos = torch.arange(Lc, device=dev)[None]

    def layer_step():
        layer(x, position_ids=pos).backward(dy)

    res["layer_L2048_d512_ms"] = round(time_gpu(layer_step, 10, 3) * 1e3, 3)
    res["layer_L2048_d512_tokens_per_s"] = round(Lc / (res["layer_L2048_d512_ms"] * 1e-3), 1)

    La, Ha = 16384, 8
    q, k, v, do = (torch.randn((1, La, Ha, Dc), generator=g).to(dev) for _ in range(4))
    o, lse = ops.attn_fwd(q, k, v, causal=True)
    f_fwd, f_bwd = attn_flops(La, La, Ha, Dc)
    tf = time_gpu(lambda: ops.attn_fwd(q, k, v, causal=True), 3, 1)
    tb = time_gpu(lambda: ops.attn_bwd(q, k, v, o, lse, do, causal=True), 3, 1)
    res["attention_L16384_8x64"] = {"fwd_ms": round(tf * 1e3, 3), "bwd_ms": round(tb * 1e3, 3),
                                    "fwd_tflops": round(f_fwd / tf / 1e12, 1), "bwd_tflops": round(f_bwd / tb / 1e12, 1),
                                    "frac_of_fp32_peak": round((f_fwd + f_bwd) / (tf + tb) / 1e12 / PEAK_FP32_TFLOPS, 3)}
    del q, k, v, do, o, lse
    M = N = K = 4096
    a, b, c = (torch.randn((M, K), generator=g).to(dev) for _ in range(3))
    ts = [time_gpu(lambda op=op: ops.gemm(op, a, b), 3, 1) for op in (ops.GEMM_NT, ops.GEMM_NN, ops.GEMM_TN)]
    res["gemm_4096x4096x4096"] = {"tflops_nt_nn_tn": [round(2.0 * M * N * K / t / 1e12, 1) for t in ts],
                                  "frac_of_fp32_peak": round(2.0 * M * N * K / max(ts) / 1e12 / PEAK_FP32_TFLOPS, 3)}
    return res


if __name__ == "__main__":
    main()
