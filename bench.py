#!/usr/bin/env python3
"""Benchmark of the QLoRA quantized base-linear hot path on one MI355X.

Workload (BASELINE.json configs[1]): block_fp8 QLoRA on the Qwen3-8B MLP --
M = 8192 tokens, hidden 4096, intermediate 12288, gate/up [12288, 4096] and
down [4096, 12288] quantized to e4m3 with 128x128 fp32 block scales, LoRA
r = 32 on all three projections, SwiGLU in between, full forward + backward.
One "step" is one forward + backward of that MLP on synthetic inputs that are
resident in HBM before the timed region starts.

Prints ONE JSON line (see the keys at the bottom).  `value` is algorithmic
TFLOP/s of the whole step (4MKN + 6Mr(K+N) per projection); `roofline` is the
fused dequant-GEMM kernel alone, timed per launch with HIP events on the launch
stream; `cpu_baseline` is the reference recipe (decode -> bf16 F.linear -> fp32
LoRA -> autograd) on the host cores over a bounded row sample.
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "QLoRA dequant-GEMM+LoRA fwd/bwd TFLOP/s & % MFMA/HBM peak, 1 GPU"
M, H, I, R, ALPHA = 8192, 4096, 12288, 32, 64
BF16_MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense bf16, published

# HBM-side bytes per launch of each config's roofline kernel, from the committed counter runs
# (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, each scaled by what the same counter reads for a plain
# 256 MiB -> 256 MiB copy).  Each entry names the profile file that holds the figures and the commands, and the
# average launch duration of the roofline kernel in that profile's own bench line: a run whose live average differs
# from it by more than 10 % is timing another kernel build (or another machine state) than the counters saw, and
# reports traffic null with the reason instead of a stale constant.  A config that has no counter run reports null.
# --traffic-bytes overrides.
MEASURED_TRAFFIC = {
    # gemm_256_kernel<int4, T=128> in 4 K splits + splitk_reduce_kernel: mean of the forward and dgrad launches
    # (64 MiB of it are the fp32 partial sums written and read back)
    0: (109.6 * 2 ** 20, "profiles/gemm_128_int4_linear_m512.txt", 0.04315),
    # gemm_dtl16_kernel (dense block-fp8, 256x256 tiles): mean over the 5 launches of a step (gate, up and down
    # forward, d_h, dx as one sum over the gate and up weights)
    1: (1070.4 * 2 ** 20, "profiles/gemm_dtl16_fp8_mlp_m8192.txt", 0.7509),
    # gemm_256_kernel<nvfp4>, 256x256 tiles (whole rounds; trailing rows in K splits) and 128x128 tiles
    # (+ splitk_reduce_kernel): mean over the 12 launches of a step, fp32 partial sums included
    2: (185.7 * 2 ** 20, "profiles/gemm_256_nvfp4_attn_m4096.txt", 0.14304),
    # gemm_dtl16_kernel<.., grouped>: mean over the 4 launches of a step (gate|up forward over two banks, down
    # forward, d_h, dx as one sum over both banks)
    3: (1402.4 * 2 ** 20, "profiles/gemm_dtl16_fp8_grouped_moe_e128.txt", 0.6325),
    # skinny_gemv_kernel (M = 1), skinny_rows_kernel (M <= 16) and skinny_split_kernel + skinny_epilogue_kernel
    # (M = 32, 64): mean per forward over the 32 cases (includes the fp32 partial tiles of the two-launch cases
    # written and read back: 23.3 MiB of it are algorithmic)
    4: (39.3 * 2 ** 20, "profiles/skinny_kernels_decode_shapes.txt", 0.01712),
    # merge_prep_kernel + merge_kernel<fp8>: mean per call (re-quantise 96 MiB, publish 144 MiB algorithmic)
    5: (134.4 * 2 ** 20, "profiles/merge_kernel_fp8_mlp_weights.txt", 0.04168),
    # gemm_256_kernel<nf4>: mean of the forward and dgrad launches
    6: (748.2 * 2 ** 20, "profiles/gemm_256_nf4_mlp_m8192.txt", 0.84180),
    # gemm_256_kernel<nvfp4 GKN, grouped>: mean over the 6 launches of a step
    7: (893.9 * 2 ** 20, "profiles/gemm_256_nvfp4_gkn_grouped_moe_e128.txt", 0.52825),
    # merge_prep_kernel + merge_kernel<nvfp4>: mean per call over amax / re-quantise / publish of the four weights
    9: (59.0 * 2 ** 20, "profiles/merge_kernel_nvfp4_attn_weights.txt", 0.03500),
}


def step_flops(m: int) -> float:
    per = lambda K, N: 4.0 * m * K * N + 6.0 * m * R * (K + N)
    return 2 * per(H, I) + per(I, H)


def gen(shape, std, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(dtype)


def build_modules():
    """Three BlockFP8QLoRALinear modules built on the CPU (so the CPU baseline can
    decode the very same bytes)."""
    from xorl_amd.qlora import QLoRALinear

    mods = {}
    for i, (name, (N, K)) in enumerate({"gate": (I, H), "up": (I, H), "down": (H, I)}.items()):
        lin = torch.nn.Linear(K, N, bias=False)
        with torch.no_grad():
            lin.weight.copy_(gen((N, K), 0.02, 100 + i))
        m = QLoRALinear.from_module(lin, r=R, lora_alpha=ALPHA, quant_format="block_fp8")
        with torch.no_grad():
            m.lora_A.copy_(gen((R, K), 0.02, 200 + i))
            m.lora_B.copy_(gen((N, R), 0.02, 300 + i))
        mods[name] = m
    return mods


def cpu_baseline(mods, rows: int, warmups: int = 2, runs: int = 5):
    """Reference recipe on host cores over `rows` tokens of the same workload."""
    from oracle import decode_np as NP
    from oracle import recipe as RC

    torch.set_num_threads(os.cpu_count())
    x = gen((rows, H), 1.0, 1, torch.bfloat16)
    dy = gen((rows, H), 1.0, 2, torch.bfloat16)

    def run():
        w = {}
        for k, m in mods.items():    # the reference decodes every weight in every forward
            packed = m.packed_weight_f32.detach().contiguous().view(torch.uint8).numpy()
            s = m.weight_block_scales.contiguous().view(torch.float32).numpy()
            w[k] = torch.from_numpy(NP.fp8_decode(packed, s, m.out_features, m.in_features)[0])   # fp32, as the reference
        xx = x.clone().requires_grad_(True)
        P = {k: (m.lora_A.detach().clone().requires_grad_(True), m.lora_B.detach().clone().requires_grad_(True))
             for k, m in mods.items()}
        g = RC.linear_forward_recipe(xx, w["gate"], *P["gate"], ALPHA / R)
        u = RC.linear_forward_recipe(xx, w["up"], *P["up"], ALPHA / R)
        h = RC.silu_and_mul_recipe(g, u)
        y = RC.linear_forward_recipe(h, w["down"], *P["down"], ALPHA / R)
        y.backward(dy)
        return y

    for _ in range(warmups):
        run()
    times = []
    for _ in range(runs):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    dt = sorted(times)[len(times) // 2]
    return {
        "value": step_flops(rows) / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": os.cpu_count(),
        "kind": "port",
        "sample": f"{'all ' if rows == M else ''}{rows} of {M} token rows of the same MLP, decode+fwd+bwd, torch CPU ops on the oracle decode: "
                  f"median of {runs} runs after {warmups} warm-ups, {dt:.2f} s per run "
                  f"(min {min(times):.2f}, max {max(times):.2f})",
    }


def zipf_routing(T, E, topk, seed, empty=2, device="cpu"):
    """Seeded router output whose per-expert token counts follow Zipf(s=1.1) over a random
    permutation of the experts; the `empty` least popular experts are never chosen."""
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(E, generator=g)
    pmf = 1.0 / torch.arange(1, E + 1, dtype=torch.float64) ** 1.1
    logits = torch.log(pmf / pmf.sum())[perm.argsort()].float()
    gumbel = -torch.log(-torch.log(torch.rand(T, E, generator=g).clamp_min(1e-9)))
    z = logits[None, :] + gumbel
    z[:, perm[-empty:]] = -1e9
    rw, sel = torch.topk(torch.softmax(z, -1), topk, dim=-1)
    rw = rw / rw.sum(-1, keepdim=True)
    return rw.to(torch.bfloat16).to(device), sel.int().to(device)


def dense_module(fmt, N, K, r, alpha, seed, dev):
    from xorl_amd.qlora import QLoRALinear

    lin = torch.nn.Linear(K, N, bias=False, device=dev)
    g = torch.Generator(device=dev).manual_seed(seed)
    with torch.no_grad():
        lin.weight.copy_(torch.randn(N, K, generator=g, device=dev) * 0.02)
    m = QLoRALinear.from_module(lin, r=r, lora_alpha=alpha, quant_format=fmt)
    with torch.no_grad():
        m.lora_A.copy_(torch.randn(r, K, generator=g, device=dev) * 0.02)
        m.lora_B.copy_(torch.randn(N, r, generator=g, device=dev) * 0.02)
    return m


def other_config(cfg: int, dev):
    """Builds BASELINE.json configs[0], [2], [3] or [4] (or the merge passes, 5 and 9, or the NF4 variant of configs[1], 6)
    on the device.  Returns
    (step_fn, work_per_step, unit_is_bytes, workload_text, kernel_text)."""
    lin_flops = lambda m, K, N, r: 4.0 * m * K * N + 6.0 * m * r * (K + N)
    rnd = lambda *shape, seed: torch.randn(*shape, generator=torch.Generator(device=dev).manual_seed(seed),
                                           device=dev).to(torch.bfloat16)
    if cfg == 0:
        m = dense_module("int4", 4096, 4096, 16, 32, 10, dev)
        x, dy = rnd(512, 4096, seed=1).requires_grad_(True), rnd(512, 4096, seed=2)

        def step():
            x.grad = m.lora_A.grad = m.lora_B.grad = None
            m(x).backward(dy)
        return (step, lin_flops(512, 4096, 4096, 16), False,
                "configs[0]: int4 (group 128, bf16 absmax/7 scales) QLoRA linear 4096->4096, M=512, r=16, fwd+bwd",
                "gemm_256_kernel<int4> with 128x128 tiles in 4 K splits + splitk_reduce_kernel (fused dequant-GEMM, forward and dgrad launches)")
    if cfg == 2:
        Mtok, Hd = 4096, 5120
        shapes = {"q": (8192, Hd), "k": (1024, Hd), "v": (1024, Hd), "o": (Hd, 8192)}
        mods = {k: dense_module("nvfp4", N, K, 16, 32, 20 + i, dev) for i, (k, (N, K)) in enumerate(shapes.items())}
        xs = {k: rnd(Mtok, K, seed=30 + i).requires_grad_(True) for i, (k, (N, K)) in enumerate(shapes.items())}
        dys = {k: rnd(Mtok, N, seed=40 + i) for i, (k, (N, K)) in enumerate(shapes.items())}

        def step():
            for k, m in mods.items():
                xs[k].grad = m.lora_A.grad = m.lora_B.grad = None
                m(xs[k]).backward(dys[k])
        return (step, sum(lin_flops(Mtok, K, N, 16) for (N, K) in shapes.values()), False,
                "configs[2]: nvfp4 QLoRA Qwen3-32B attention projections q/k/v/o, hidden 5120, M=4096, r=16, fwd+bwd",
                "gemm_256_kernel<nvfp4> with 256x256 tiles (whole rounds of the chip; trailing tile rows in K splits + splitk_reduce_kernel) and 128x128 tiles (k/v forward and dgrad): fused dequant-GEMM, forward and dgrad launches")
    if cfg in (3, 7, 8):
        # 7 / 8 are not BASELINE configs: configs[3] with the banks held as nvfp4 / NF4 (4-bit GKN storage)
        from xorl_amd.qlora import BlockFP8QLoRAMoeExperts, NF4QLoRAMoeExperts, NvFP4QLoRAMoeExperts

        E, Hd, I, T, topk, r = 128, 2048, 768, 16384, 8, 16
        cls, fmt_name, kfmt = {3: (BlockFP8QLoRAMoeExperts, "block_fp8", "fp8"), 7: (NvFP4QLoRAMoeExperts, "nvfp4", "nvfp4 GKN"),
                               8: (NF4QLoRAMoeExperts, "NF4", "nf4 GKN")}[cfg]
        m = cls(E, E, I, Hd, r=r, lora_alpha=2 * r, hybrid_shared=False).to(dev)
        g = torch.Generator(device=dev).manual_seed(50)
        w = lambda *shape: torch.randn(*shape, generator=g, device=dev) * 0.02
        m.load_weights(w(E, Hd, I), w(E, Hd, I), w(E, I, Hd))
        m = m.to(dev)
        with torch.no_grad():
            for name in ("gate_proj", "up_proj", "down_proj"):
                getattr(m, f"{name}_lora_A").copy_(w(*getattr(m, f"{name}_lora_A").shape))
                getattr(m, f"{name}_lora_B").copy_(w(*getattr(m, f"{name}_lora_B").shape))
        rw, sel = zipf_routing(T, E, topk, seed=3, device=dev)
        counts = torch.bincount(sel.flatten().long(), minlength=E)
        assert int((counts == 0).sum()) >= 1, "the routing must leave some experts empty"
        x, dy = rnd(T, Hd, seed=51).requires_grad_(True), rnd(T, Hd, seed=52)
        params = [p for p in m.parameters() if p.requires_grad]

        def step():
            x.grad = None
            for p in params:
                p.grad = None
            m(x, rw, sel).backward(dy)
        R = T * topk
        return (step, R * (12.0 * Hd * I + 18.0 * r * (Hd + I)), False,
                f"{'configs[3]' if cfg == 3 else 'configs[3] shapes with ' + fmt_name + ' banks (not a BASELINE config)'}: "
                f"grouped {fmt_name} QLoRA Qwen3-30B-A3B experts, E=128, hidden 2048, intermediate 768, "
                f"top-8 of 16384 tokens, Zipf(1.1) counts (max {int(counts.max())}, {int((counts == 0).sum())} empty), "
                f"per-expert r=16, fwd+bwd",
                (f"gemm_dtl16_kernel<contract_cols true|false, 8 waves, grouped> (fused block-fp8 dequant grouped GEMM, "
                 f"forward and dgrad launches)") if cfg == 3 else
                f"gemm_256_kernel<{kfmt}, grouped> (fused dequant grouped GEMM, forward and dgrad launches)")
    if cfg == 4:
        shapes = {"q": (4096, 4096), "kv": (1024, 4096), "gate_up": (12288, 4096), "down": (4096, 12288)}
        cases, total = [], 0.0
        for fmt in ("int4", "block_fp8"):
            for i, (k, (N, K)) in enumerate(shapes.items()):
                m = dense_module(fmt, N, K, 16, 32, 60 + i, dev)
                wbytes = (K * N / 2 + 2 * K * N / 128) if fmt == "int4" else (K * N + 4 * ((K + 127) // 128) * ((N + 127) // 128))
                for Mtok in (1, 8, 32, 64):
                    cases.append((m, rnd(Mtok, K, seed=70 + Mtok)))
                    total += wbytes + 2 * Mtok * K + 2 * Mtok * N + 4 * 16 * (K + N)

        def step():
            with torch.no_grad():
                for m, x in cases:
                    m(x)
        return (step, total, True,
                "configs[4]: skinny-M forward, M in {1,8,32,64} x {q 4096->4096, kv 4096->1024, gate/up 4096->12288, "
                "down 12288->4096} x {int4, block_fp8}, r=16 (32 forwards per step)",
                "skinny_gemv_kernel<int4|fp8> (M = 1, dot products), skinny_rows_kernel<int4|fp8> (M <= 16, one launch) "
                "and skinny_split_kernel<int4|fp8> + skinny_epilogue_kernel (M = 32, 64) (weight-streaming fused "
                "dequant-GEMV/GEMM; the timed region is the whole forward)")
    if cfg == 5:
        # not a BASELINE config: the merge / re-quantise pass over configs[1]'s three block_fp8 weights (r = 32)
        from xorl_amd.functional import merge_dense, merge_requant_fp8

        mods = [dense_module("block_fp8", N, K, 32, 64, 80 + i, dev) for i, (N, K) in
                enumerate(((12288, 4096), (12288, 4096), (4096, 12288)))]
        outs = [(torch.empty(m.out_features, m.in_features, dtype=torch.uint8, device=dev),
                 torch.empty((m.out_features + 127) // 128, (m.in_features + 127) // 128, dtype=torch.float32, device=dev))
                for m in mods]
        total = 0.0
        for m in mods:
            nk = m.out_features * m.in_features
            total += 2 * (nk + 4 * ((m.out_features + 127) // 128) * ((m.in_features + 127) // 128)) + (nk + 2 * nk)

        def step():
            with torch.no_grad():
                for m, (po, so) in zip(mods, outs):
                    merge_requant_fp8(m._quant_weight(), m.lora_A, m.lora_B, 32, 2.0, po, so)
                    merge_dense(m._quant_weight(), m.lora_A, m.lora_B, 32, 2.0, torch.bfloat16)
        return (step, total, True,
                "merge pass (not a BASELINE config): decode + LoRA update + re-encode (block_fp8 -> block_fp8) and "
                "decode + update -> bf16, for gate/up [12288,4096] and down [4096,12288], r=32",
                "merge_kernel<fp8> (fused decode + low-rank update + re-quantise / publish)")
    if cfg == 9:
        # not a BASELINE config: the nvfp4 merge / re-quantise pass over configs[2]'s four weights (r = 16): tensor amax
        # of the merged weight, re-encode against it, and the bf16 publish
        from xorl_amd.functional import merge_amax, merge_dense, merge_requant_nvfp4

        mods = [dense_module("nvfp4", N, K, 16, 32, 120 + i, dev) for i, (N, K) in
                enumerate(((8192, 5120), (1024, 5120), (1024, 5120), (5120, 8192)))]
        total = 0.0
        for m in mods:
            nk = m.out_features * m.in_features
            packed = nk / 2 + nk / 16
            total += packed + 2 * packed + (packed + 2 * nk)       # amax pass reads; requant reads + writes; publish

        def step():
            with torch.no_grad():
                for m in mods:
                    qw = m._quant_weight()
                    amax = merge_amax(qw, m.lora_A, m.lora_B, 16, 2.0)
                    merge_requant_nvfp4(qw, m.lora_A, m.lora_B, 16, 2.0, amax)
                    merge_dense(qw, m.lora_A, m.lora_B, 16, 2.0, torch.bfloat16)
        return (step, total, True,
                "nvfp4 merge pass (not a BASELINE config): tensor amax of decode + LoRA update, re-encode (nvfp4 -> nvfp4) "
                "and decode + update -> bf16, for q [8192,5120], k/v [1024,5120], o [5120,8192], r=16",
                "merge_kernel<nvfp4> (fused decode + low-rank update + amax / re-quantise / publish)")
    if cfg == 6:
        # not a BASELINE config: configs[1]'s three projections held as NF4 (group 64, fp32 absmax scales)
        Mtok = 8192
        shapes = {"gate": (12288, 4096), "up": (12288, 4096), "down": (4096, 12288)}
        mods = {k: dense_module("nf4", N, K, 32, 64, 90 + i, dev) for i, (k, (N, K)) in enumerate(shapes.items())}
        xs = {k: rnd(Mtok, K, seed=94 + i).requires_grad_(True) for i, (k, (N, K)) in enumerate(shapes.items())}
        dys = {k: rnd(Mtok, N, seed=97 + i) for i, (k, (N, K)) in enumerate(shapes.items())}

        def step():
            for k, m in mods.items():
                xs[k].grad = m.lora_A.grad = m.lora_B.grad = None
                m(xs[k]).backward(dys[k])
        return (step, sum(lin_flops(Mtok, K, N, 32) for (N, K) in shapes.values()), False,
                "NF4 (not a BASELINE config): QLoRA Qwen3-8B MLP projections gate/up 4096->12288, down 12288->4096 "
                "as NF4 group 64, M=8192, r=32, fwd+bwd of each linear",
                "gemm_256_kernel<nf4> (fused dequant-GEMM, forward and dgrad launches)")
    raise SystemExit(f"bench.py: unknown --config {cfg}")


def calibrate_copy(dev):
    """One plain elementwise copy of known traffic: 256 MiB read + 256 MiB written."""
    src = torch.ones(64 << 20, dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    torch.mul(src, 1.0, out=dst)
    torch.cuda.synchronize()
    del src, dst


def traffic_of(args, live_avg_launch_ms, cfg=None):
    """-> (traffic bytes or None, provenance text).  The committed counter figure of this config, unless the run's
    own average launch duration says that it times something else than the counters measured."""
    cfg = args.config if cfg is None else cfg
    if args.traffic_bytes is not None and cfg == args.config:
        return args.traffic_bytes, "--traffic-bytes"
    entry = MEASURED_TRAFFIC.get(cfg)
    if entry is None:
        return None, "no counter run committed for this config"
    nbytes, profile, ref_ms = entry
    if live_avg_launch_ms <= 0 or abs(live_avg_launch_ms / ref_ms - 1.0) > 0.10:
        return None, (f"stale: {profile} measured its counters at {ref_ms:.4f} ms per launch, this run averages "
                      f"{live_avg_launch_ms:.4f} ms; re-run the --pmc passes named in that file")
    return nbytes, f"{profile} ({ref_ms:.4f} ms per launch there, {live_avg_launch_ms:.4f} ms here)"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-rows", type=int, default=M,
                    help="token rows of the CPU baseline (0 = skip); default: the whole workload, 2 warm-ups + 5 timed runs "
                         "of about 4.5 s each")
    ap.add_argument("--no-secondary", action="store_true",
                    help="config 1 only: skip the `secondary` measurements (configs[4] decode shapes against the HBM "
                         "roofline, configs[3] grouped experts against the MFMA roofline) that the default run appends")
    ap.add_argument("--config", type=int, default=1,
                    help="BASELINE.json configs index; 1 (default) is the headline workload, the others report the "
                         "same JSON for their own workload (no CPU baseline)")
    ap.add_argument("--unfused", action="store_true",
                    help="config 1 only: call the three QLoRA linears and the SwiGLU kernel one by one instead of the "
                         "fused MLP entry points (same arithmetic; for A/B timing)")
    ap.add_argument("--reference-path", action="store_true",
                    help="config 1 only: run the step the way the reference does -- every weight decoded to bf16 once per step "
                         "(HIP decode kernel) and kept for the backward, library GEMMs (torch -> hipBLASLt) for the base products, "
                         "the LoRA branch in fp32 torch ops (qlora/modules/linear.py:378-382), autograd for the backward -- "
                         "to time that organisation on this GPU beside the fused path; no roofline figure")
    ap.add_argument("--no-graph", action="store_true",
                    help="config 4 only: issue the 32 forwards of a step eagerly instead of replaying them as one HIP graph")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="before the warmup, run one plain 256 MiB -> 256 MiB elementwise copy so that a counter "
                         "run (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) holds a kernel of known traffic to scale by")
    ap.add_argument("--traffic-bytes", type=float, default=None,
                    help="HBM bytes per launch of the roofline kernel from such counter runs (reported as "
                         "roofline.traffic; default: the committed measurement of that config, else null)")
    ap.add_argument("--routed-decode", choices=("block_fp8", "nvfp4", "nf4"), default=None,
                    help="not a BASELINE config: only the routed expert MLP of configs[3]'s banks (in this format) for 1-64 "
                         "tokens, forward only -- the table that the default run carries as its third `secondary` entry")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs the QLoRA path on ONE GPU; --gpus must be 1 "
                 "(no collectives or sharding are part of it)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP device visible")

    from xorl_amd import _C
    from xorl_amd.functional import silu_and_mul

    dev = torch.device("cuda:0")
    if args.routed_decode:
        print(json.dumps({"metric": "routed expert MLP forward for a handful of tokens (not a BASELINE config)", "unit": "GB/s",
                          "n_gpus": 1, "data": "synthetic", "config": {"workload": ROUTED_DECODE_WORKLOAD + "; " + args.routed_decode},
                          "cases": routed_decode_table(dev, fmt=args.routed_decode)}))
        return
    if args.config != 1:
        return run_other(args, dev)
    mods_cpu = build_modules()
    cpu = cpu_baseline(mods_cpu, args.cpu_rows) if args.cpu_rows > 0 else None
    mods = {k: m.to(dev) for k, m in mods_cpu.items()}
    x = gen((M, H), 1.0, 1, torch.bfloat16).to(dev).requires_grad_(True)
    dy = gen((M, H), 1.0, 2, torch.bfloat16).to(dev)
    params = [p for m in mods.values() for p in (m.lora_A, m.lora_B)]

    from xorl_amd.qlora import qlora_mlp_forward

    def reference_linear(m, inp, w):
        lora = (inp.float() @ m.lora_A.t().float()) @ m.lora_B.t().float() * m.scaling
        return torch.nn.functional.linear(inp, w) + lora.to(inp.dtype)

    def step():
        x.grad = None
        for p in params:
            p.grad = None
        if args.reference_path:
            w = {k: m._dequantize_weight().to(torch.bfloat16) for k, m in mods.items()}
            h = silu_and_mul(reference_linear(mods["gate"], x, w["gate"]), reference_linear(mods["up"], x, w["up"]))
            y = reference_linear(mods["down"], h, w["down"])
        elif args.unfused:        # the three modules and the SwiGLU kernel one by one
            y = mods["down"](silu_and_mul(mods["gate"](x), mods["up"](x)))
        else:                     # the same MLP through the library's fused forward / backward (xq_mlp_fwd / xq_mlp_bwd)
            y = qlora_mlp_forward(mods["gate"], mods["up"], mods["down"], x)
        y.backward(dy)

    L = _C.lib()
    if args.calibrate_copy:
        calibrate_copy(dev)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    L.xq_profile_enable(1)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    n, ms, fl = ctypes.c_int(0), ctypes.c_double(0), ctypes.c_double(0)
    _C.check(L.xq_profile_collect(ctypes.byref(n), ctypes.byref(ms), ctypes.byref(fl)))
    L.xq_profile_enable(0)

    ms_per_step = dt / args.steps * 1e3
    value = step_flops(M) / (dt / args.steps) / 1e12
    achieved = fl.value / (ms.value * 1e-3) / 1e12 if ms.value > 0 else 0.0
    avg_launch_ms = ms.value / max(n.value, 1)
    traffic, traffic_source = traffic_of(args, avg_launch_ms)
    out = {
        "metric": METRIC,
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "configs[1]: block_fp8 QLoRA Qwen3-8B MLP fwd+bwd, M=8192, hidden 4096, "
                               "intermediate 12288, LoRA r=32 on gate/up/down, SwiGLU",
                   "tokens": M, "hidden": H, "intermediate": I, "lora_r": R, "format": "block_fp8"},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": BF16_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / BF16_MFMA_PEAK_TFLOPS, "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": "gemm_dtl16_kernel<contract_cols true|false, 8 waves> (dense fused block-fp8 dequant-GEMM, "
                               "256x256x64 tiles: gate, up and down forward, down dgrad, gate+up dgrad as one sum)"
                               if not args.unfused else
                               "gemm_dtl16_kernel<contract_cols true|false, 8 waves> (dense fused block-fp8 dequant-GEMM, "
                               "forward and dgrad launches)",
                     "launches": n.value, "avg_launch_ms": avg_launch_ms},
        "cpu_baseline": cpu,
    }
    if args.reference_path:
        out["path"] = "reference organisation: decode to bf16 + library GEMMs + fp32 LoRA branch + autograd (not the product path)"
        out["roofline"] = None
    elif not args.unfused and not args.no_secondary:
        del mods, x, dy, params
        torch.cuda.empty_cache()
        out["secondary"] = secondary_measurements(args, dev)
    print(json.dumps(out))


def measure_other(args, dev, cfg, steps, warmup):
    """One of the other workloads, measured like the headline one -> the dict of its JSON line."""
    from xorl_amd import _C

    step, work, is_bytes, workload, kernel = other_config(cfg, dev)
    L = _C.lib()
    if args.calibrate_copy:
        calibrate_copy(dev)
    use_graph = cfg == 4 and not args.no_graph
    if use_graph:
        # the decode-regime step is 32 launch-bound forwards: replay it as one HIP graph (what a serving loop
        # does).  Captured after an eager warm-up on a side stream; every replay runs the same kernels on the
        # same buffers.  The per-forward roofline figure is taken from eager steps after the timed region,
        # because event records inside a graph cannot be read back.
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        run = graph.replay
        workload += "; the step is replayed as one HIP graph"
    else:
        run = step
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    if not use_graph:
        L.xq_profile_enable(1)
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    if use_graph:
        L.xq_profile_enable(1)
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
    n, ms, fl = ctypes.c_int(0), ctypes.c_double(0), ctypes.c_double(0)
    _C.check(L.xq_profile_collect(ctypes.byref(n), ctypes.byref(ms), ctypes.byref(fl)))
    L.xq_profile_enable(0)
    scale, unit, peak = (1e9, "GB/s", 8000.0) if is_bytes else (1e12, "TFLOP/s", BF16_MFMA_PEAK_TFLOPS)
    achieved = fl.value / (ms.value * 1e-3) / scale if ms.value > 0 else 0.0
    avg_launch_ms = ms.value / max(n.value, 1)
    traffic, traffic_source = traffic_of(args, avg_launch_ms, cfg)
    return {
        "metric": METRIC, "value": work / dt / scale, "unit": unit, "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic", "config": {"workload": workload},
        "roofline": {"bound": "hbm" if is_bytes else "mfma", "achieved": achieved, "peak": peak, "unit": unit,
                     "frac": achieved / peak, "traffic": traffic, "traffic_source": traffic_source, "kernel": kernel,
                     "launches": n.value, "avg_launch_ms": avg_launch_ms},
        "cpu_baseline": None}


def run_other(args, dev):
    print(json.dumps(measure_other(args, dev, args.config, args.steps, args.warmup)))


# ---- configs[4] case by case: microseconds and GB/s of every (format, projection, M) forward
DECODE_SHAPES = {"q": (4096, 4096), "kv": (1024, 4096), "gate_up": (12288, 4096), "down": (4096, 12288),
                 "gate|up fused": (24576, 4096)}       # the last one is the reference's default fused module, not a configs[4] case
COLD_FOOTPRINT = 640 << 20      # bytes of weight copies a case rotates through: 2.5 x the 256 MB memory-side cache


def _graph_time_us(run, pool, reps: int, replays: int) -> float:
    """`run()` (which makes `reps` launches) captured as one HIP graph after an eager warm-up on a side stream; the median
    over `replays` replays of the time per launch, events on the launch stream."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, pool=pool):
        run()
    graph.replay()
    torch.cuda.synchronize()
    times = []
    for _ in range(replays):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1) * 1e3 / reps)
    del graph
    return sorted(times)[len(times) // 2]


def _read_probe(t, out):
    from xorl_amd import _C

    _C.check(_C.lib().xq_read_probe(t.data_ptr(), t.numel() * t.element_size(), out.data_ptr(), _C.stream_ptr(t.device)))


def decode_case_table(dev, reps: int = 24, replays: int = 5):
    """Every configs[4] forward on its own: `reps` forwards back to back as one HIP graph (launch boundaries included, no
    host time), timed with events on the launch stream, median of `replays` replays.  Two figures per case: "cold" rotates
    through copies of the weight whose total size exceeds the 256 MB memory-side cache, so every byte comes from HBM as it
    does in a model whose layers do not fit that cache (this is the roofline figure); "hot" replays one weight, which
    that cache may serve.  `read_probe_*`: a kernel that only reads the weight's packed bytes, timed the same way -- the
    measured ceiling for a one-shot read of that size, launch boundary included."""
    from xorl_amd.functional import QuantWeight, qlora_linear

    rows = []
    g = torch.Generator(device=dev).manual_seed(7)
    # one memory pool for all the graphs: the forwards' workspaces then sit at the same few addresses in every graph, and
    # the library's per-workspace slots (which stay with a captured workspace for good) are not used up case by case
    pool = torch.cuda.graph_pool_handle()
    probe_out = torch.zeros(1, dtype=torch.int32, device=dev)
    for fmt in ("int4", "block_fp8"):
        for name, (N, K) in DECODE_SHAPES.items():
            m = dense_module(fmt, N, K, 16, 32, 60, dev)
            qw = m._quant_weight()
            wbytes = qw.packed.numel() * qw.packed.element_size() + qw.scales.numel() * qw.scales.element_size()
            n_copies = max(2, -(-COLD_FOOTPRINT // wbytes))
            copies = [qw] + [QuantWeight(qw.fmt, qw.layout, qw.packed.clone(), qw.scales.clone(), qw.scale_dtype, qw.rows, qw.cols,
                                         qw.group, global_scale=qw.global_scale) for _ in range(n_copies - 1)]
            A, B, sc = m.lora_A.detach(), m.lora_B.detach(), m.scaling
            # the measured ceiling for this weight: a kernel that only reads the packed bytes, in the same kind of graph
            read_us = {}
            for mode, ws in (("cold", copies), ("hot", copies[:1])):
                read_us[mode] = _graph_time_us(lambda: [_read_probe(ws[i % len(ws)].packed, probe_out) for i in range(reps)], pool, reps,
                                               replays)
            pbytes = qw.packed.numel() * qw.packed.element_size()
            for Mtok in (1, 8, 32, 64):
                x = torch.randn(Mtok, K, generator=g, device=dev).to(torch.bfloat16)
                algo = wbytes + 2 * Mtok * K + 2 * Mtok * N + 4 * 16 * (K + N)
                us = {}
                for mode, ws in (("cold", copies), ("hot", copies[:1])):
                    def run():
                        with torch.no_grad():
                            for i in range(reps):
                                qlora_linear(x, ws[i % len(ws)], A, B, 16, sc)
                    us[mode] = _graph_time_us(run, pool, reps, replays)
                rows.append({"format": fmt, "proj": name, "N": N, "K": K, "M": Mtok, "bytes": algo,
                             "us": round(us["cold"], 2), "GBps": round(algo / us["cold"] / 1e3, 1),
                             "frac": round(algo / us["cold"] / 1e3 / 8000.0, 4),
                             "us_hot": round(us["hot"], 2), "GBps_hot": round(algo / us["hot"] / 1e3, 1),
                             "read_probe_us": round(read_us["cold"], 2), "read_probe_GBps": round(pbytes / read_us["cold"] / 1e3, 1),
                             "read_probe_us_hot": round(read_us["hot"], 2)})
            del copies, m, qw
            torch.cuda.empty_cache()
    return rows


ROUTED_DECODE_WORKLOAD = ("the routed expert MLP of configs[3]'s banks (E=128, hidden 2048, intermediate 768, top-8, r=16) for 1-64 "
                          "tokens, forward only, nothing differentiated; per forward, 16 routings per HIP graph (touched experts "
                          "from HBM); `bytes` = packed bytes of the touched experts")


def routed_decode_table(dev, sets: int = 16, replays: int = 5, fmt: str = "block_fp8"):
    """The routed expert MLP of configs[3]'s banks for a handful of tokens with nothing to differentiate: the
    weight-streaming form (xq_grouped_fwd_infer) beside the training forward (xq_grouped_fwd) on the same calls, `sets`
    forwards with different routings per HIP graph so that the touched experts come from HBM."""
    import xorl_amd.moe_functional as MF
    from xorl_amd.qlora import BlockFP8QLoRAMoeExperts, NF4QLoRAMoeExperts, NvFP4QLoRAMoeExperts

    E, Hd, I, topk, r = 128, 2048, 768, 8, 16
    cls = {"nvfp4": NvFP4QLoRAMoeExperts, "nf4": NF4QLoRAMoeExperts}.get(fmt, BlockFP8QLoRAMoeExperts)
    per_expert = {"nvfp4": Hd * I // 2 + Hd * I // 16 + 4, "nf4": Hd * I // 2 + Hd * I // 64 * 4}.get(fmt, Hd * I + (Hd // 128) * (I // 128) * 4)
    m = cls(E, E, I, Hd, r=r, lora_alpha=2 * r, hybrid_shared=False).to(dev)
    g = torch.Generator(device=dev).manual_seed(50)
    w = lambda *shape: torch.randn(*shape, generator=g, device=dev) * 0.02
    m.load_weights(w(E, Hd, I), w(E, Hd, I), w(E, I, Hd))
    m = m.to(dev)
    pool = torch.cuda.graph_pool_handle()
    rows = []
    for T in (1, 4, 8, 16, 64):
        calls = []
        for i in range(sets):
            rw, sel = zipf_routing(max(T, 8), E, topk, seed=3 + i, device=dev)
            calls.append((torch.randn(T, Hd, generator=g, device=dev).to(torch.bfloat16), rw[:T].contiguous(), sel[:T].contiguous()))
        touched = sum(int(torch.unique(c[2]).numel()) for c in calls) / sets
        nbytes = touched * 3 * per_expert
        us = {}
        for name, on in (("streaming", True), ("training_forward", False)):
            MF.DECODE_PATH = on

            def run():
                with torch.no_grad():
                    for c in calls:
                        m(*c)
            us[name] = _graph_time_us(run, pool, sets, replays)
        MF.DECODE_PATH = True
        rows.append({"tokens": T, "experts_touched": touched, "bytes": nbytes, "us": us["streaming"],
                     "GBps": nbytes / us["streaming"] / 1e3, "frac": nbytes / us["streaming"] / 1e3 / 8000.0,
                     "us_training_forward": us["training_forward"]})
    del m
    torch.cuda.empty_cache()
    return rows


def secondary_measurements(args, dev):
    """The other two regimes of the path, measured in the same run as the headline line: configs[4] (skinny M, HBM
    roofline; per case and over the 32 BASELINE cases) and configs[3] (grouped experts, MFMA roofline)."""
    out = []
    table = decode_case_table(dev)
    base = [r for r in table if r["proj"] != "gate|up fused"]
    tot_b, tot_us = sum(r["bytes"] for r in base), sum(r["us"] for r in base)
    agg = tot_b / tot_us / 1e3
    c4 = measure_other(args, dev, 4, 20, 5)
    out.append({
        "workload": "configs[4]: skinny-M forward, M in {1,8,32,64} x {q, kv, gate/up, down of Qwen3-8B} x {int4, block_fp8}, r=16; "
                    "`cases` times every forward on its own (24 back to back in one HIP graph, weights rotating through "
                    f"{COLD_FOOTPRINT >> 20} MiB of copies so that they come from HBM; *_hot: one weight replayed, which the 256 MB "
                    "memory-side cache may serve; read_probe_*: a kernel that only reads the packed bytes, timed the same way); `achieved` is "
                    "the 32 BASELINE cases' bytes over the sum of their times; "
                    "`graph_step` replays the 32 forwards on one set of weights as one HIP graph",
        "bound": "hbm", "achieved": agg, "peak": 8000.0, "unit": "GB/s", "frac": agg / 8000.0,
        "traffic": c4["roofline"]["traffic"], "traffic_source": c4["roofline"]["traffic_source"],
        "kernel": c4["roofline"]["kernel"],
        "graph_step": {"value": c4["value"], "unit": "GB/s", "ms_per_step": c4["ms_per_step"],
                       "eager_per_forward_achieved": c4["roofline"]["achieved"], "avg_forward_ms": c4["roofline"]["avg_launch_ms"]},
        "cases": table,
    })
    torch.cuda.empty_cache()
    c3 = measure_other(args, dev, 3, 10, 3)
    out.append({"workload": c3["config"]["workload"], "value": c3["value"], "unit": "TFLOP/s", "ms_per_step": c3["ms_per_step"],
                **c3["roofline"]})
    torch.cuda.empty_cache()
    out.append({"workload": "not a BASELINE config: " + ROUTED_DECODE_WORKLOAD + "; block_fp8",
                "bound": "hbm", "peak": 8000.0, "unit": "GB/s",
                "kernel": "decode_stream_kernel (+ decode_route / decode_mid / decode_final), xq_grouped_fwd_infer",
                "cases": routed_decode_table(dev)})
    return out


if __name__ == "__main__":
    main()
