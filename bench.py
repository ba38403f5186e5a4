#!/usr/bin/env python3
"""Benchmark of the quantized-weight matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]            # all five configurations
    python bench.py --workload NAME [...]                          # one workload

A step is one pass of the hot path over one batch of synthetic input, inputs
already resident in HBM.  Decode workloads rotate over enough distinct copies of
the weights (>= 512 MiB) that no launch can be served by the 256 MiB Infinity
Cache.  The timed region is a HIP graph holding exactly K steps (the path is
launch-bound at ~2-5 us per kernel otherwise), replayed between two
synchronisations; `ms_per_step` is the median over the replays of that host-clocked
time per step, and the replays' event-clocked median and 10th / 90th percentile are
reported beside it.  One JSON line is printed.

With no --workload the line's headline is configs[2] (the MoE decode layer, the
configuration the metric is quoted on) and `extra.configs` carries every
configuration of the baseline with its own value, roofline, CPU baseline and
parity: configs[0] (FP8 GEMV), configs[1] at B = 1, 4, 8 (MXFP4 GEMV),
configs[3] at M=512,N=7168 (the metric's "M=512") and M=4096,N=18432 (FP8 GEMM),
configs[4] (MoE prefill layer) and configs[2].
"""
from __future__ import annotations

import argparse
import json
import math
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
ROTATE_BYTES = 512 << 20       # >= 2x the 256 MiB Infinity Cache
SEED_BASE = 0xF3771E


def traffic_from_profile(name: str | None, kernels: tuple[str, ...]):
    """HBM bytes per launch of the named kernels (read + write, summed over `kernels`) from the
    hardware-counter table of profiles/<name>: two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE)
    scaled by a plain copy of known size; the summary holds the commands.  None when the summary
    or a kernel's row is missing, so a renamed kernel cannot leave a stale figure behind."""
    if not name:
        return None
    path = os.path.join(ROOT, "profiles", name)
    if not os.path.exists(path):
        return None
    rows, in_table = {}, False
    for line in open(path):
        if "HBM read MB" in line:
            in_table = True
            continue
        if in_table:
            m = re.match(r"\s+(\S.*?)\s+(\d+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s*$", line)
            if m:
                rows[m.group(1)] = (float(m.group(5)) + float(m.group(6))) * 1e6
    total = 0.0
    for kernel in kernels:
        # "name+": a step launches several instantiations of the kernel, sum them all
        every = kernel.endswith("+")
        hit = [v for k, v in rows.items() if k.startswith(kernel.rstrip("+"))]
        if not hit:
            return None
        total += sum(hit) if every else max(hit)
    return int(total)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="steps of the timed region; default 50 (MoE decode, FP8 GEMM), 10 (MoE prefill), 200 (others)")
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="all",
                    choices=["all", "moe_decode", "mxfp4_gemv", "fp8_gemv", "dense_ffn", "shared_ffn", "fp8_gemm", "moe_prefill", "router",
                             "routing_chain", "expert_upload", "hc_producer"])
    ap.add_argument("--batch", type=int, default=1, help="tokens per GEMV step (1, 4 or 8)")
    ap.add_argument("--matrices", type=int, default=1,
                    help="GEMV workloads: independent matrices (distinct weight copies) per launch, 1..32")
    ap.add_argument("--m", type=int, default=512,
                    help="rows of the FP8 GEMM workload (512, 2048, 4096; up to 32 rows are a decode batch, an HBM-bound "
                         "step) and of the shared FFN workload")
    ap.add_argument("--tile-schedule", action="store_true",
                    help="shared_ffn: keep the MFMA tile schedule for a decode batch (for comparison)")
    ap.add_argument("--n", type=int, default=7168, help="output features of the FP8 GEMM workload (7168, 18432)")
    ap.add_argument("--tokens", type=int, default=8192, help="tokens of the MoE prefill workload")
    ap.add_argument("--decode-tokens", type=int, default=64,
                    help="tokens of the MoE decode workload (configs[2] is 64; with fewer than about 16 the active "
                         "experts fit the 256 MiB Infinity Cache and the figure is no longer an HBM rate)")
    ap.add_argument("--hot-experts", type=int, default=0,
                    help="MoE decode: route every token into the first N experts only (concentrated routing)")
    ap.add_argument("--decode-shape", default=None,
                    help="MoE decode: HIDDEN,INTERMEDIATE,TOPK of another model's layer, e.g. 4096,2048,6 "
                         "(DeepSeek-V4 Flash); the default is BASELINE.json's 7168,2048,8")
    ap.add_argument("--capacity-bound", dest="known_groups", action="store_false",
                    help="MoE decode: withhold the host's routed slot ids, so that the layer chooses its regime "
                         "from the slot capacity instead of the batch's distinct experts (the default passes them)")
    ap.add_argument("--weight-order", "--expert-order", dest="expert_order", choices=("block-major", "row-major"),
                    default="block-major",
                    help="MXFP4 decode workloads: weights as prepared at upload / slot install (default) or in "
                         "checkpoint order")
    ap.add_argument("--cpu-seconds", type=float, default=10.0,
                    help="budget of the headline's CPU baseline leg (the other configurations of the default run "
                         "get a third of it each)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch one plain 256 MiB -> 256 MiB elementwise copy, the known-size kernel that "
                         "hardware-counter runs are scaled by")
    return ap.parse_args()


# ----------------------------------------------------------------------------- workloads

class GemvWorkload:
    """configs[1]: MXFP4 dense GEMV N=4096, K=7168 (fused gate+up), BF16 in/out;
    or configs[0] on the GPU: FP8 N=K=4096 with fp32 128x128 block scales."""

    def __init__(self, ctx, name: str, batch: int, weight_order: str = "block-major", matrices: int = 1):
        import torch

        from ferrule_amd.provider import HipArtifactLinearShape as S

        self.ctx, self.name, self.batch, self.matrices = ctx, name, batch, matrices
        if name == "mxfp4_gemv":
            self.profile = "mxfp4_gemv_config2.txt" if batch == 1 else f"mxfp4_gemv_config2_batch{batch}.txt"
        else:
            self.profile = "fp8_gemv_config1.txt" if batch == 1 else None
        self.profile_kernels = ("skinny_gemv_kernel",)
        self.dominant = "skinny_gemv_kernel"
        gen = torch.Generator(device="cuda").manual_seed(SEED_BASE + 2)
        if name == "mxfp4_gemv":
            self.n, self.k = 4096, 7168
            w = torch.randn((self.n, self.k), generator=gen, device="cuda", dtype=torch.float32) * 0.02
            packed, scales = ctx.pack_fp4_rows_from_f32(w)          # the reference's FP4 recipe, on device
            self.shape = S.fp4_e2m1_packed_with_e8m0_scale(self.n, self.k)
            self.label = f"configs[1] MXFP4 dense GEMV N=4096 K=7168 B={batch}"
        else:
            self.n, self.k = 4096, 4096
            w = torch.randn((self.n, self.k), generator=gen, device="cuda", dtype=torch.float32) * 0.02
            tiles = w.reshape(32, 128, 32, 128)
            scales = (tiles.abs().amax(dim=(1, 3)) / 448.0).contiguous()                 # fp32 [32,32]
            q = (tiles / scales[:, None, :, None]).clamp(-448, 448).reshape(self.n, self.k)
            packed = q.to(torch.float8_e4m3fn).view(torch.uint8)
            self.shape = S.fp8_e4m3_with_f32_scale(self.n, self.k)
            self.label = f"configs[0] FP8 GEMV N=K=4096 fp32 block scales B={batch}"
        wb, sb = self.shape.storage_lengths()
        self.bytes_per_step = matrices * (wb + sb + batch * self.k * 2 + batch * self.n * 2)
        self.flops_per_step = matrices * 2 * self.n * self.k * batch
        copies = -(-ROTATE_BYTES // (wb + sb))
        from ferrule_amd.provider import HipArtifactLinearHandle

        self.handles = [HipArtifactLinearHandle(self.shape, packed.reshape(-1).clone(), scales.reshape(-1).clone())
                        for _ in range(copies)]
        if weight_order == "block-major":
            # the one-off reorder done when the artifact is uploaded (not part of a step)
            prepare = ctx.prepare_mxfp4_block_major if name == "mxfp4_gemv" else ctx.prepare_fp8_block_major
            self.handles = [prepare(h) for h in self.handles]
            self.label += ", block-major weights"
        self.x = torch.randn((batch, self.k), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
        self.out = torch.empty((batch, self.n), dtype=torch.bfloat16, device="cuda")
        self.outs = [self.out] + [torch.empty_like(self.out) for _ in range(matrices - 1)]
        self.host = (packed.cpu().numpy(), scales.cpu().numpy(), self.x.float().cpu().numpy())
        self.cursor = 0
        if matrices > 1:
            self.label += f", {matrices} matrices per launch"
            self.profile = f"mxfp4_gemv_config2_{matrices}_matrices.txt" if name == "mxfp4_gemv" and batch == 1 else None
            self.profile_kernels = ("skinny_gemv_multi_kernel",)
            self.dominant = "skinny_gemv_multi_kernel"

    def step(self):
        if self.matrices == 1:
            self.ctx.artifact_linear_gemv_bf16_into(self.handles[self.cursor % len(self.handles)], self.x, self.out)
            self.cursor += 1
            return
        picked = [self.handles[(self.cursor + i) % len(self.handles)] for i in range(self.matrices)]
        self.ctx.artifact_linears_gemv_bf16_into(picked, [self.x] * self.matrices, self.outs)
        self.cursor += self.matrices

    def check(self):
        """Parity of the last output against the CPU checker (the checker is not timed here)."""
        import numpy as np
        import torch

        from oracle import parity
        from oracle import pyoracle as po

        w, s, x = self.host
        self.step()
        torch.cuda.synchronize()
        ax = np.abs(x.astype(np.float64))
        if self.name == "mxfp4_gemv":
            want = po.linear_fp4(w, s, self.n, self.k, x, threads=8)
            absprod = np.stack([po.abs_linear_fp4(w, s, self.n, self.k, row, threads=8) for row in ax])
        else:
            want = po.linear_fp8(w, s, self.n, self.k, x, threads=8)
            absprod = np.stack([po.abs_linear_fp8(w, s, self.n, self.k, row, threads=8) for row in ax])
        worst, decided = 0, 0
        for out in self.outs:       # every matrix of a multi-matrix launch (they hold the same weights)
            w1, d1 = parity.compare_bf16(out.view(torch.int16).cpu().numpy().view(np.uint16), want, absprod, self.k)
            worst, decided = max(worst, w1), decided + d1
        return {"max_bf16_ulp": worst, "decided_by_error_bound": decided, "elements": int(want.size) * len(self.outs),
                "sample": "every output of the timed batch, every matrix of the launch, against the CPU matvec"}

    def cpu_baseline(self, seconds: float):
        """The reference's CPU path as it really runs (dequantize the whole matrix to f32 on
        every call, then the sequential matvec), one thread, timed for about `seconds`."""
        from oracle import pyoracle as po

        w, s, x = self.host
        fn = (lambda: po.linear_fp4(w, s, self.n, self.k, x[:1], materialized=True)) if self.name == "mxfp4_gemv" \
            else (lambda: po.linear_fp8(w, s, self.n, self.k, x[:1], materialized=True))
        fn()
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or time.perf_counter() - t0 < seconds:
            fn()
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        one_token_bytes = self.bytes_per_step // self.matrices - (self.batch - 1) * (self.k * 2 + self.n * 2)
        port = {"value": one_token_bytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{reps} full single-token calls of the same matrix, whole-matrix dequant per call "
                          f"as in LinearWeight::reference_matvec ({dt * 1e3:.1f} ms each)"}
        threads = min(16, os.cpu_count() or 1)
        fused = (lambda: po.linear_fp4(w, s, self.n, self.k, x[:1], threads=threads)) if self.name == "mxfp4_gemv" \
            else (lambda: po.linear_fp8(w, s, self.n, self.k, x[:1], threads=threads))
        fused()
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or time.perf_counter() - t0 < min(3.0, seconds):
            fused()
            reps += 1
        dt2 = (time.perf_counter() - t0) / reps
        multi = {"value": one_token_bytes / dt2 / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                 "sample": f"{reps} calls, rows split over {threads} threads, dequant fused into the dot product"}
        return port, multi


class DenseFfnWorkload:
    """Dense SwiGLU FFN of a decode batch in GEMV form at DeepSeek-V4's shared-expert shape
    (4096 -> 2048 -> 4096, FP8 e4m3 with E8M0 128x128 block scales, BF16 activations): gate and up as
    two matrices of one GEMV launch, then down, which forms silu(gate) * up from the two rows of f32 sums as
    it stages them.  Two launches per step; weight copies rotate."""

    input_size, inter, output_size = 4096, 2048, 4096

    def __init__(self, ctx, batch: int, weight_order: str = "block-major"):
        import torch

        from ferrule_amd import synthetic

        self.ctx, self.batch = ctx, batch
        gen = torch.Generator(device="cuda").manual_seed(SEED_BASE + 12)
        shapes = ((self.inter, self.input_size), (self.inter, self.input_size), (self.output_size, self.inter))
        first = [synthetic.device_fp8_linear(ctx, gen, n, k, "e8m0") for n, k in shapes]
        weight_bytes = sum(h.weight.numel() + h.scale.numel() for h in first)
        copies = -(-ROTATE_BYTES // weight_bytes)
        from ferrule_amd.provider import HipArtifactLinearHandle

        self.sets = [first] + [[HipArtifactLinearHandle(h.shape, h.weight.clone(), h.scale.clone()) for h in first]
                               for _ in range(copies - 1)]
        self.row_major = first
        if weight_order == "block-major":
            self.sets = [[ctx.prepare_fp8_block_major(h) for h in trio] for trio in self.sets]
        self.handles = self.sets
        self.x = torch.randn((batch, self.input_size), generator=gen, device="cuda").to(torch.bfloat16)
        self.out = torch.empty((batch, self.output_size), dtype=torch.bfloat16, device="cuda")
        self.hidden = torch.empty((2, batch, self.inter), dtype=torch.float32, device="cuda")
        self.bytes_per_step = weight_bytes + batch * (self.input_size * 2 + self.inter * 16 + self.output_size * 2)
        self.flops_per_step = 2 * batch * 3 * self.inter * self.input_size
        self.dominant = "skinny_gemv_multi_kernel (gate, up) + skinny_gemv_kernel (SwiGLU input)"
        self.profile = "dense_ffn_decode_4096_2048.txt" if batch == 1 else None
        self.profile_kernels = ("skinny_gemv_multi_kernel", "skinny_gemv_kernel")
        self.label = (f"dense SwiGLU FFN, decode batch {batch}: {self.input_size} -> {self.inter} -> {self.output_size}, "
                      f"FP8 e4m3 weights with E8M0 block scales, {weight_order} weights")
        self.cursor = 0

    def step(self):
        g, u, d = self.sets[self.cursor % len(self.sets)]
        self.ctx.dense_ffn_decode(g, u, d, self.x, out=self.out, hidden=self.hidden)
        self.cursor += 1

    def _host(self):
        return [(h.weight.cpu().numpy().reshape(h.shape.out_features, -1),
                 h.scale.cpu().numpy().reshape(h.shape.out_features // 128, -1)) for h in self.row_major]

    def check(self):
        import numpy as np
        import torch

        from oracle import parity

        self.cursor = 0
        self.step()
        torch.cuda.synchronize()
        host = self._host()
        x = self.x.float().cpu().numpy()
        bits = self.out.view(torch.int16).cpu().numpy().view(np.uint16)
        worst, decided = 0, 0
        rows = sorted({0, self.batch - 1})
        for b in rows:
            want, bound, _ = parity.swiglu_ffn_reference(("fp8", 128, 128), *host, self.input_size, self.inter,
                                                         self.output_size, x[b], threads=8)
            w_, d_, _ = parity.compare_bf16_bounded(bits[b], want, bound, max_decided_fraction=0.005)
            worst, decided = max(worst, w_), decided + d_
        return {"max_bf16_ulp": worst, "decided_by_error_bound": decided, "elements": len(rows) * self.output_size,
                "sample": f"{len(rows)} rows of the timed batch against the CPU chain (SwiGluFfn::reference_execute)"}

    def cpu_baseline(self, seconds: float):
        from oracle import pyoracle as po

        (gw, gs), (uw, us), (dw, ds) = self._host()
        x = self.x.float().cpu().numpy()[0]

        def chain(**kw):
            g = po.linear_fp8(gw, gs, self.inter, self.input_size, x, **kw)[0]
            u = po.linear_fp8(uw, us, self.inter, self.input_size, x, **kw)[0]
            h = (g / (1 + __import__("numpy").exp(-g)) * u).astype("float32")
            po.linear_fp8(dw, ds, self.output_size, self.inter, h, **kw)

        one_row = self.bytes_per_step - (self.batch - 1) * (self.input_size * 2 + self.inter * 16 + self.output_size * 2)
        results = []
        for kw, budget, what in (({"materialized": True}, seconds, "whole-matrix dequant per linear as in LinearWeight::reference_matvec"),
                                 ({"threads": min(16, os.cpu_count() or 1)}, min(3.0, seconds), "rows split over the threads, dequant fused")):
            chain(**kw)
            reps, t0 = 0, time.perf_counter()
            while reps < 2 or time.perf_counter() - t0 < budget:
                chain(**kw)
                reps += 1
            dt = (time.perf_counter() - t0) / reps
            results.append({"value": one_row / dt / 1e9, "unit": "GB/s", "cores": kw.get("threads", 1), "kind": "port",
                            "sample": f"{reps} single-row FFN calls ({dt * 1e3:.1f} ms each), {what}"})
        return results[0], results[1]


class MoeDecodeWorkload:
    """configs[2]: MoE decode layer, 64 tokens, hidden 7168, 256 MXFP4 experts (gate+up
    [4096,7168] as two [2048,7168] matrices, down [7168,2048]), top-8 routing with expert ids
    drawn uniformly without replacement and softmax router weights.  A step is the whole
    layer: invocation flag reset and route plan (one fused launch), gate/up+SwiGLU, down, ranked combine
    with the single BF16 writeback.  The 5 GB of active expert weights exceed the 256 MiB
    Infinity Cache 20-fold, so every step streams them from HBM without rotation."""

    tokens, k, experts, hidden, inter = 64, 8, 256, 7168, 2048

    def __init__(self, ctx, expert_order="block-major", tokens=64, hot_experts=0, experts=None, known_groups=False,
                 shape=None):
        import numpy as np
        import torch

        if shape is not None:      # (hidden, routed intermediate, top-k): another model's layer
            self.hidden, self.inter, self.k = shape

        from ferrule_amd import synthetic

        self.tokens = tokens
        self.ctx = ctx
        if experts is None:
            experts = synthetic.build_device_experts(ctx, self.experts, self.hidden, self.inter, SEED_BASE + 3)
        self.table, self.handles = experts
        self.expert_order = expert_order
        if expert_order == "block-major":
            # the one-off reorder an expert gets when it is installed in a slot (not part of a step);
            # the row-major handles stay for the CPU check
            self.table = synthetic.block_major_table(ctx, self.handles)
        rng = synthetic.rng_for(3)
        self.x_host = synthetic.bf16_activations(rng, (self.tokens, self.hidden))
        if hot_experts:
            self.ids, self.weights = synthetic.concentrated_routing(rng, self.tokens, self.k, self.experts, hot_experts)
        else:
            self.ids, self.weights = synthetic.uniform_routing(rng, self.tokens, self.k, self.experts)
        self.x = torch.from_numpy(self.x_host).to(torch.bfloat16).cuda()
        self.slots = torch.from_numpy(self.ids.ravel().astype(np.int32)).cuda()
        self.gens = torch.ones(self.tokens * self.k, dtype=torch.int32, device="cuda")
        self.wts = torch.from_numpy(self.weights.ravel()).cuda()
        self.out = torch.empty((self.tokens, self.hidden), dtype=torch.bfloat16, device="cuda")
        self.plan = ctx.expert_group_route_plan(self.experts, self.tokens * self.k, self.tokens, self.hidden,
                                                self.inter, self.hidden)
        self.distinct = int(len(np.unique(self.ids)))
        per_matrix = lambda n, kk: n * kk // 2 + n * kk // 32
        self.gate_up_weight_bytes = self.distinct * 2 * per_matrix(self.inter, self.hidden)
        self.down_weight_bytes = self.distinct * per_matrix(self.hidden, self.inter)
        # A small batch activates few experts (one token: top-k of them, 187 MB), which would stay in the
        # 256 MiB Infinity Cache from one step to the next; successive steps then take other routings
        # (as successive layers of a model do), so that the weights of a step come from HBM.
        self.routings = [(self.slots, self.wts, self.ids.ravel().tolist())]
        weight_bytes = self.gate_up_weight_bytes + self.down_weight_bytes
        if not hot_experts and weight_bytes < ROTATE_BYTES:
            distinct = [self.distinct]
            for _ in range(min(15, -(-2 * ROTATE_BYTES // weight_bytes))):
                ids, weights = synthetic.uniform_routing(rng, self.tokens, self.k, self.experts)
                self.routings.append((torch.from_numpy(ids.ravel().astype(np.int32)).cuda(),
                                      torch.from_numpy(weights.ravel()).cuda(), ids.ravel().tolist()))
                distinct.append(int(len(np.unique(ids))))
            mean = sum(distinct) / len(distinct)
            self.gate_up_weight_bytes = int(mean * 2 * per_matrix(self.inter, self.hidden))
            self.down_weight_bytes = int(mean * per_matrix(self.hidden, self.inter))
        self.turn = 0
        act = self.tokens * self.hidden * 2
        self.bytes_per_step = self.gate_up_weight_bytes + self.down_weight_bytes + act + self.tokens * self.k * 8 + act
        self.flops_per_step = self.tokens * self.k * 2 * (2 * self.inter * self.hidden + self.hidden * self.inter)
        # dominant kernel: gate/up streams 2/3 of the weights, reads x, writes h in f32
        self.dominant = "moe_gate_up_kernel"
        self.dominant_bytes = self.gate_up_weight_bytes + act + self.tokens * self.k * self.inter * 4
        baseline_shape = (self.hidden, self.inter, self.k) == (7168, 2048, 8)
        self.label = (f"{'configs[2] ' if self.tokens == 64 and not hot_experts and baseline_shape else ''}MoE decode layer: {self.tokens} "
                      f"tokens, hidden {self.hidden}, {self.experts} MXFP4 experts, top-{self.k} ({self.distinct} "
                      f"distinct experts active{', routes concentrated on them' if hot_experts else ''}), "
                      f"{expert_order} expert weights")
        self.rotated = len(self.routings)
        # The host holds the routed slot ids of this batch (it uploaded them), so the plan call derives the
        # number of active expert groups from them and the layer chooses its regime from that count;
        # --capacity-bound withholds them: the layer then sees the slot capacity only.
        self.known_groups = known_groups
        self.active_groups = None
        self.label += f", host passes its {self.distinct} routed slots" if known_groups else ", slot capacity as the group bound"
        self.profile = "moe_decode_layer_config3.txt" if self.tokens == 64 and not hot_experts and baseline_shape and \
            expert_order == "block-major" else None
        self.profile_kernels = ("moe_gate_up_kernel",)

    def step(self, stages: int = 0):
        c = self.ctx
        slots, wts, host_slots = self.routings[self.turn % len(self.routings)]
        self.turn += 1
        c.prepare_decode_route_plan(self.plan, self.table, slots, self.gens, wts, self.k,
                                    host_route_slots=host_slots if self.known_groups else None)
        c.moe_decode_from_prepared_plan(self.plan, self.table, self.x, self.out, stages=stages,
                                        active_groups=self.active_groups)

    def dominant_step(self):
        from ferrule_amd import abi

        self.ctx.moe_decode_from_prepared_plan(self.plan, self.table, self.x, None, stages=abi.MOE_DECODE_SKIP_DOWN,
                                               active_groups=self.active_groups)

    def _host_expert(self, e):
        from ferrule_amd import synthetic

        return synthetic.host_expert(self.handles[e])

    def check(self):
        import numpy as np
        import torch

        from oracle import parity

        self.turn = 0      # the routing that self.ids / self.weights describe
        self.step()
        torch.cuda.synchronize()
        assert int(self.plan.route_error.item()) == 0
        sample = sorted({0, min(5, self.tokens - 1), self.tokens // 2, self.tokens - 1})
        host = {int(e): self._host_expert(int(e)) for e in np.unique(self.ids[sample])}
        want, bound, routes, route_bounds = parity.moe_layer_reference(
            host, self.x_host[sample], self.ids[sample], self.weights[sample], self.hidden, self.inter, threads=8)
        got = self.out.view(torch.int16).cpu().numpy().view(np.uint16)[sample]
        worst, decided, worst_decided = parity.compare_bf16_bounded(got, want, bound, max_decided_fraction=0.005)
        got_routes = self.plan.route_output.cpu().numpy()[:self.tokens * self.k].reshape(self.tokens, self.k, -1)[sample]
        assert (np.abs(got_routes.astype(np.float64) - routes) <= route_bounds + 1e-30).all()
        return {"max_bf16_ulp": worst, "decided_by_error_bound": decided, "worst_ulp_among_decided": worst_decided,
                "elements": int(want.size), "route_outputs_relative_rms_error": float(f"{parity.relative_rms(got_routes, routes):.3g}"),
                "sample": f"{len(sample)} tokens x {self.k} routes of the timed batch against the CPU executor, "
                          f"route outputs (f32) inside the derived forward-error bound, BF16 outputs by the 2-ulp rule"}

    def cpu_baseline(self, seconds: float):
        """CpuReferenceExpertExecutor as it runs: per route, dequantize three whole matrices to
        f32 and do three sequential matvecs, one thread.  A few routes are timed and the layer
        (512 routes) is extrapolated linearly."""
        import numpy as np

        from oracle import pyoracle as po

        routes = [(t, j) for t in range(self.tokens) for j in range(self.k)]
        done, t0 = 0, time.perf_counter()
        cache = {}
        spent = 0.0
        while done < 2 or spent < seconds:
            t, j = routes[done]
            e = int(self.ids[t, j])
            if e not in cache:
                cache[e] = self._host_expert(e)
            (gw, gs), (uw, us), (dw, ds) = cache[e]
            t1 = time.perf_counter()
            g = po.linear_fp4(gw, gs, self.inter, self.hidden, self.x_host[t], materialized=True)
            u = po.linear_fp4(uw, us, self.inter, self.hidden, self.x_host[t], materialized=True)
            h = (g / (1 + np.exp(-g)) * u * self.weights[t, j]).astype(np.float32)
            po.linear_fp4(dw, ds, self.hidden, self.inter, h, materialized=True)
            spent += time.perf_counter() - t1
            done += 1
        per_route = spent / done
        layer = per_route * len(routes)
        port = {"value": self.bytes_per_step / layer / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{done} of {len(routes)} routes timed ({per_route * 1e3:.0f} ms each, whole-matrix dequant "
                          f"per linear as in CpuReferenceExpertExecutor), layer time extrapolated linearly to "
                          f"{layer:.1f} s"}
        threads = min(16, os.cpu_count() or 1)
        done2, spent2 = 0, 0.0
        while done2 < 4 or spent2 < min(3.0, seconds):
            t, j = routes[done2 % done]
            (gw, gs), (uw, us), (dw, ds) = cache[int(self.ids[t, j])]
            t1 = time.perf_counter()
            po.expert_execute_fp4(gw, gs, uw, us, dw, ds, self.hidden, self.inter, self.x_host[t],
                                  float(self.weights[t, j]), threads=threads)
            spent2 += time.perf_counter() - t1
            done2 += 1
        layer2 = spent2 / done2 * len(routes)
        multi = {"value": self.bytes_per_step / layer2 / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                 "sample": f"{done2} routes, rows split over {threads} threads, dequant fused into the dot product, "
                           f"extrapolated to {layer2:.2f} s per layer"}
        return port, multi


class Fp8GemmWorkload:
    """configs[3]: packed prefill FP8 GEMM, BF16 rows [M,7168] ~N(0,1) quantised to FP8-K128 (its own
    launch, timed as part of the step), weight [N,7168] E4M3 with 128x128 fp32 block scales, BF16 out."""

    bound, unit, peak = "mfma", "TFLOP/s", 5000.0

    def __init__(self, ctx, m: int, n: int):
        import torch

        from ferrule_amd.provider import HipArtifactLinearHandle
        from ferrule_amd.provider import HipArtifactLinearShape as S

        self.ctx, self.m, self.n, self.k = ctx, m, n, 7168
        gen = torch.Generator(device="cuda").manual_seed(SEED_BASE + 4)
        w = torch.randn((n, self.k), generator=gen, device="cuda", dtype=torch.float32) * 0.02
        tiles = w.reshape(n // 128, 128, self.k // 128, 128)
        scales = (tiles.abs().amax(dim=(1, 3)) / 448.0).contiguous()
        packed = (tiles / scales[:, None, :, None]).clamp(-448, 448).reshape(n, self.k).to(torch.float8_e4m3fn)
        self.handle = HipArtifactLinearHandle(S.fp8_e4m3_with_f32_scale(n, self.k), packed.view(torch.uint8).reshape(-1),
                                              scales.reshape(-1))
        self.handles = [self.handle]
        self.decode = m <= 32      # the library streams the weights for these row counts: an HBM-bound step
        if self.decode:
            copies = -(-ROTATE_BYTES // (n * self.k))
            self.handles += [HipArtifactLinearHandle(self.handle.shape, self.handle.weight.clone(), self.handle.scale.clone())
                             for _ in range(copies - 1)]
        self.cursor = 0
        self.x = torch.randn((m, self.k), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16).float()
        self.out = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        self.xq, self.xs = ctx.pack_fp8_rows_from_f32(self.x)
        self.flops_per_step = 2 * m * n * self.k
        self.bytes_per_step = n * self.k + scales.numel() * 4 + m * self.k * 4 + m * self.k + m * (self.k // 128) + m * n * 2
        self.dominant = "fp8_block_gemm_kernel"
        self.profile = {(512, 7168): "fp8_gemm_m512_n7168_config4.txt",
                        (2048, 7168): "fp8_gemm_m2048_n7168_config4.txt",
                        (4096, 18432): "fp8_gemm_m4096_n18432_config4.txt"}.get((m, n))
        self.profile_kernels = ("fp8_block_gemm_kernel",)
        self.dominant_flops = self.flops_per_step
        self.label = f"configs[3] FP8 GEMM M={m} N={n} K=7168, fp32 128x128 weight scales, FP8-K128 activations, BF16 out"
        self.rotated = len(self.handles)
        if self.decode:
            self.bound, self.unit, self.peak = "hbm", "GB/s", HBM_PEAK_GBS
            self.dtype = "e4m3 activations x e4m3 weights, f32 accumulate"
            self.dominant = "fp8_rows_kernel"
            self.profile = f"fp8_rows_m{m}_n{n}.txt"
            self.profile_kernels = ("fp8_rows_kernel",)
            self.dominant_bytes = n * self.k + scales.numel() * 4 + m * self.k + m * (self.k // 128) + m * n * 2
            self.label = (f"FP8 projection of a decode batch (decode-row schedule): M={m} N={n} K=7168, fp32 128x128 "
                          f"weight scales, FP8-K128 activations, BF16 out")

    def step(self):
        import torch

        from ferrule_amd import abi

        a = abi.QuantizeArgs(kind=abi.QUANTIZE_FP8_PACKED, value_offset=0, value_len=self.m * self.k, row_width=self.k,
                             block_size=128, rope_dim=0, reserved=0, values=self.x.data_ptr(),
                             packed=self.xq.data_ptr(), scales=self.xs.data_ptr())
        self.ctx._core("FP8 pack", self.ctx.lib.ferrule_hip_core_quantize_launch, a)
        self.ctx.fp8_block_gemm(self.xq, self.xs, self.handles[self.cursor % len(self.handles)], self.out)
        self.cursor += 1

    def dominant_step(self):
        self.ctx.fp8_block_gemm(self.xq, self.xs, self.handles[self.cursor % len(self.handles)], self.out)
        self.cursor += 1

    def _sample(self, rows):
        import numpy as np

        from oracle import pyoracle as po

        w = self.handle.weight.cpu().numpy().reshape(self.n, self.k)
        s = self.handle.scale.cpu().numpy().reshape(self.n // 128, self.k // 128)
        x = self.x[rows].cpu().numpy()
        return w, s, po.simulate_fp8_act_quant(x, self.k, 128)

    def check(self):
        import numpy as np
        import torch

        from oracle import parity
        from oracle import pyoracle as po

        self.step()
        torch.cuda.synchronize()
        rows = sorted({(j * (self.m - 1)) // 7 for j in range(8)})    # eight rows spread over the batch
        w, s, xq = self._sample(rows)
        want = po.linear_fp8(w, s, self.n, self.k, xq, threads=8)
        absprod = np.stack([po.abs_linear_fp8(w, s, self.n, self.k, np.abs(r.astype(np.float64)), threads=8) for r in xq])
        got = self.out[rows].view(torch.int16).cpu().numpy().view(np.uint16)
        worst, decided = parity.compare_bf16(got, want, absprod, self.k)
        return {"max_bf16_ulp": worst, "decided_by_error_bound": decided, "elements": int(want.size),
                "sample": f"{len(rows)} rows of the timed batch against the CPU matvec"}

    def cpu_baseline(self, seconds: float):
        from oracle import pyoracle as po

        w, s, xq = self._sample([0])
        reps, t0 = 0, time.perf_counter()
        while reps < 1 or time.perf_counter() - t0 < seconds:
            po.linear_fp8(w, s, self.n, self.k, xq, materialized=True)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        per_row = (self.n * self.k + self.n * self.k // 4096) / 1e9 if self.decode else 2 * self.n * self.k / 1e12
        port = {"value": per_row / dt, "unit": self.unit, "cores": 1, "kind": "port",
                "sample": f"{reps} rows of the {self.m} (one LinearWeight::reference_matvec each, whole-matrix dequant "
                          f"per call, {dt * 1e3:.0f} ms per row)"}
        threads = min(16, os.cpu_count() or 1)
        reps, t0 = 0, time.perf_counter()
        while reps < 2 or time.perf_counter() - t0 < min(3.0, seconds):
            po.linear_fp8(w, s, self.n, self.k, xq, threads=threads)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        multi = {"value": per_row / dt, "unit": self.unit, "cores": threads, "kind": "port",
                 "sample": f"{reps} rows, output rows split over {threads} threads, dequant fused"}
        return port, multi


class SharedFfnWorkload:
    """The dense FP8 shared FFN behind ferrule_hip_shared_ffn_launch for a decode batch at DeepSeek-V4's
    shared-expert shape (4096 -> 2048 -> 4096, E4M3 weights with E8M0 128x128 block scales, FP8-K128
    activations in, f32 out): up to 32 rows take the decode-row schedule (gate/up stream, quantiser, down
    stream).  Weight sets rotate; the check is bit-equality with the tile schedule plus the CPU chain."""

    input_size, inter, output_size = 4096, 2048, 4096
    dtype = "e4m3 activations x e4m3 weights, f32 accumulate"

    def __init__(self, ctx, rows: int, tile_schedule: bool = False):
        import torch

        from ferrule_amd import synthetic
        from ferrule_amd.provider import HipArtifactLinearHandle

        self.ctx, self.rows, self.tile_schedule = ctx, rows, tile_schedule
        gen = torch.Generator(device="cuda").manual_seed(SEED_BASE + 13)
        shapes = ((self.inter, self.input_size), (self.inter, self.input_size), (self.output_size, self.inter))
        first = [synthetic.device_fp8_linear(ctx, gen, n, k, "e8m0") for n, k in shapes]
        weight_bytes = sum(h.weight.numel() + h.scale.numel() for h in first)
        copies = -(-ROTATE_BYTES // weight_bytes)
        self.sets = [first] + [[HipArtifactLinearHandle(h.shape, h.weight.clone(), h.scale.clone()) for h in first]
                               for _ in range(copies - 1)]
        self.handles = self.sets
        self.x = torch.randn((rows, self.input_size), generator=gen, device="cuda").to(torch.bfloat16).float()
        self.xq, self.xs = ctx.pack_fp8_rows_from_f32(self.x)
        self.out = torch.zeros((rows, self.output_size), dtype=torch.float32, device="cuda")
        per_row = self.input_size * 33 // 32 + self.inter * (4 + 1 + 1) + self.output_size * 4
        self.bytes_per_step = weight_bytes + rows * per_row
        self.flops_per_step = 2 * rows * 3 * self.inter * self.input_size
        self.dominant = "fp8_rows_kernel (gate/up) + quantize_vec_kernel + fp8_rows_kernel (down)"
        self.profile = f"shared_ffn_rows_m{rows}.txt"
        self.profile_kernels = ("fp8_rows_kernel+", "quantize_vec_kernel")
        self.label = (f"shared FFN (FP8 x FP8), decode batch {rows}: {self.input_size} -> {self.inter} -> "
                      f"{self.output_size}, E8M0 block scales, {'tile' if tile_schedule else 'decode-row'} schedule")
        self.cursor = 0
        self.last = None

    def step(self):
        g, u, d = self.sets[self.cursor % len(self.sets)]
        self.last = self.ctx.shared_ffn(self.xq, self.xs, g, u, d, self.out, tile_schedule=self.tile_schedule)
        self.cursor += 1

    def check(self):
        import numpy as np
        import torch

        from oracle import parity
        from oracle import pyoracle as po

        self.cursor = 0
        self.step()
        torch.cuda.synchronize()
        h_gpu, hq, hs = (t.cpu().numpy() for t in self.last)
        got = self.out.cpu().numpy()
        # the other schedule gives the same bits
        g, u, d = self.sets[0]
        other = torch.zeros_like(self.out)
        oh, oq, os_ = self.ctx.shared_ffn(self.xq, self.xs, g, u, d, other, tile_schedule=not self.tile_schedule)
        torch.cuda.synchronize()
        same = bool(torch.equal(other.view(torch.int32), self.out.view(torch.int32)) and torch.equal(oq, self.last[1]) and
                    torch.equal(os_, self.last[2]) and torch.equal(oh.view(torch.int32), self.last[0].view(torch.int32)))
        assert same, "the decode-row and the tile schedule of the shared FFN differ"
        # row 0 against the CPU chain: the quantiser exactly on the device's h, the down projection of those bytes
        (gw, gs), (uw, us), (dw, ds) = [(h.weight.cpu().numpy().reshape(h.shape.out_features, -1),
                                         h.scale.cpu().numpy().reshape(h.shape.out_features // 128, -1)) for h in self.sets[0]]
        xdq = po.simulate_fp8_act_quant(self.x[:1].cpu().numpy(), self.input_size, 128)
        gg = po.linear_fp8(gw, gs, self.inter, self.input_size, xdq, threads=8)[0]
        uu = po.linear_fp8(uw, us, self.inter, self.input_size, xdq, threads=8)[0]
        h_ref = (np.array([po.silu(float(v)) for v in gg], np.float32) * uu).astype(np.float32)
        eps = self.input_size * 2.0 ** -24 + parity.MFMA_BLOCK_EPS
        ax = np.abs(xdq[0].astype(np.float64))
        dg = eps * po.abs_linear_fp8(gw, gs, self.inter, self.input_size, ax, threads=8)
        du = eps * po.abs_linear_fp8(uw, us, self.inter, self.input_size, ax, threads=8)
        bound = 1.1 * np.abs(uu) * dg + np.abs(gg) * du + dg * du + np.abs(h_ref) * 2.0 ** -21
        assert (np.abs(h_gpu[0] - h_ref) <= bound + 1e-30).all(), "hidden values outside the forward-error bound"
        want_q, want_s = po.pack_fp8_act(h_gpu[:1], self.inter, 128)
        assert np.array_equal(hq[:1].ravel(), want_q.ravel()) and np.array_equal(hs[:1].ravel(), want_s.ravel())
        hdq = po.simulate_fp8_act_quant(h_gpu[:1], self.inter, 128)
        y = po.linear_fp8(dw, ds, self.output_size, self.inter, hdq, threads=8)[0]
        absprod = po.abs_linear_fp8(dw, ds, self.output_size, self.inter, np.abs(hdq[0].astype(np.float64)), threads=8)
        err = np.abs(got[0].astype(np.float64) - y.astype(np.float64))
        limit = (self.inter * 2.0 ** -24 + parity.MFMA_BLOCK_EPS) * absprod + np.abs(y) * 2.0 ** -23
        assert (err <= limit).all(), "down projection outside the forward-error bound"
        dist = np.abs(parity.ordered(po.bf16_bits_array(got[0])) - parity.ordered(po.bf16_bits_array(y)))
        return {"max_bf16_ulp": int(dist.max()), "same_bits_as_other_schedule": same, "elements": int(y.size),
                "sample": "row 0 of the timed batch stage by stage against the CPU chain; every buffer against the "
                          "other schedule bit for bit"}

    def cpu_baseline(self, seconds: float):
        from oracle import pyoracle as po

        (gw, gs), (uw, us), (dw, ds) = [(h.weight.cpu().numpy().reshape(h.shape.out_features, -1),
                                         h.scale.cpu().numpy().reshape(h.shape.out_features // 128, -1)) for h in self.sets[0]]
        x = self.x[0].cpu().numpy()

        def chain(**kw):
            xq = po.simulate_fp8_act_quant(x, self.input_size, 128)
            g = po.linear_fp8(gw, gs, self.inter, self.input_size, xq, **kw)[0]
            u = po.linear_fp8(uw, us, self.inter, self.input_size, xq, **kw)[0]
            h = po.simulate_fp8_act_quant((g / (1 + __import__("numpy").exp(-g)) * u).astype("float32"), self.inter, 128)
            po.linear_fp8(dw, ds, self.output_size, self.inter, h, **kw)

        one_row = self.bytes_per_step - (self.rows - 1) * (self.bytes_per_step - sum(
            h.weight.numel() + h.scale.numel() for h in self.sets[0])) // self.rows
        results = []
        for kw, budget, what in (({"materialized": True}, seconds, "whole-matrix dequant per linear as in LinearWeight::reference_matvec"),
                                 ({"threads": min(16, os.cpu_count() or 1)}, min(3.0, seconds), "rows split over the threads, dequant fused")):
            chain(**kw)
            reps, t0 = 0, time.perf_counter()
            while reps < 2 or time.perf_counter() - t0 < budget:
                chain(**kw)
                reps += 1
            dt = (time.perf_counter() - t0) / reps
            results.append({"value": one_row / dt / 1e9, "unit": "GB/s", "cores": kw.get("threads", 1), "kind": "port",
                            "sample": f"{reps} single-row FFN calls ({dt * 1e3:.1f} ms each), {what}"})
        return results[0], results[1]


class MoePrefillWorkload:
    """configs[4]: MoE prefill layer, T tokens (8192), 256 MXFP4 experts, top-8 with Zipf(1.1) popularity.
    A step = FP8-K128 quantisation of the BF16 rows, invocation flag reset, route plan, grouped gate/up + SwiGLU +
    requantisation, grouped down, rank-ordered fp32 combine with the BF16 writeback."""

    bound, unit, peak = "mfma", "TFLOP/s", 5000.0
    k, experts, hidden, inter = 8, 256, 7168, 2048

    def __init__(self, ctx, tokens: int, experts=None, expert_order: str = "block-major"):
        import numpy as np
        import torch

        from ferrule_amd import synthetic

        self.ctx, self.tokens = ctx, tokens
        if experts is None:
            experts = synthetic.build_device_experts(ctx, self.experts, self.hidden, self.inter, SEED_BASE + 5)
        self.table, self.handles = experts
        if expert_order == "block-major":
            # the one prepared copy an expert gets when it is installed in a slot; the decode layer reads the same
            self.table = synthetic.block_major_table(ctx, self.handles)
        rng = synthetic.rng_for(5)
        self.ids, self.weights = synthetic.zipf_routing(rng, tokens, self.k, self.experts)
        gen = torch.Generator(device="cuda").manual_seed(SEED_BASE + 5)
        self.x = torch.randn((tokens, self.hidden), generator=gen, device="cuda").to(torch.bfloat16).float()
        self.xq, self.xs = ctx.pack_fp8_rows_from_f32(self.x)
        self.slots = torch.from_numpy(self.ids.ravel().astype(np.int32)).cuda()
        self.gens = torch.ones(tokens * self.k, dtype=torch.int32, device="cuda")
        self.wts = torch.from_numpy(self.weights.ravel()).cuda()
        self.out = torch.zeros((tokens, self.hidden), dtype=torch.float32, device="cuda")
        self.plan = ctx.expert_group_route_plan(self.experts, tokens * self.k, tokens, self.hidden, self.inter,
                                                self.hidden)
        self._plan()
        torch.cuda.synchronize()
        self.meta = self.plan.host_metadata()     # the 16-byte readback, once (routing is fixed)
        rows = tokens * self.k
        self.flops_per_step = rows * (2 * self.hidden * 2 * self.inter + 2 * self.inter * self.hidden)
        per_matrix = lambda n, kk: n * kk // 2 + n * kk // 32
        distinct = int(len(np.unique(self.ids)))
        self.bytes_per_step = distinct * 3 * per_matrix(self.inter, self.hidden) + tokens * self.hidden * 6
        # the two grouped GEMM kernels of one launch (gate/up + down), timed together
        self.dominant = "grouped_gate_up_chained_kernel + grouped_down_chained_kernel"
        self.dominant_flops = self.flops_per_step
        self.profile = "moe_prefill_layer_config5.txt" if tokens == 8192 else None
        self.profile_kernels = ("grouped_gate_up_chained_kernel", "grouped_down_chained_kernel")
        self.label = (f"configs[4] MoE prefill layer: {tokens} tokens, hidden {self.hidden}, {self.experts} MXFP4 "
                      f"experts, top-{self.k}, Zipf(1.1) popularity (largest group {self.meta['max_group_rows']} rows), "
                      f"{expert_order} expert weights")
        self.rotated = 1

    def _plan(self):
        c = self.ctx
        # flags only: every live row of route_output is rewritten in full by the down GEMM and the
        # checked reducer skips tokens with an unwritten route
        c.begin_expert_group_route_invocation(self.plan, self.tokens * self.k, clear_output=False)
        c.prepare_expert_group_route_plan(self.plan, self.table, self.slots, self.gens, self.wts, self.k)

    def step(self):
        from ferrule_amd import abi

        c = self.ctx
        a = abi.QuantizeArgs(kind=abi.QUANTIZE_FP8_PACKED, value_offset=0, value_len=self.tokens * self.hidden,
                             row_width=self.hidden, block_size=128, rope_dim=0, reserved=0, values=self.x.data_ptr(),
                             packed=self.xq.data_ptr(), scales=self.xs.data_ptr())
        # the plan's small launches first: the activation quantiser is a bandwidth-bound pass, and right behind
        # the previous step's combine it would share the HBM with the write-back of that step's results
        self._plan()
        c._core("FP8 pack", c.lib.ferrule_hip_core_quantize_launch, a)
        c.grouped_fp4_moe_from_prepared_plan(self.plan, self.table, self.xq, self.xs, meta=self.meta)
        self.out.zero_()
        c.reduce_moe_route_outputs_ranked(self.plan.route_output, self.tokens, self.k, self.hidden, self.out,
                                          self.plan.route_written, self.plan.route_error)

    def dominant_step(self):
        self.ctx.grouped_fp4_moe_from_prepared_plan(self.plan, self.table, self.xq, self.xs, meta=self.meta)

    def _host_expert(self, e):
        from ferrule_amd import synthetic

        return synthetic.host_expert(self.handles[e])

    def check(self):
        """One token x 8 routes of the timed batch against the CPU executor with FP8-K128 activation
        quantisation.  The device's hidden values differ from the CPU's in the last fp32 bits, so a value
        on a rounding boundary of the quantiser may take the neighbouring code: the comparison is against
        the CPU chain plus the exactly computed effect of the device's own codes (read from the workspace),
        inside the fp32 / MFMA summation bound of the down projection."""
        import numpy as np
        import torch

        from oracle import parity
        from oracle import pyoracle as po

        self.step()
        torch.cuda.synchronize()
        assert int(self.plan.route_error.item()) == 0
        hq, hs = self.ctx.grouped_workspace_views(self.plan, self.meta)
        rows = self.tokens * self.k
        row_of_route = torch.empty(rows, dtype=torch.long, device="cuda")
        row_of_route[self.plan.route_indices[:rows].long()] = torch.arange(rows, device="cuda")
        dec = np.array([po.decode_fp8_e4m3fn_byte(i) for i in range(256)], np.float64)
        within, flips, elements = 0, 0, 0
        tokens = sorted({11, self.tokens - 5}) if self.tokens > 16 else [0]
        for t in tokens:
            x = self.x[t].cpu().numpy()
            ys, delta, absdown = [], np.zeros(self.hidden, np.float64), np.zeros(self.hidden, np.float64)
            for j in range(self.k):
                (gw, gs), (uw, us), (dw, ds) = self._host_expert(int(self.ids[t, j]))
                y, h = po.expert_execute_fp4(gw, gs, uw, us, dw, ds, self.hidden, self.inter, x, float(self.weights[t, j]),
                                             act_quant_block=128, threads=8, return_hidden=True)
                ys.append(y)
                row = int(row_of_route[t * self.k + j].item())
                h_gpu = dec[hq[row].cpu().numpy()] * np.repeat(2.0 ** (hs[row].cpu().numpy().astype(np.float64) - 127), 128)
                delta += po.dequantize_fp4(dw, ds, self.hidden, self.inter).astype(np.float64) @ (h_gpu - h.astype(np.float64))
                absdown += po.abs_linear_fp4(dw, ds, self.hidden, self.inter, np.abs(h_gpu), threads=8)
            want = po.accumulate_routes(np.stack(ys))
            got = self.out[t].cpu().numpy()
            err = np.abs(got.astype(np.float64) - (want.astype(np.float64) + delta))
            bound = 2.0 * (self.inter * 2.0 ** -24 + parity.MFMA_BLOCK_EPS) * absdown + \
                (np.abs(got) + np.abs(want)).astype(np.float64) * 2.0 ** -8
            assert (err <= bound).all(), "prefill layer differs from the CPU chain beyond quantiser code flips"
            dist = np.abs(parity.ordered(po.bf16_bits_array(got)) - parity.ordered(po.bf16_bits_array(want)))
            within += int((dist <= 2).sum())
            flips += int((dist > 2).sum())
            elements += int(want.size)
        return {"within_2_bf16_ulp_of_cpu_chain": float(f"{within / elements:.4f}"),
                "explained_by_quantiser_code_flips": flips, "elements": elements,
                "sample": f"{len(tokens)} tokens x 8 routes of the timed batch against the CPU executor with FP8-K128 act-quant"}

    def cpu_baseline(self, seconds: float):
        from oracle import pyoracle as po

        flops_route = 2 * self.hidden * 2 * self.inter + 2 * self.inter * self.hidden
        routes = [(t, j) for t in range(0, self.tokens, max(1, self.tokens // 64)) for j in range(self.k)]
        x = self.x.cpu().numpy()
        done, spent, cache = 0, 0.0, {}
        while done < 2 or spent < seconds:
            t, j = routes[done % len(routes)]
            e = int(self.ids[t, j])
            if e not in cache:
                cache[e] = self._host_expert(e)
            (gw, gs), (uw, us), (dw, ds) = cache[e]
            t1 = time.perf_counter()
            xq = po.simulate_fp8_act_quant(x[t], self.hidden, 128)
            g = po.linear_fp4(gw, gs, self.inter, self.hidden, xq, materialized=True)[0]
            u = po.linear_fp4(uw, us, self.inter, self.hidden, xq, materialized=True)[0]
            h = po.simulate_fp8_act_quant((g / (1 + __import__("numpy").exp(-g)) * u * self.weights[t, j]).astype("float32"),
                                          self.inter, 128)
            po.linear_fp4(dw, ds, self.hidden, self.inter, h, materialized=True)
            spent += time.perf_counter() - t1
            done += 1
        per = spent / done
        port = {"value": flops_route / per / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
                "sample": f"{done} of {self.tokens * self.k} routes, stratified over tokens ({per * 1e3:.0f} ms each, "
                          f"whole-matrix dequant per linear as in CpuReferenceExpertExecutor)"}
        threads = min(16, os.cpu_count() or 1)
        done2, spent2 = 0, 0.0
        while done2 < 4 or spent2 < min(3.0, seconds):
            t, j = routes[done2 % min(done, len(routes))]
            (gw, gs), (uw, us), (dw, ds) = cache[int(self.ids[t, j])]
            t1 = time.perf_counter()
            po.expert_execute_fp4(gw, gs, uw, us, dw, ds, self.hidden, self.inter, x[t], float(self.weights[t, j]),
                                  act_quant_block=128, threads=threads)
            spent2 += time.perf_counter() - t1
            done2 += 1
        multi = {"value": flops_route / (spent2 / done2) / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                 "sample": f"{done2} routes, rows split over {threads} threads, dequant fused"}
        return port, multi


# ----------------------------------------------------------------------------- main

class RouterWorkload:
    """The step before the route plan: sqrt-softplus score top-8 of 256 experts with bias for a
    batch of tokens (8192 = the prefill layer's batch, 64 = the decode layer's), f32 logits in,
    int32 ids and f32 weights out."""

    experts, k, scale = 256, 8, 2.5

    def __init__(self, ctx, tokens: int):
        import torch

        self.ctx, self.tokens = ctx, tokens
        gen = torch.Generator(device="cuda").manual_seed(SEED_BASE + 6)
        one = tokens * self.experts * 4
        copies = max(1, min(64, -(-ROTATE_BYTES // one)))
        self.handles = [torch.randn((tokens, self.experts), generator=gen, device="cuda", dtype=torch.float32) * 2.5
                        for _ in range(copies)]
        self.bias = torch.randn(self.experts, generator=gen, device="cuda", dtype=torch.float32) * 0.25
        self.idx = torch.empty((tokens, self.k), dtype=torch.int32, device="cuda")
        self.w = torch.empty((tokens, self.k), dtype=torch.float32, device="cuda")
        self.bytes_per_step = one + self.experts * 4 + tokens * self.k * 8
        self.flops_per_step = 0
        self.dtype = "f32 scores, 64-bit integer selection keys"
        self.dominant = "router_select_kernel"
        self.profile = "router_topk_8192_tokens.txt" if tokens == 8192 else None
        self.profile_kernels = ("router_select_kernel",)
        self.label = (f"router: sqrt-softplus score top-{self.k} of {self.experts} experts with bias, {tokens} tokens "
                      f"(the producer of the route plan's input)")
        self.cursor = 0

    def step(self):
        self.ctx.dsv4_router_topk_sqrt_softplus_rows_from_device_into(
            self.handles[self.cursor % len(self.handles)], self.bias, self.tokens, self.experts, self.k, self.scale,
            self.idx, self.w)
        self.cursor += 1

    def check(self):
        import torch

        from oracle.parity import check_score_router as _check_score_router

        self.cursor = 0
        self.step()
        torch.cuda.synchronize()
        near = _check_score_router(self.handles[0].cpu().numpy(), self.bias.cpu().numpy(), self.k, self.scale,
                                   self.idx.cpu().numpy(), self.w.cpu().numpy())
        return {"rows": self.tokens, "rows_differing_only_inside_the_score_tolerance": near,
                "ids": "equal to the CPU checker's except at selection values closer than 8 ulp",
                "weights": "within 16 ulp"}

    def cpu_baseline(self, seconds: float):
        from oracle import pyoracle as po

        logits, bias = self.handles[0].cpu().numpy(), self.bias.cpu().numpy()
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or time.perf_counter() - t0 < min(seconds, 5.0):
            po.router_kernel_rows(1, logits, self.k, self.scale, bias=bias)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        port = {"value": self.bytes_per_step / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{reps} full batches of {self.tokens} rows through the sequential restatement of the "
                          f"reference kernel ({dt * 1e3:.2f} ms each)"}
        return port, dict(port)


class RoutingChainWorkload(RouterWorkload):
    """Everything between the router logits and the grouped GEMMs, on the device: score router, slot
    resolution against the stable expert table (all 256 experts resident, slots permuted), invocation flag
    reset and the four-kind route plan (or, up to 2048 routes, the fused decode plan)."""

    def __init__(self, ctx, tokens: int):
        import torch

        from ferrule_amd.provider import HipExpertSlotPointers

        super().__init__(ctx, tokens)
        self.table = ctx.expert_slot_table(self.experts, self.experts)
        order = torch.randperm(self.experts, generator=torch.Generator().manual_seed(7)).tolist()
        for e in order:   # addresses are never dereferenced by these kernels
            ctx.install_expert_slot(self.table, e, HipExpertSlotPointers(*[(e * 6 + m + 1) * 256 for m in range(6)]))
        routes = tokens * self.k
        self.workspace = ctx.expert_route_resolve_workspace(routes, 64)
        self.plan = ctx.expert_group_route_plan(self.experts, routes, tokens, 7168, 2048, 7168)
        self.fused = routes <= 2048
        # logits + bias + ids/weights out; ids in, slots/generations/markers/control out; plan: slots,
        # generations, weights in, (token, route, weight) permutation out
        self.bytes_per_step += routes * (4 + 16) + routes * (12 + 12)
        self.profile = None
        self.label = (f"routing chain: router (top-{self.k} of {self.experts}) -> slot resolve -> route plan, "
                      f"{tokens} tokens, {routes} routes, {'fused decode plan' if self.fused else 'four-kind plan'}")

    def step(self):
        c, routes = self.ctx, self.tokens * self.k
        super().step()
        c.resolve_expert_routes(self.table, self.idx.view(-1), routes, self.workspace)
        ws = self.workspace
        if self.fused:
            c.prepare_decode_route_plan(self.plan, self.table, ws.route_slots, ws.route_generations, self.w.view(-1),
                                        self.k)
        else:
            c.begin_expert_group_route_invocation(self.plan, routes, clear_output=False)
            c.prepare_expert_group_route_plan(self.plan, self.table, ws.route_slots, ws.route_generations,
                                              self.w.view(-1), self.k)

    def dominant_step(self):
        RouterWorkload.step(self)

    def check(self):
        import numpy as np
        import torch

        from oracle import pyoracle as po

        parity = super().check()
        self.cursor = 0
        self.step()
        torch.cuda.synchronize()
        ids = self.idx.cpu().numpy().ravel()
        state = po.ExpertTableState(self.experts, self.experts)
        for e in range(self.experts):
            b = self.table.host.binding(e)
            state.publish(1, e, b.slot, b.generation, self.table.host.pointers_at(b.slot).as_tuple())
        slots, gens, markers, control = state.resolve(ids, 64, ids.size)
        ok = np.array_equal(self.workspace.route_slots.cpu().numpy(), slots) and \
            np.array_equal(self.workspace.route_generations.cpu().numpy(), gens) and \
            int(self.workspace.miss_control[0].item()) == 0
        meta = self.plan.host_metadata()
        counts = np.bincount(slots, minlength=self.experts)
        indptr = self.plan.expert_route_indptr.cpu().numpy()[:meta["active_group_count"] + 1]
        active = self.plan.active_expert_slots.cpu().numpy()[:meta["active_group_count"]]
        ok = ok and np.array_equal(np.diff(indptr), counts[active]) and int(indptr[-1]) == ids.size
        assert ok, "routing chain disagrees with the CPU checker"
        parity["resolve_and_plan"] = "slots, generations and per-slot route counts equal the CPU checker's"
        return parity


class ExpertUploadWorkload:
    """Routed experts of configs[2]'s shape from a safetensors shard to prepared device slots: a step
    materialises eight experts (23.4 MB each: file -> one of two pinned staging frames -> device arena,
    then the block-major reorder of the three matrices on the device, host copy and transfer overlapped).
    `value` is the end-to-end rate of a step; the roofline entry is the reorder kernel alone (reads and
    writes every byte once)."""

    hidden, inter, experts = 7168, 2048, 8

    def __init__(self, ctx, directory: str):
        import numpy as np
        import torch
        from safetensors.torch import save_file

        from ferrule_amd import expert_artifacts as EA

        self.ctx, self.EA = ctx, EA
        gen = torch.Generator().manual_seed(SEED_BASE + 7)
        tensors = {}
        for e in range(self.experts):
            for name, (n, k) in (("w1", (self.inter, self.hidden)), ("w3", (self.inter, self.hidden)),
                                 ("w2", (self.hidden, self.inter))):
                tensors[f"layers.0.ffn.experts.{e}.{name}.weight"] = \
                    torch.randint(-128, 128, (n, k // 2), generator=gen, dtype=torch.int8)
                tensors[f"layers.0.ffn.experts.{e}.{name}.scale"] = \
                    torch.randint(118, 124, (n, k // 32), generator=gen, dtype=torch.uint8).view(torch.float8_e8m0fnu)
        os.makedirs(directory, exist_ok=True)
        save_file(tensors, os.path.join(directory, "experts.safetensors"))
        self.host = {name: t.view(torch.uint8).numpy().copy() for name, t in tensors.items()}
        del tensors
        self.index = EA.RoutedExpertArtifactIndex.open(directory)
        self.shape = EA.HipRoutedExpertShape(self.hidden, self.inter, self.hidden)
        self.arena = EA.HipRoutedExpertArena(ctx, self.shape, self.experts, block_major=True)
        self.bundles = [self.index.bundle(0, e) for e in range(self.experts)]
        for _ in range(self.experts):
            self.arena.allocate_frame()
        self.expert_bytes = self.bundles[0].payload_bytes()
        self.bytes_per_step = self.experts * self.expert_bytes
        self.flops_per_step = 0
        self.dominant = "mxfp4_block_major_kernel"
        self.dominant_bytes = 2 * self.expert_bytes
        self.dtype = "u8 (bytes moved unchanged, then permuted)"
        self.handles = self.bundles
        self.cursor = 0
        self.label = (f"expert upload: {self.experts} MXFP4 experts per step (gate+up [4096,7168], down [7168,2048], "
                      f"{self.expert_bytes} bytes each) from a safetensors shard to prepared device frames")
        self.capturable = False

    def step(self):
        done = self.EA.materialize_routed_experts(self.ctx, self.arena, range(self.experts), self.bundles)
        self.raw, self.prepared = done[0]
        self.cursor += 1

    def dominant_step(self):
        for i in range(3):
            views = self.arena.views(self.arena.prepared, 0)
            self.ctx.prepare_mxfp4_block_major_into(self.raw0[i], views[2 * i], views[2 * i + 1])

    def check(self):
        import numpy as np

        self.cursor = 0
        self.step()
        self.raw0 = self.raw
        ok = True
        for handle, name in zip(self.raw, ("w1", "w3", "w2")):
            ok &= np.array_equal(handle.weight.cpu().numpy(), self.host[f"layers.0.ffn.experts.0.{name}.weight"].ravel())
            ok &= np.array_equal(handle.scale.cpu().numpy(), self.host[f"layers.0.ffn.experts.0.{name}.scale"].ravel())
        assert ok, "device bytes differ from the shard's"
        return {"device_bytes_equal_file_bytes": True, "tensors": 6}

    def cpu_baseline(self, seconds: float):
        import numpy as np

        # the reference's CPU staging of the same payload: read the six ranges into host memory
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or time.perf_counter() - t0 < min(seconds, 3.0):
            for linear in self.bundles[reps % self.experts].linears():
                for s in (linear.weight, linear.scale):
                    with open(s.path, "rb") as f:
                        f.seek(s.offset)
                        f.read(s.bytes)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        port = {"value": self.expert_bytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{reps} experts read from the shard into host memory ({dt * 1e3:.2f} ms each, page cache warm)"}
        return port, dict(port)


class HcProducerWorkload:
    """The producer of a layer's FP8 activations: HC state f32 [tokens, 4, 4096] -> mix/split, hidden,
    normalized (f32) and packed E4M3 + E8M0 scales, one launch.  Algorithmic bytes per token: the state
    (16 H) once, hidden and normalized (4 H each), packed (H), scales and split outputs; plus the
    function matrix (24 x 4 H floats) once per launch."""

    hc, hidden, iters = 4, 4096, 4

    def __init__(self, ctx, tokens: int):
        import torch

        self.ctx, self.tokens = ctx, tokens
        gen = torch.Generator(device="cuda").manual_seed(SEED_BASE + 8)
        mix, H = 24, self.hidden
        per_copy = tokens * self.hc * H * 4
        copies = max(1, min(8, -(-ROTATE_BYTES // per_copy)))
        self.handles = [torch.randn((tokens, self.hc, H), generator=gen, device="cuda", dtype=torch.float32)
                        for _ in range(copies)]
        self.function = torch.randn((mix, self.hc * H), generator=gen, device="cuda", dtype=torch.float32) / 128.0
        self.scale = torch.tensor([0.8, 1.3, 0.6], device="cuda")
        self.base = torch.randn(mix, generator=gen, device="cuda") * 0.3
        self.weight = 1.0 + 0.1 * torch.randn(H, generator=gen, device="cuda")
        self.out = None
        self.bytes_per_step = tokens * (self.hc * H * 4 + 2 * H * 4 + H + H // 128 + (mix + 24) * 4) + mix * self.hc * H * 4
        self.flops_per_step = 2 * tokens * mix * self.hc * H
        self.dominant = "hc_mix_kernel + hc_producer_kernel"
        self.dtype = "f32 (FP32 MFMA dot products, separately rounded elsewhere), E4M3 + E8M0 out"
        self.profile = "hc_producer_8192_tokens.txt" if tokens == 8192 else None
        self.profile_kernels = ("hc_mix_kernel", "hc_producer_kernel")
        self.label = f"HC producer: {tokens} tokens, hc 4, hidden {H}, {self.iters} Sinkhorn iterations"
        self.cursor = 0

    def step(self):
        self.out = self.ctx.hc_pre_rmsnorm_fp8_into(self.handles[self.cursor % len(self.handles)], self.function,
                                                    self.scale, self.base, self.weight, self.iters, 1e-6, 1e-6, 1e-6,
                                                    out=self.out)
        self.cursor += 1

    def _sample(self):
        return sorted({0, min(1, self.tokens - 1), self.tokens // 2, self.tokens - 1})   # valid rows only

    def check(self):
        import numpy as np
        import torch

        from oracle import pyoracle as po

        self.cursor = 0
        self.step()
        torch.cuda.synchronize()
        rows = self._sample()
        want = po.hc_producer(self.handles[0][rows].cpu().numpy(), self.function.cpu().numpy(), self.scale.cpu().numpy(),
                              self.base.cpu().numpy(), self.weight.cpu().numpy(), self.iters, 1e-6, 1e-6, 1e-6)
        got = {k: v[rows].cpu().numpy() for k, v in self.out.items()}
        worst = 0.0
        for name, key in (("mix", "raw_dots"), ("pre", "pre"), ("post", "post"), ("comb", "comb"), ("hidden", "hidden"),
                          ("normalized", "normalized")):
            worst = max(worst, float(np.abs(got[name] - want[key]).max() / max(1.0, np.abs(want[key]).max())))
        assert worst <= 2e-5, f"HC producer differs from the CPU checker by {worst}"
        packed, scales = po.pack_fp8_act(got["normalized"], self.hidden, 128)
        assert np.array_equal(got["packed"], packed.reshape(len(rows), -1)) and \
            np.array_equal(got["scales"], scales.reshape(len(rows), -1))
        return {"rows_checked": len(rows), "max_relative_difference_f32": worst,
                "fp8_bytes": "equal to the CPU quantiser on the device's normalized values"}

    def cpu_baseline(self, seconds: float):
        from oracle import pyoracle as po

        state = self.handles[0][: min(self.tokens, 64)].cpu().numpy()
        args = (self.function.cpu().numpy(), self.scale.cpu().numpy(), self.base.cpu().numpy(), self.weight.cpu().numpy(),
                self.iters, 1e-6, 1e-6, 1e-6)
        reps, t0 = 0, time.perf_counter()
        while reps < 2 or time.perf_counter() - t0 < min(seconds, 5.0):
            po.hc_producer(state, *args)
            reps += 1
        dt = (time.perf_counter() - t0) / reps / state.shape[0]
        per_token = (self.bytes_per_step - 24 * self.hc * self.hidden * 4) / self.tokens
        port = {"value": per_token / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{reps} x {state.shape[0]} tokens through hc_pre -> rms_norm -> FP8 pack on one core "
                          f"({dt * 1e3:.3f} ms per token)"}
        return port, dict(port)


METRIC = "HBM GB/s (% of peak) for FP8/MXFP4 MoE GEMV; MFMA TFLOPS at M=512 grouped GEMM"


def _percentile(sorted_values, q):
    at = q * (len(sorted_values) - 1)
    lo, hi = int(math.floor(at)), int(math.ceil(at))
    return sorted_values[lo] + (sorted_values[hi] - sorted_values[lo]) * (at - lo)


def measure(ctx, wl, steps: int, warmup: int, cpu_seconds: float, no_cpu: bool, calibrate: bool = False) -> dict:
    """Parity check, then W warm-up steps, then exactly K steps timed as one HIP graph between two
    synchronisations; the dominant kernel alone between two events on its launch stream; the CPU
    baseline.  Returns the fields of one JSON line."""
    import torch

    parity = wl.check()
    if calibrate:
        src = torch.ones(64 << 20, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        torch.neg(src, out=dst)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # eager: W warm-up steps, then exactly K steps between synchronisations
    for _ in range(warmup):
        wl.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        wl.step()
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) * 1e3 / steps

    # graph: the same K steps captured once, replayed as the timed region
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    ctx._stream = side
    capturable = getattr(wl, "capturable", True)
    per_step = []
    with torch.cuda.stream(side):
        wl.step()
        side.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if capturable:
            with torch.cuda.graph(graph, stream=side):
                for _ in range(steps):
                    wl.step()
            for _ in range(max(1, warmup // 10)):
                graph.replay()
            side.synchronize()
            # every replay is exactly K steps between two synchronisations, clocked on the host (and
            # between two events for the distribution); at least 200 steps in all
            walls = []
            for _ in range(1 + max(5, -(-200 // steps))):
                t0 = time.perf_counter()
                start.record(side)
                graph.replay()
                stop.record(side)
                side.synchronize()
                walls.append((time.perf_counter() - t0) * 1e3 / steps)
                per_step.append(start.elapsed_time(stop) / steps)
            first_wall_ms = walls[0]
            wall_ms = sorted(walls)[len(walls) // 2]
        else:
            # a step with host work in it (file reads, a host-to-device copy it waits for): timed eagerly
            t0 = time.perf_counter()
            for _ in range(steps):
                wl.step()
            side.synchronize()
            wall_ms = first_wall_ms = (time.perf_counter() - t0) * 1e3 / steps
            for _ in range(5):
                t1 = time.perf_counter()
                for _ in range(max(1, steps // 5)):
                    wl.step()
                side.synchronize()
                per_step.append((time.perf_counter() - t1) * 1e3 / max(1, steps // 5))
        kernel_ms = sorted(per_step)[len(per_step) // 2]
        dominant, dominant_bytes = getattr(wl, "dominant", "skinny_gemv_kernel"), wl.bytes_per_step
        if hasattr(wl, "dominant_step"):
            # the dominant kernel alone, K launches between two events on the launch stream
            dominant_bytes = getattr(wl, "dominant_bytes", wl.bytes_per_step)
            for _ in range(3):
                wl.dominant_step()
            side.synchronize()
            start.record(side)
            for _ in range(steps):
                wl.dominant_step()
            stop.record(side)
            side.synchronize()
            kernel_ms = start.elapsed_time(stop) / steps
    ctx._stream = None

    mfma = getattr(wl, "bound", "hbm") == "mfma"
    gbs = wl.bytes_per_step / (wall_ms * 1e-3) / 1e9
    tflops = wl.flops_per_step / (wall_ms * 1e-3) / 1e12
    if mfma:
        achieved = getattr(wl, "dominant_flops", wl.flops_per_step) / (kernel_ms * 1e-3) / 1e12
        peak, unit, per_launch_key, per_launch = wl.peak, "TFLOP/s", "algorithmic_flops_per_launch", wl.dominant_flops
    else:
        achieved = dominant_bytes / (kernel_ms * 1e-3) / 1e9
        peak, unit, per_launch_key, per_launch = HBM_PEAK_GBS, "GB/s", "algorithmic_bytes_per_launch", dominant_bytes
    ordered_steps = sorted(per_step)
    result = {
        "value": round(tflops if mfma else gbs, 1), "unit": unit, "steps": steps, "warmup": warmup,
        "ms_per_step": round(wall_ms, 6),
        "dtype": "e4m3 activations x (e2m1|e4m3) weights, f32 accumulate" if mfma
                 else getattr(wl, "dtype", "bf16 activations x (e2m1|e4m3) weights, f32 accumulate"),
        "config": {"workload": wl.label, "algorithmic_bytes_per_step": wl.bytes_per_step,
                   "algorithmic_flops_per_step": wl.flops_per_step,
                   ("routings_rotated" if hasattr(wl, "routings") else "weight_copies_rotated"):
                       getattr(wl, "rotated", None) or len(wl.handles),
                   "timed_region": "one HIP graph of K steps" if capturable else "K eager steps"},
        "roofline": {"bound": "mfma" if mfma else "hbm", "kernel": dominant, "achieved": round(achieved, 1),
                     "peak": peak, "unit": unit, "frac": round(achieved / peak, 4),
                     per_launch_key: per_launch, "avg_launch_ms": round(kernel_ms, 6),
                     "traffic": traffic_from_profile(getattr(wl, "profile", None), getattr(wl, "profile_kernels", ()))},
        "extra": {"pct_of_peak": round(100 * (tflops / peak if mfma else gbs / HBM_PEAK_GBS), 2),
                  "eager_ms_per_step": round(eager_ms, 6), "first_replay_ms_per_step": round(first_wall_ms, 6), "gbs": round(gbs, 1), "tflops": round(tflops, 3),
                  "replays": {"count": len(per_step), "steps_each": steps if capturable else max(1, steps // 5),
                              "median_ms_per_step": round(_percentile(ordered_steps, 0.5), 6),
                              "p10_ms_per_step": round(_percentile(ordered_steps, 0.1), 6),
                              "p90_ms_per_step": round(_percentile(ordered_steps, 0.9), 6)},
                  "parity": parity},
    }
    if mfma:
        # for information: the MXFP4/FP6 peak, which the mixed FP8 x FP4 instruction does not issue at
        result["extra"]["pct_of_fp4_peak"] = round(100 * tflops / 10100.0, 2)
    if not no_cpu:
        port, multi = wl.cpu_baseline(cpu_seconds)
        result["cpu_baseline"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in port.items()}
        result["extra"]["cpu_multicore"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in multi.items()}
    return result


def headline(result: dict) -> dict:
    """One measured workload -> the JSON line of the benchmark contract."""
    line = {"metric": METRIC, "value": result["value"], "unit": result["unit"], "n_gpus": 1, "steps": result["steps"],
            "warmup": result["warmup"], "ms_per_step": result["ms_per_step"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": result["dtype"], "data": "synthetic",
            "config": result["config"], "roofline": result["roofline"]}
    if "cpu_baseline" in result:
        line["cpu_baseline"] = result["cpu_baseline"]
    line["extra"] = result["extra"]
    return line


def default_steps(workload: str) -> int:
    return {"moe_decode": 50, "fp8_gemm": 50, "moe_prefill": 10}.get(workload, 200)


def run_all(ctx, args) -> dict:
    """Every configuration of the baseline in one run; configs[2] (the headline) last."""
    import gc

    import torch

    from ferrule_amd import synthetic

    side_cpu = max(2.0, args.cpu_seconds / 3.0)
    entries = []

    def run(name, make, steps):
        t0 = time.perf_counter()
        wl = make()
        result = measure(ctx, wl, steps, args.warmup, side_cpu, args.no_cpu)
        entry = {"name": name, **{k: result[k] for k in ("value", "unit", "steps", "ms_per_step", "dtype", "config",
                                                         "roofline")}}
        if "cpu_baseline" in result:
            entry["cpu_baseline"] = result["cpu_baseline"]
            entry["cpu_multicore"] = result["extra"]["cpu_multicore"]
        entry["replays"] = result["extra"]["replays"]
        entry["parity"] = result["extra"]["parity"]
        entries.append(entry)
        print(f"bench.py: {name}: {result['value']} {result['unit']}, {result['roofline']['frac']:.3f} of peak "
              f"({time.perf_counter() - t0:.0f} s)", file=sys.stderr, flush=True)
        del wl
        gc.collect()
        torch.cuda.empty_cache()
        return result

    run("configs[0] fp8_gemv", lambda: GemvWorkload(ctx, "fp8_gemv", 1, args.expert_order), 200)
    for batch in (1, 4, 8):
        run(f"configs[1] mxfp4_gemv B={batch}", lambda: GemvWorkload(ctx, "mxfp4_gemv", batch, args.expert_order), 200)
    # beside configs[1], not in its place: the same matrix shape when a layer's independent linears
    # share one launch (eight distinct matrices here), which is how a decode step would issue them
    run("configs[1] mxfp4_gemv B=1, 8 matrices per launch",
        lambda: GemvWorkload(ctx, "mxfp4_gemv", 1, args.expert_order, matrices=8), 200)
    # a layer's worth of dense decode linears of one format in one launch: where the GEMV reaches the HBM rate
    run("configs[1] mxfp4_gemv B=1, 32 matrices per launch",
        lambda: GemvWorkload(ctx, "mxfp4_gemv", 1, args.expert_order, matrices=32), 100)
    # the FP8-activation entry points at decode row counts: the row count selects a stream over the weights
    run("fp8_gemm at decode rows, M=1 N=7168", lambda: Fp8GemmWorkload(ctx, 1, 7168), 200)
    run("fp8_gemm at decode rows, M=16 N=7168", lambda: Fp8GemmWorkload(ctx, 16, 7168), 200)
    run("shared_ffn at decode rows, M=1", lambda: SharedFfnWorkload(ctx, 1), 200)
    run("configs[3] fp8_gemm M=512 N=7168", lambda: Fp8GemmWorkload(ctx, 512, 7168), 50)
    run("configs[3] fp8_gemm M=2048 N=7168", lambda: Fp8GemmWorkload(ctx, 2048, 7168), 50)
    run("configs[3] fp8_gemm M=4096 N=18432", lambda: Fp8GemmWorkload(ctx, 4096, 18432), 50)
    run("configs[4] moe_prefill", lambda: MoePrefillWorkload(ctx, 8192, expert_order=args.expert_order), 10)
    steps = args.steps if args.steps is not None else default_steps("moe_decode")
    t0 = time.perf_counter()
    wl = MoeDecodeWorkload(ctx, args.expert_order, args.decode_tokens, args.hot_experts, known_groups=args.known_groups,
                               shape=tuple(int(v) for v in args.decode_shape.split(",")) if args.decode_shape else None)
    result = measure(ctx, wl, steps, args.warmup, args.cpu_seconds, args.no_cpu, args.calibrate)
    print(f"bench.py: configs[2] moe_decode: {result['value']} {result['unit']} ({time.perf_counter() - t0:.0f} s)",
          file=sys.stderr, flush=True)
    line = headline(result)
    line["extra"]["configs"] = entries
    # the same layer when the routes concentrate on 16 of the 256 experts (32 rows per expert): fewer weight
    # bytes per step, the packed + general kernels instead of the packed ones alone
    t0 = time.perf_counter()
    hot = MoeDecodeWorkload(ctx, args.expert_order, args.decode_tokens, 16, experts=(wl.table, wl.handles),
                            known_groups=args.known_groups)
    hot_result = measure(ctx, hot, steps, args.warmup, 0.0, True)
    line["extra"]["concentrated_routing"] = {k: hot_result[k] for k in ("value", "unit", "ms_per_step", "config", "roofline")}
    line["extra"]["concentrated_routing"]["parity"] = hot_result["extra"]["parity"]
    print(f"bench.py: moe_decode, routes on 16 experts: {hot_result['ms_per_step']} ms per step "
          f"({time.perf_counter() - t0:.0f} s)", file=sys.stderr, flush=True)
    return line


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); the path shards by "
              "output rows / experts with no exchange between GPUs inside a layer", file=sys.stderr)
        sys.exit(2)

    import torch

    from ferrule_amd.provider import HipArtifactOperatorContext

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the provider has no CPU path", file=sys.stderr)
        sys.exit(2)
    ctx = HipArtifactOperatorContext(0)
    if args.workload == "all":
        print(json.dumps(run_all(ctx, args)))
        return
    if args.steps is None:
        args.steps = default_steps(args.workload)
    if args.workload == "moe_decode":
        wl = MoeDecodeWorkload(ctx, args.expert_order, args.decode_tokens, args.hot_experts, known_groups=args.known_groups,
                               shape=tuple(int(v) for v in args.decode_shape.split(",")) if args.decode_shape else None)
    elif args.workload == "fp8_gemm":
        wl = Fp8GemmWorkload(ctx, args.m, args.n)
    elif args.workload == "moe_prefill":
        wl = MoePrefillWorkload(ctx, args.tokens, expert_order=args.expert_order)
    elif args.workload == "dense_ffn":
        wl = DenseFfnWorkload(ctx, args.batch, args.expert_order)
    elif args.workload == "shared_ffn":
        wl = SharedFfnWorkload(ctx, args.m if args.m <= 32 else 1, args.tile_schedule)
    elif args.workload == "router":
        wl = RouterWorkload(ctx, args.tokens)
    elif args.workload == "routing_chain":
        wl = RoutingChainWorkload(ctx, args.tokens)
    elif args.workload == "hc_producer":
        wl = HcProducerWorkload(ctx, args.tokens)
    elif args.workload == "expert_upload":
        import tempfile

        wl = ExpertUploadWorkload(ctx, os.path.join(tempfile.gettempdir(), "ferrule_amd_bench_experts"))
    else:
        wl = GemvWorkload(ctx, args.workload, args.batch, args.expert_order, args.matrices)
    print(json.dumps(headline(measure(ctx, wl, args.steps, args.warmup, args.cpu_seconds, args.no_cpu, args.calibrate))))


if __name__ == "__main__":
    main()
