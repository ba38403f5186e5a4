#!/usr/bin/env python3
"""Benchmark of the quantized-weight matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the hot path over one batch of synthetic input, inputs
already resident in HBM.  Decode workloads rotate over enough distinct copies of
the weights (>= 512 MiB) that no launch can be served by the 256 MiB Infinity
Cache.  The timed region is a HIP graph holding exactly K launches (the path is
launch-bound at ~2-5 us per kernel otherwise); the same K launches issued eagerly
are reported under "extra".  One JSON line is printed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
ROTATE_BYTES = 512 << 20       # >= 2x the 256 MiB Infinity Cache


# HBM bytes per launch of the dominant kernel from hardware counters (FETCH_SIZE + WRITE_SIZE, two
# rocprofv3 --pmc runs scaled by the --calibrate copy); the summaries with the commands are under profiles/.
MEASURED_TRAFFIC_BYTES = {
    "moe_gate_up_kernel": 3745300000,  # profiles/moe_decode_layer_config3.txt
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="default 50 (MoE layer) / 200 (GEMV)")
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="moe_decode",
                    choices=["moe_decode", "mxfp4_gemv", "fp8_gemv"])
    ap.add_argument("--batch", type=int, default=1, help="tokens per GEMV step (1, 4 or 8)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="budget of the CPU baseline leg")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch one plain 256 MiB -> 256 MiB elementwise copy, the known-size kernel that "
                         "hardware-counter runs are scaled by")
    return ap.parse_args()


# ----------------------------------------------------------------------------- workloads

class GemvWorkload:
    """configs[1]: MXFP4 dense GEMV N=4096, K=7168 (fused gate+up), BF16 in/out;
    or configs[0] on the GPU: FP8 N=K=4096 with fp32 128x128 block scales."""

    def __init__(self, ctx, name: str, batch: int):
        import torch

        from ferrule_amd.provider import HipArtifactLinearShape as S

        self.ctx, self.name, self.batch = ctx, name, batch
        gen = torch.Generator(device="cuda").manual_seed(0xF3771E + 2)
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
        self.bytes_per_step = wb + sb + batch * self.k * 2 + batch * self.n * 2
        self.flops_per_step = 2 * self.n * self.k * batch
        copies = -(-ROTATE_BYTES // (wb + sb))
        from ferrule_amd.provider import HipArtifactLinearHandle

        self.handles = [HipArtifactLinearHandle(self.shape, packed.reshape(-1).clone(), scales.reshape(-1).clone())
                        for _ in range(copies)]
        self.x = torch.randn((batch, self.k), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
        self.out = torch.empty((batch, self.n), dtype=torch.bfloat16, device="cuda")
        self.host = (packed.cpu().numpy(), scales.cpu().numpy(), self.x.float().cpu().numpy())
        self.cursor = 0

    def step(self):
        self.ctx.artifact_linear_gemv_bf16_into(self.handles[self.cursor % len(self.handles)], self.x, self.out)
        self.cursor += 1

    def check(self):
        """Parity of the last output against the CPU checker (the checker is not timed here)."""
        import numpy as np
        import torch

        from oracle import pyoracle as po
        from tests import helpers as H

        w, s, x = self.host
        self.step()
        torch.cuda.synchronize()
        if self.name == "mxfp4_gemv":
            want = po.linear_fp4(w, s, self.n, self.k, x, threads=8)
            deq = po.dequantize_fp4(w, s, self.n, self.k)
        else:
            want = po.linear_fp8(w, s, self.n, self.k, x, threads=8)
            deq = po.dequantize_fp8(w, s, self.n, self.k)
        absprod = np.abs(x.astype(np.float64)) @ np.abs(deq.astype(np.float64)).T
        worst, decided = H.compare_bf16(self.out.view(torch.int16).cpu().numpy().view(np.uint16), want, absprod, self.k)
        return {"max_bf16_ulp": worst, "decided_by_error_bound": decided, "elements": int(want.size)}

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
        one_token_bytes = self.bytes_per_step - (self.batch - 1) * (self.k * 2 + self.n * 2)
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


class MoeDecodeWorkload:
    """configs[2]: MoE decode layer, 64 tokens, hidden 7168, 256 MXFP4 experts (gate+up
    [4096,7168] as two [2048,7168] matrices, down [7168,2048]), top-8 routing with expert ids
    drawn uniformly without replacement and softmax router weights.  A step is the whole
    layer: invocation reset, route plan (4 launches), gate/up+SwiGLU, down, ranked combine
    with the single BF16 writeback.  The 5 GB of active expert weights exceed the 256 MiB
    Infinity Cache 20-fold, so every step streams them from HBM without rotation."""

    tokens, k, experts, hidden, inter = 64, 8, 256, 7168, 2048

    def __init__(self, ctx):
        import numpy as np
        import torch

        from tests.test_moe_gpu import _routing, build_device_experts
        from tests import helpers as H

        self.ctx = ctx
        self.table, self.handles = build_device_experts(ctx, self.experts, self.hidden, self.inter, H.SEED_BASE + 3)
        rng = H.rng_for(3)
        self.x_host = H.bf16_activations(rng, (self.tokens, self.hidden))
        self.ids, self.weights = _routing(rng, self.tokens, self.k, self.experts)
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
        act = self.tokens * self.hidden * 2
        self.bytes_per_step = self.gate_up_weight_bytes + self.down_weight_bytes + act + self.tokens * self.k * 8 + act
        self.flops_per_step = self.tokens * self.k * 2 * (2 * self.inter * self.hidden + self.hidden * self.inter)
        # dominant kernel: gate/up streams 2/3 of the weights, reads x, writes h as hi+lo BF16
        self.dominant = "moe_gate_up_kernel"
        self.dominant_bytes = self.gate_up_weight_bytes + act + self.tokens * self.k * self.inter * 4
        self.label = (f"configs[2] MoE decode layer: {self.tokens} tokens, hidden {self.hidden}, {self.experts} MXFP4 "
                      f"experts, top-{self.k} ({self.distinct} distinct experts active)")
        self.rotated = 1

    def step(self, stages: int = 0):
        c = self.ctx
        c.begin_expert_group_route_invocation(self.plan, self.tokens * self.k)
        c.prepare_expert_group_route_plan(self.plan, self.table, self.slots, self.gens, self.wts, self.k)
        c.moe_decode_from_prepared_plan(self.plan, self.table, self.x, self.out, stages=stages)

    def dominant_step(self):
        from ferrule_amd import abi

        self.ctx.moe_decode_from_prepared_plan(self.plan, self.table, self.x, None, stages=abi.MOE_DECODE_SKIP_DOWN)

    def _host_expert(self, e):
        return [(h.weight.cpu().numpy().reshape(h.shape.out_features, -1),
                 h.scale.cpu().numpy().reshape(h.shape.out_features, -1), None) for h in self.handles[e]]

    def check(self):
        import numpy as np
        import torch

        from tests import helpers as H
        from tests.test_moe_gpu import _oracle_moe

        self.step()
        torch.cuda.synchronize()
        sample = [5]
        host = {int(e): self._host_expert(int(e)) for e in self.ids[sample].ravel()}
        want, absdown = _oracle_moe(host, self.x_host[sample], self.ids[sample], self.weights[sample], self.hidden,
                                    self.inter)
        got = self.out.view(torch.int16).cpu().numpy().view(np.uint16)[sample]
        worst, decided = H.compare_bf16(got, want, 4.0 * absdown, self.hidden + self.inter)
        return {"max_bf16_ulp": worst, "decided_by_error_bound": decided, "elements": int(want.size),
                "sample": "1 token x 8 routes of the timed batch against the CPU executor"}

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
            (gw, gs, _), (uw, us, _), (dw, ds, _) = cache[e]
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
            (gw, gs, _), (uw, us, _), (dw, ds, _) = cache[int(self.ids[t, j])]
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


# ----------------------------------------------------------------------------- main

def main():
    args = parse_args()
    if args.steps is None:
        args.steps = 50 if args.workload == "moe_decode" else 200
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); the path shards by "
              "output rows / experts with no exchange, see DESIGN.md", file=sys.stderr)
        sys.exit(2)

    import torch

    from ferrule_amd.provider import HipArtifactOperatorContext

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the provider has no CPU path", file=sys.stderr)
        sys.exit(2)
    ctx = HipArtifactOperatorContext(0)
    wl = MoeDecodeWorkload(ctx) if args.workload == "moe_decode" else GemvWorkload(ctx, args.workload, args.batch)
    parity = wl.check()
    if args.calibrate:
        src = torch.ones(64 << 20, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        torch.neg(src, out=dst)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # eager: W warm-up steps, then exactly K steps between synchronisations
    for _ in range(args.warmup):
        wl.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        wl.step()
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # graph: the same K launches captured once, replayed as the timed region
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    ctx._stream = side
    with torch.cuda.stream(side):
        wl.step()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(args.steps):
                wl.step()
        for _ in range(max(1, args.warmup // 10)):
            graph.replay()
        side.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        start.record(side)
        graph.replay()
        stop.record(side)
        side.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        kernel_ms = start.elapsed_time(stop) / args.steps
        dominant, dominant_bytes = getattr(wl, "dominant", "skinny_gemv_kernel"), wl.bytes_per_step
        if hasattr(wl, "dominant_step"):
            # the dominant kernel alone, K launches between two events on the launch stream
            dominant_bytes = wl.dominant_bytes
            for _ in range(3):
                wl.dominant_step()
            side.synchronize()
            start.record(side)
            for _ in range(args.steps):
                wl.dominant_step()
            stop.record(side)
            side.synchronize()
            kernel_ms = start.elapsed_time(stop) / args.steps
    ctx._stream = None

    gbs = wl.bytes_per_step / (wall_ms * 1e-3) / 1e9
    achieved = dominant_bytes / (kernel_ms * 1e-3) / 1e9
    line = {
        "metric": "HBM GB/s (% of peak) for FP8/MXFP4 MoE GEMV; MFMA TFLOPS at M=512 grouped GEMM",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 activations x (e2m1|e4m3) weights, f32 accumulate", "data": "synthetic",
        "config": {"workload": wl.label, "algorithmic_bytes_per_step": wl.bytes_per_step,
                   "weight_copies_rotated": getattr(wl, "rotated", None) or len(wl.handles),
                   "timed_region": "one HIP graph of K steps"},
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "algorithmic_bytes_per_launch": dominant_bytes, "avg_launch_ms": round(kernel_ms, 6),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(dominant)},
        "extra": {"pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2), "eager_ms_per_step": round(eager_ms, 6),
                  "eager_gbs": round(wl.bytes_per_step / (eager_ms * 1e-3) / 1e9, 1),
                  "tflops": round(wl.flops_per_step / (wall_ms * 1e-3) / 1e12, 3), "parity": parity},
    }
    if not args.no_cpu:
        port, multi = wl.cpu_baseline(args.cpu_seconds)
        line["cpu_baseline"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in port.items()}
        line["extra"]["cpu_multicore"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in multi.items()}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
