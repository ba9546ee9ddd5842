"""Benchmark of the MORTAR sparse-MLP path on one MI355X.

Step = one pass of the carved SwiGLU MLP (gate_up with fused SwiGLU, then down) over one batch of synthetic
tokens.  Workload at N=1: d_model 2048, d_ff 5632, 16x16 BCSR at 25 % block density, ternary codes with one
fp32 scale per block, 4096-token prefill (the shapes of benchmark configs 2/3).  The same run also times
the decode GEMVs (batch 1/4/16/64), the ReMoE-routed prefill, and a bounded CPU baseline on the host cores.

Prints ONE JSON line.  `value` = prefill tokens/s with inputs resident in HBM.
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

D_MODEL, D_FF, DENSITY, TOKENS = 2048, 5632, 0.25, 4096
N_CLUSTERS, TOP_K = 352, 88
PEAK_BF16_TFLOPS, PEAK_HBM_GBS = 2500.0, 8000.0
# HBM-side bytes per launch (read + written) measured with `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` on this
# workload and calibrated on a plain copy; the runs and factors are in profiles/bench_prefill_step_hbm_traffic_pmc.md
# and profiles/bench_all_legs_hbm_traffic_pmc.md.  Not measured live: counters need the profiler.
TRAFFIC_GATE_UP_BYTES = 41.57e6 + 46.14e6
TRAFFIC_DOWN_BYTES = 60.41e6 + 17.68e6
TRAFFIC_DECODE_STACK_BYTES = (263.05e6 + 4.54e6) + (145.54e6 + 1.83e6)   # gate_up + down launches, 160 layers, b = 1
TRAFFIC_SOURCE = ("constant from profiles/bench_prefill_step_hbm_traffic_pmc.md and profiles/bench_all_legs_hbm_traffic_pmc.md "
                  "(rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command); not measured in this run")


SETTLE_MS = 100.0       # set from --precondition-ms in main()


def event_time_ms(fn, iters: int, warmup: int = 2, settle: bool = False) -> float:
    """Average duration of fn() measured with HIP events on the current stream.  With `settle`, fn runs untimed for
    SETTLE_MS first: a leg of prefill-sized kernels that follows a leg of small ones starts at lower clocks, and a timed
    region of a few milliseconds would measure that ramp (the same effect the headline step is preconditioned against)."""
    import torch
    if settle and SETTLE_MS > 0:
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < SETTLE_MS * 1e-3:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def _dense_twin(spec, tokens: int, dtype, budget_s: float) -> dict:
    """The reference's CPU-expressible form of the carved MLP (scatter the kept blocks into dense matrices, as
    morph/sparse/stk/ops/matrix_ops.py:37-49 / morph/inference/engine.py:74-84 do, then torch.nn.functional.linear and
    silu * up) timed through PyTorch on the host cores."""
    import numpy as np
    import torch
    import torch.nn.functional as F
    from oracle import mortar_oracle as O
    from mortar_amd import synth
    d_model, d_ff = spec["d_model"], spec["d_ff"]
    mats = []
    for k in ("gate_up", "down"):
        m = spec[k]
        mats.append(torch.from_numpy(O.to_dense(O.effective_blocks(m["codes"], m["scales"]), m["row_idx"], m["col_idx"], m["shape"])).to(dtype))
    x = torch.from_numpy(synth.synth_x(tokens, d_model, seed=999)).to(dtype)

    def run():
        gu = F.linear(x, mats[0])
        return F.linear(F.silu(gu[:, :d_ff]) * gu[:, d_ff:], mats[1])
    with torch.no_grad():
        run()
        t0 = time.perf_counter(); run(); t1 = time.perf_counter() - t0
        reps = max(1, min(200, int(budget_s / max(t1, 1e-4))))
        t0 = time.perf_counter()
        for _ in range(reps):
            run()
        dt = time.perf_counter() - t0
    return {"value": reps * tokens / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{reps} passes over {tokens} tokens, d{d_model}/ff{d_ff}, dense-scatter weights + F.linear + silu*up in "
                      f"{str(dtype).replace('torch.', '')} through PyTorch, {dt:.1f} s"}


def cpu_baseline(spec, sample_tokens: int) -> dict:
    """Host-core baselines on a bounded sample (reported only): the C restatement of the blockwise path (oracle,
    'port'), and the reference's CPU-expressible twin - dense-scatter weights + torch.nn.functional.linear in fp32 and
    bf16 - on the headline shape and on benchmark config 0's single 768 -> 2048 product."""
    import numpy as np
    import torch
    import torch.nn.functional as F
    from oracle import c_oracle, mortar_oracle as O
    from mortar_amd import synth
    x = O.bf16_bits(synth.synth_x(sample_tokens, D_MODEL, seed=999))
    c_oracle.mlp_bf16(x[:8], spec["gate_up"], spec["down"], D_FF)            # warm caches / thread pool
    t0 = time.perf_counter()
    c_oracle.mlp_bf16(x, spec["gate_up"], spec["down"], D_FF)
    t1 = time.perf_counter() - t0
    reps = max(1, min(800, int(round(10.0 / max(t1, 1e-3)))))                # about 10 s of CPU work
    t0 = time.perf_counter()
    for _ in range(reps):
        c_oracle.mlp_bf16(x, spec["gate_up"], spec["down"], D_FF)
    dt = time.perf_counter() - t0
    res = {"value": reps * sample_tokens / dt, "unit": "tokens/s", "cores": c_oracle.num_threads(), "kind": "port",
           "sample": f"{reps} passes over {sample_tokens} tokens of the same d{D_MODEL}/ff{D_FF} MLP, blockwise C "
                     f"BCSR restatement (OpenMP), {dt:.1f} s"}
    twin_tokens = min(sample_tokens, 1024)
    res["dense_twin_fp32"] = _dense_twin(spec, twin_tokens, torch.float32, 5.0)
    res["dense_twin_bf16"] = _dense_twin(spec, twin_tokens, torch.bfloat16, 5.0)
    # benchmark config 0: one 768 -> 2048 product on 64 tokens, the reference's own CPU-runnable case
    m0 = synth.synth_matrix(2048, 768, DENSITY, seed=100)
    W0 = torch.from_numpy(O.to_dense(O.effective_blocks(m0["codes"], m0["scales"]), m0["row_idx"], m0["col_idx"], m0["shape"]))
    x0 = torch.from_numpy(synth.synth_x(64, 768, seed=101))
    c0 = {}
    for name, dt_ in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
        Wd, xd = W0.to(dt_), x0.to(dt_)
        with torch.no_grad():
            F.linear(xd, Wd)
            n = 2000
            t0 = time.perf_counter()
            for _ in range(n):
                F.linear(xd, Wd)
            c0[name] = {"us_per_call": (time.perf_counter() - t0) / n * 1e6}
    xb0 = O.bf16_bits(synth.synth_x(64, 768, seed=101))
    t0 = time.perf_counter()
    for _ in range(200):
        c_oracle.bcsr_spmm_bf16(xb0, m0["codes"], m0["scales"], m0["col_idx"], m0["offsets"])
    c0["blockwise_c_port"] = {"us_per_call": (time.perf_counter() - t0) / 200 * 1e6}
    res["config0_single_spmm_64x768x2048"] = {"dense_linear": c0, "cores": torch.get_num_threads()}
    return res


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="prefill only (for profiling one kernel)")
    ap.add_argument("--cpu-tokens", type=int, default=TOKENS)
    ap.add_argument("--precondition-ms", type=float, default=300.0,
                    help="untimed run of the step before the warm-up steps, so that the clocks have settled")
    args = ap.parse_args()
    global SETTLE_MS
    SETTLE_MS = min(100.0, args.precondition_ms)
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the path shards by tokens with replicated weights; "
                 "no multi-GPU code is part of it). Use --gpus 1.")

    import numpy as np
    import torch
    import mortar_amd
    from mortar_amd import ops, synth

    dev = torch.device("cuda:0")
    spec = synth.synth_mlp(D_MODEL, D_FF, DENSITY, seed=0)
    Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    x = torch.from_numpy(synth.synth_x(TOKENS, D_MODEL, seed=1)).to(torch.bfloat16).to(dev)
    h = torch.empty((TOKENS, D_FF), dtype=torch.bfloat16, device=dev)
    y = torch.empty((TOKENS, D_MODEL), dtype=torch.bfloat16, device=dev)
    ws = torch.empty(ops.mlp_hidden_bytes(TOKENS, D_FF), dtype=torch.uint8, device=dev)

    def step():
        # the MLP forward as the module runs it: gate_up + SwiGLU, then down, hidden activations in the library's layout
        ops.mlp(x, Wgu, Wdn, out=y, hidden=ws)

    # Preconditioning (untimed, before the W warm-up steps): the first ~0.1 s of work on an idle GPU runs 15-25 % slower
    # than the steady state (measured: 130 against 107 us per step inside one process) while the clocks settle, so a timed
    # region that starts 5 steps after idle measures the ramp, not the kernels.  The same step runs for about 0.3 s first.
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < args.precondition_ms * 1e-3:
        for _ in range(50):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps

    flops_gu = 2.0 * TOKENS * 256 * Wgu.nnz
    flops_dn = 2.0 * TOKENS * 256 * Wdn.nnz
    it = max(10, args.steps)
    # per-kernel durations inside the step sequence (gate_up and down alternating, as in the timed region): HIP events on
    # the launch stream around every launch
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(it)]
    step()
    torch.cuda.synchronize()
    for e in evs:
        e[0].record()
        ops.mlp(x, Wgu, Wdn, out=y, hidden=ws, phase=1)          # the same two launches, one at a time
        e[1].record()
        ops.mlp(x, Wgu, Wdn, out=y, hidden=ws, phase=2)
        e[2].record()
    torch.cuda.synchronize()
    ms_gu = sum(e[0].elapsed_time(e[1]) for e in evs) / it
    ms_dn = sum(e[1].elapsed_time(e[2]) for e in evs) / it
    out = {
        "metric": "sparse-MLP prefill tokens/s @ d_model=2048, d_ff=5632, 25% block density, 4096 tokens",
        "value": TOKENS / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic", "precondition_ms": args.precondition_ms,
        "config": {"workload": "carved SwiGLU MLP prefill, d_model 2048 / d_ff 5632, 16x16 BCSR 25 % uniform, "
                               "ternary + per-block scale, 4096 tokens bf16 (benchmark configs 2/3 shapes)",
                   "tokens": TOKENS, "nnz_blocks": [Wgu.nnz, Wdn.nnz]},
        "effective_tflops": (flops_gu + flops_dn) / (ms * 1e-3) / 1e12,
        "roofline": {"bound": "mfma", "kernel": "mortar_resident_kernel<32 tokens, gate_up + SwiGLU>",
                     "achieved": flops_gu / (ms_gu * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops_gu / (ms_gu * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, "traffic": TRAFFIC_GATE_UP_BYTES,
                     "traffic_source": TRAFFIC_SOURCE,
                     "algorithmic_bytes": TOKENS * (D_MODEL + D_FF) * 2 + Wgu.weight_bytes, "ms": ms_gu},
        "roofline_down": {"bound": "mfma", "kernel": "mortar_segmented_kernel<32 tokens, plain> (down, K segments copied asynchronously from the tile-ordered hidden activations)",
                          "achieved": flops_dn / (ms_dn * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                          "frac": flops_dn / (ms_dn * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, "traffic": TRAFFIC_DOWN_BYTES,
                          "traffic_source": TRAFFIC_SOURCE,
                          "algorithmic_bytes": TOKENS * (D_MODEL + D_FF) * 2 + Wdn.weight_bytes, "ms": ms_dn},
    }

    if not args.no_extras:
        # ---- decode: one MLP per call (2 launches), weights warm in cache --------------------------------
        dec = {}
        wbytes = Wgu.weight_bytes + Wdn.weight_bytes
        for B in (1, 4, 16, 64):
            xb = x[:B].contiguous()
            hb = torch.empty((B, D_FF), dtype=torch.bfloat16, device=dev)
            yb = torch.empty((B, D_MODEL), dtype=torch.bfloat16, device=dev)

            def dstep():
                ops.gemv(xb, Wgu, swiglu_out=True, out=hb)
                ops.gemv(hb, Wdn, out=yb)
            t = event_time_ms(dstep, 200, 20)
            abytes = B * (2 * D_MODEL + 2 * D_FF) * 2
            dec[f"b{B}"] = {"us_per_mlp": t * 1e3, "tokens_per_s": B / (t * 1e-3),
                            "algorithmic_GBps": (wbytes + abytes) / (t * 1e-3) / 1e9}
        out["decode_warm"] = dec
        # ---- the same, replayed from a HIP graph of 32 consecutive MLPs (no host launch cost in the figure) ----
        gdec = {}
        for B in (1, 4, 16):
            xb = x[:B].contiguous()
            hb = torch.empty((B, D_FF), dtype=torch.bfloat16, device=dev)
            yb = torch.empty((B, D_MODEL), dtype=torch.bfloat16, device=dev)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    ops.gemv(xb, Wgu, swiglu_out=True, out=hb)
                    ops.gemv(hb, Wdn, out=yb)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(32):
                    ops.gemv(xb, Wgu, swiglu_out=True, out=hb)
                    ops.gemv(hb, Wdn, out=yb)
            t = event_time_ms(graph.replay, 20, 3) / 32
            gdec[f"b{B}"] = {"us_per_mlp": t * 1e3, "tokens_per_s": B / (t * 1e-3),
                             "algorithmic_GBps": (wbytes + B * (2 * D_MODEL + 2 * D_FF) * 2) / (t * 1e-3) / 1e9}
        out["decode_graph"] = gdec
        # ---- routed decode: RMSNorm -> router (two-launch HIP front end) -> tile lists -> routed gate_up -> masked down.
        # 16 clusters of 352 neurons, 4 x 4 product keys, k = 8: the reference's deploy router shape (fused_router.py).
        from mortar_amd.engine import MortarDecodeMLP
        rmlp = synth.mlp_module(spec, dev)
        rmlp.enable_routing(n_clusters=16, activation_ratio=0.5, n_sub_keys=4)
        rdec_mlp = MortarDecodeMLP(rmlp)
        rt = rmlp.router
        rdec = {}
        with torch.no_grad():
            for B in (1, 16):
                xb = x[:B].contiguous()
                xn = ops.rmsnorm(xb)
                t_fused = event_time_ms(lambda: rt.route(xn), 100, 10)
                t_torch = event_time_ms(lambda: ops.remoe_gates(rt.group_logits(xn, 0), rt.activation_k), 100, 10)
                t_eager = event_time_ms(lambda: rdec_mlp(xb), 100, 10)
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    for _ in range(3):
                        rdec_mlp(xb)
                torch.cuda.current_stream().wait_stream(side)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    for _ in range(16):
                        rdec_mlp(xb)
                t_graph = event_time_ms(graph.replay, 20, 3) / 16
                rdec[f"b{B}"] = {"us_per_mlp_graph": t_graph * 1e3, "us_per_mlp_eager": t_eager * 1e3,
                                 "router_us_eager": t_fused * 1e3, "router_us_eager_torch_ops": t_torch * 1e3}
                del graph
        out["decode_routed"] = rdec
        del rmlp, rdec_mlp
        # ---- decode, cold: stream distinct weight sets so that the Infinity Cache cannot hold them --------
        n_sets = 160                                                 # 160 x 2.37 MB = 379 MB > 256 MB
        packs = []
        for i in range(n_sets):
            packs.append((Wgu, Wdn) if i == 0 else (Wgu.clone_weights(), Wdn.clone_weights()))
        cold = {}
        for B in (1, 4, 16, 64):                                     # the batches of benchmark config 2
            xb = x[:B].contiguous()
            hb = torch.empty((B, D_FF), dtype=torch.bfloat16, device=dev)
            yb = torch.empty((B, D_MODEL), dtype=torch.bfloat16, device=dev)

            def sweep():
                for g, d in packs:
                    ops.gemv(xb, g, swiglu_out=True, out=hb)
                    ops.gemv(hb, d, out=yb)
            t = event_time_ms(sweep, 5, 1) / n_sets
            abytes = B * (2 * D_MODEL + 2 * D_FF) * 2
            gbps = (wbytes + abytes) / (t * 1e-3) / 1e9
            cold[f"b{B}"] = {"us_per_mlp": t * 1e3, "tokens_per_s": B / (t * 1e-3), "algorithmic_GBps": gbps,
                             "frac_hbm": gbps / PEAK_HBM_GBS}
        out["decode_cold"] = cold
        # ---- decode, layer-batched: the 160 weight sets in TWO launches (gate_up stack, down stack) ---------
        stack = {}
        for B in (1, 4, 16, 64):
            xb = x[:B].contiguous()
            hs = [torch.empty((B, D_FF), dtype=torch.bfloat16, device=dev) for _ in range(n_sets)]
            ys = [torch.empty((B, D_MODEL), dtype=torch.bfloat16, device=dev) for _ in range(n_sets)]
            up = ops.LayerStack([g for g, _ in packs], [xb] * n_sets, hs, swiglu=True)
            dn = ops.LayerStack([d for _, d in packs], hs, ys, swiglu=False)
            t_up = event_time_ms(up.run, 10, 2)
            t_dn = event_time_ms(dn.run, 10, 2)
            b_up = n_sets * (Wgu.weight_bytes + B * (D_MODEL + D_FF) * 2)
            b_dn = n_sets * (Wdn.weight_bytes + B * (D_MODEL + D_FF) * 2)
            stack[f"b{B}"] = {"us_per_mlp": (t_up + t_dn) * 1e3 / n_sets, "tokens_per_s": B * n_sets / ((t_up + t_dn) * 1e-3),
                              "gate_up_ms": t_up, "gate_up_GBps": b_up / (t_up * 1e-3) / 1e9,
                              "down_ms": t_dn, "down_GBps": b_dn / (t_dn * 1e-3) / 1e9,
                              "algorithmic_GBps": (b_up + b_dn) / ((t_up + t_dn) * 1e-3) / 1e9,
                              "frac_hbm": (b_up + b_dn) / ((t_up + t_dn) * 1e-3) / 1e9 / PEAK_HBM_GBS}
            del up, dn, hs, ys
        out["decode_stack"] = stack
        out["roofline_decode"] = {"bound": "hbm", "kernel": "mortar_resident_kernel<4 tokens>, gate_up + down launches of 160 layers each, b=1",
                                  "form": "bandwidth probe: 160 independent MLP weight sets per launch (two launches), not a model's "
                                          "decode step; one real MLP per step is `one_mlp_per_step` below",
                                  "one_mlp_per_step": {k: {"us_per_mlp": v["us_per_mlp"], "achieved": v["algorithmic_GBps"],
                                                           "frac": v["algorithmic_GBps"] / PEAK_HBM_GBS,
                                                           "form": "gate_up + down launches of ONE MLP, HIP-graph replay, weights warm in cache"}
                                                       for k, v in gdec.items()},
                                  "traffic_over_algorithmic": TRAFFIC_DECODE_STACK_BYTES / float(n_sets * (wbytes + (2 * D_MODEL + 2 * D_FF) * 2)),
                                  "achieved": stack["b1"]["algorithmic_GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                  "frac": stack["b1"]["frac_hbm"], "traffic": TRAFFIC_DECODE_STACK_BYTES,
                                  "traffic_source": TRAFFIC_SOURCE,
                                  "by_batch": {k: {"achieved": v["algorithmic_GBps"], "frac": v["frac_hbm"]} for k, v in stack.items()},
                                  "algorithmic_bytes": n_sets * (wbytes + (2 * D_MODEL + 2 * D_FF) * 2)}
        # ---- ReMoE-routed prefill (benchmark config 3) ----------------------------------------------------
        logits = torch.from_numpy(synth.synth_logits(TOKENS, N_CLUSTERS, seed=2)).to(dev)

        def routed():
            # the module's default for prefill-sized calls: gates multiplied in gate_up's epilogue, plain down
            gates, _ = ops.remoe_gates(logits, TOP_K)
            ops.mlp(x, Wgu, Wdn, gates=gates, out=y, hidden=ws)

        def routed_lists():
            # the optional skipping form: token lists per (tile, cluster), routed gate_up, masked down
            gates, active = ops.remoe_gates(logits, TOP_K)
            route = ops.remoe_route(active, ops.route_tile(Wgu, TOKENS))
            ops.gateup_swiglu(x, Wgu, gates=gates, route=route, out=h)
            ops.spmm(h, Wdn, active=active, out=y)
        # the four forms are timed in turn, three rounds, medians: the same conditions for the routed forms and the
        # unrouted step they are compared with
        rounds = {"unrouted": [], "routed": [], "lists": [], "gates": []}
        for r in range(3):
            rounds["unrouted"].append(event_time_ms(step, it, settle=(r == 0)))
            rounds["routed"].append(event_time_ms(routed, it))
            rounds["lists"].append(event_time_ms(routed_lists, it))
            rounds["gates"].append(event_time_ms(lambda: ops.remoe_gates(logits, TOP_K), it))
        t_unrouted, t, t_lists, t_gates = (sorted(rounds[k])[1] for k in ("unrouted", "routed", "lists", "gates"))
        act_now = ops.remoe_gates(logits, TOP_K)[1]
        n_act = int(act_now.sum())
        act_frac = n_act / (TOKENS * N_CLUSTERS)
        cnt_now = ops.remoe_route(act_now, ops.route_tile(Wgu, TOKENS))[0].to(torch.int64)
        sub_exec = int(((cnt_now + 15) // 16).sum())             # 16-token MFMA sub-tiles the routed gate_up executes
        fl_active = (flops_gu + flops_dn) * act_frac          # products whose hidden cluster is active for the token
        out["routed_prefill"] = {"ms": t, "tokens_per_s": TOKENS / (t * 1e-3), "active_fraction": act_frac,
                                 "unrouted_ms_same_conditions": t_unrouted, "vs_unrouted": t / t_unrouted, "gates_launch_ms": t_gates,
                                 "form": "remoe_gates + MLP with the gates multiplied in gate_up's epilogue (module default)",
                                 "token_list_form": {"ms": t_lists, "vs_unrouted": t_lists / t_unrouted,
                                                     "gather_efficiency": n_act / (16.0 * sub_exec),      # active tokens per executed MFMA column
                                                     "mfma_subtiles_executed": sub_exec / float(cnt_now.numel() * (ops.route_tile(Wgu, TOKENS) // 16)),
                                                     "form": "remoe_gates + remoe_route + routed gate_up + masked down (route_skip=True)"},
                                 "roofline": {"bound": "mfma", "kernel": "remoe_gates + gated gate_up + down",
                                              "achieved": fl_active / (t * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                              "frac": fl_active / (t * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, "traffic": None,
                                              "note": "FLOPs of active (token, cluster) pairs only; a cluster is one 16-neuron row unit, "
                                                      "so a 32-token tile keeps about 8 active tokens per unit and the weight unpack, "
                                                      "which bounds the kernel, does not shrink with the active share: nothing is skipped"}}
        # ---- the router that produces those logits in a model (TileRouter over 352 clusters, 19 x 19 product keys): the dense
        # query projection through the library, everything behind it in one launch; beside it the eager torch ops
        from mortar_amd.routing import TileRouter
        torch.manual_seed(3)
        rt352 = TileRouter(N_CLUSTERS, D_MODEL, activation_ratio=TOP_K / N_CLUSTERS).to(dev).eval()
        with torch.no_grad():
            qv = torch.nn.functional.linear(x.float(), rt352.query_proj.weight)
            t_route = event_time_ms(lambda: rt352.route(x), 10, 2, settle=True)
            t_tail = event_time_ms(lambda: ops.router_tail(qv, rt352.iter_embed[0], rt352.query_norm.weight, rt352.query_norm.bias,
                                                           rt352.query_norm.eps, rt352.sub_keys_a, rt352.sub_keys_b,
                                                           rt352.group_bias, rt352.activation_k), 10, 2)
            t_torch = event_time_ms(lambda: ops.remoe_gates(rt352.group_logits(x, 0), rt352.activation_k), 10, 2)
        out["router_prefill"] = {"route_ms": t_route, "tail_kernel_ms": t_tail, "eager_torch_ops_ms": t_torch,
                                 "form": "TileRouter.route at 4096 tokens: fp32 query projection (library GEMM, 34 GFLOP) + one launch for "
                                         "LayerNorm, sub-key scores, ranked product-key logits and gates; eager = the module's torch ops + gates kernel"}
        del qv, rt352
        # ---- the reference's own deploy format: ONE scale per matrix (pack_mortar_ternary), same shapes ----------
        spec_u = {k: dict(spec[k]) for k in ("gate_up", "down")}
        spec_u["gate_up"]["scales"], spec_u["down"]["scales"] = np.float32(0.05), np.float32(0.03)
        Ugu, Udn = synth.to_pack(spec_u["gate_up"], dev), synth.to_pack(spec_u["down"], dev)

        def ustep():
            ops.mlp(x, Ugu, Udn, out=y, hidden=ws)
        t = event_time_ms(ustep, it, settle=True)
        xb = x[:1].contiguous()
        upacks = [(Ugu, Udn) if i == 0 else (Ugu.clone_weights(), Udn.clone_weights()) for i in range(n_sets)]
        hs = [torch.empty((1, D_FF), dtype=torch.bfloat16, device=dev) for _ in range(n_sets)]
        ys = [torch.empty((1, D_MODEL), dtype=torch.bfloat16, device=dev) for _ in range(n_sets)]
        up = ops.LayerStack([g for g, _ in upacks], [xb] * n_sets, hs, swiglu=True)
        dn = ops.LayerStack([d for _, d in upacks], hs, ys, swiglu=False)
        t_s = event_time_ms(up.run, 10, 2) + event_time_ms(dn.run, 10, 2)
        b_s = n_sets * (wbytes - 4 * (Wgu.nnz + Wdn.nnz) + (2 * D_MODEL + 2 * D_FF) * 2)     # no scale per block to read
        out["per_tensor_scale"] = {"prefill_ms": t, "prefill_tokens_per_s": TOKENS / (t * 1e-3),
                                   "prefill_effective_tflops": (flops_gu + flops_dn) / (t * 1e-3) / 1e12,
                                   "decode_stack_b1_us_per_mlp": t_s * 1e3 / n_sets,
                                   "decode_stack_b1_GBps": b_s / (t_s * 1e-3) / 1e9,
                                   "decode_stack_b1_frac_hbm": b_s / (t_s * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                   "note": "blocks multiplied as +-2 / 0, fp32 sums scaled once (scale-after-sum, as the "
                                           "reference's decode kernel); the headline uses per-block scales"}
        # the reference engine's own decode arithmetic on that format: fp32 activations in and out, exact products,
        # fp32 scale after the sums (mortar_gemv with fp32 x); 8 MLPs (gate_up + SwiGLU, then down) per graph replay
        f32dec = {}
        for B in (1, 16):
            xf = x[:B].float().contiguous()
            hf = torch.empty((B, D_FF), dtype=torch.float32, device=dev)
            yf = torch.empty((B, D_MODEL), dtype=torch.float32, device=dev)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    ops.gemv_f32(xf, Ugu, swiglu_out=True, out=hf)
                    ops.gemv_f32(hf, Udn, out=yf)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(8):
                    ops.gemv_f32(xf, Ugu, swiglu_out=True, out=hf)
                    ops.gemv_f32(hf, Udn, out=yf)
            t_f = event_time_ms(graph.replay, 10, 2) / 8
            f32dec[f"b{B}"] = {"us_per_mlp_graph": t_f * 1e3, "tokens_per_s": B / (t_f * 1e-3)}
            del graph
        out["per_tensor_scale"]["decode_fp32_arithmetic"] = f32dec
        del up, dn, hs, ys, upacks, Ugu, Udn

    if not args.no_extras:
        # ---- benchmark config 1: base-width MLP (d_model 768, d_ff 2048), 4 x 4096 tokens ---------------------
        spec1 = synth.synth_mlp(768, 2048, DENSITY, seed=10)
        G1, D1 = synth.to_pack(spec1["gate_up"], dev), synth.to_pack(spec1["down"], dev)
        x1 = torch.from_numpy(synth.synth_x(16384, 768, seed=11)).to(torch.bfloat16).to(dev)
        h1 = torch.empty(ops.mlp_hidden_bytes(16384, 2048), dtype=torch.uint8, device=dev)
        y1 = torch.empty((16384, 768), dtype=torch.bfloat16, device=dev)

        def step1():
            ops.mlp(x1, G1, D1, out=y1, hidden=h1)
        t = event_time_ms(step1, it, settle=True)
        fl = 2.0 * 16384 * 256 * (G1.nnz + D1.nnz)
        out["base_width_prefill"] = {"ms": t, "tokens_per_s": 16384 / (t * 1e-3), "effective_tflops": fl / (t * 1e-3) / 1e12,
                                     "frac_mfma": fl / (t * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}
        del x1, h1, y1
        # ---- benchmark config 4: 8 shared blocks x 6 iterations, Zipf(1.2) rows, RMS-normalised input ----------
        specs = [synth.synth_mlp(D_MODEL, D_FF, DENSITY, seed=20 + i, zipf_s=1.2) for i in range(8)]
        mlps4 = [synth.mlp_module(sp, dev) for sp in specs]
        fused_norm = all(ops.norm_fusable(m4.gate_up._cms.mortar_pack()) for m4 in mlps4)
        t = event_time_ms(lambda: mortar_amd.looped_core_forward(mlps4, x, 6), 3, 1, settle=True)
        fl = 6 * sum(2.0 * TOKENS * 256 * (m4.gate_up._cms.mortar_pack().nnz + m4.down._cms.mortar_pack().nnz) for m4 in mlps4)
        # static load balance of the Zipf rows, read from the schedule tables the kernels run (MortarPack.sched): gate_up's
        # resident kernel gives a workgroup a window of consecutive positions whose units its 16 waves draw dynamically, so
        # what counts is blocks per window; down's K-segmented kernel gives wave w of a 64-position window the positions
        # w, w + 16, ... and ends every K segment with a barrier, so a window costs the sum over the segments of its
        # fullest wave in that segment
        def _sched_blocks(W, rpu):
            sc = W.sched(rpu).cpu().numpy().reshape(-1, W.nseg, rpu, 4)           # [position, segment, row of unit, {g0, g1, nb, unit}]
            return sc[..., 2].astype(np.int64).sum(axis=2)                            # blocks per (position, segment)
        lb_gu, lb_dn = [], []
        for m4 in mlps4:
            Wg4, Wd4 = m4.gate_up._cms.mortar_pack(), m4.down._cms.mortar_pack()
            n_split = max(1, 256 // (-(-TOKENS // 32)))
            per = -(-(Wg4.Rb // 2) // n_split)
            bg = _sched_blocks(Wg4, 2).sum(axis=1)
            wg = np.array([bg[i:i + per].sum() for i in range(0, bg.size, per)])
            lb_gu.append(float(wg.sum() / (wg.size * wg.max())))
            bd = _sched_blocks(Wd4, 1)                                                # [position, segment]
            pad = (-bd.shape[0]) % 64
            bd = np.concatenate([bd, np.zeros((pad, bd.shape[1]), np.int64)]).reshape(-1, 4, 16, bd.shape[1]).sum(axis=1)   # [window, wave, segment]
            lb_dn.append(float(bd.sum() / (16.0 * bd.max(axis=1).sum())))             # all windows: blocks / (waves x barrier-bound blocks)
        out["looped_stack"] = {"ms": t, "mlp_calls": 48, "ms_per_mlp": t / 48, "tokens_per_s": TOKENS / (t * 1e-3),
                               "load_balance_efficiency": {"gate_up_workgroup_windows": min(lb_gu), "down_waves": min(lb_dn),
                                                           "definition": "gate_up: blocks / (windows x blocks of the fullest workgroup window); down: blocks / (16 waves x sum over "
                                                                         "windows and K segments of the fullest wave's blocks); from the schedule tables the kernels "
                                                                         "read; worst of the 8 matrices"},
                               "effective_tflops": fl / (t * 1e-3) / 1e12,
                               "frac_mfma": fl / (t * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                               "norm_fused_into_gate_up": bool(fused_norm),
                               "note": "looped_core_forward over 8 carved MLP modules x 6 iterations: RMSNorm before every MLP, "
                                       "applied while gate_up stages x when norm_fused_into_gate_up (no separate launch); two "
                                       "launches per MLP; rows follow Zipf(1.2) clipped to 5-60 %"}
        del specs, mlps4

    if not args.no_extras:
        # ---- training side (values-ternary QAT): device re-pack of W and W^T, dX through the W^T pack, dW on the
        # topology, for both matrices at the headline shapes (4096 tokens) ------------------------------------------
        from mortar_amd.pack import MortarPack
        bw = {}
        tot = 0.0
        for name, Wf in (("gate_up", Wgu), ("down", Wdn)):
            m = spec[name]
            Wq = MortarPack(None, None, m["col_idx"], m["offsets"], Wf.out_features, Wf.in_features, dev)
            vals = (torch.randn(Wf.nnz, 16, 16, device=dev) * 0.05).to(torch.bfloat16)
            sc = Wq.requantize(vals)
            Wt = Wq.transposed()
            Wt.requantize(vals, scale=sc, transpose=True)
            xin = torch.randn(TOKENS, Wf.in_features, device=dev).to(torch.bfloat16)
            dy = torch.randn(TOKENS, Wf.out_features, device=dev).to(torch.bfloat16)
            dx = torch.empty_like(xin)
            dw = torch.empty(Wf.nnz, 16, 16, dtype=torch.bfloat16, device=dev)
            fl = 2.0 * TOKENS * 256 * Wf.nnz
            t_rq = event_time_ms(lambda: Wt.requantize(vals, scale=Wq.requantize(vals, sync=False), transpose=True, sync=False), 10, settle=True)
            t_dx = event_time_ms(lambda: ops.spmm(dy, Wt, out=dx), 10, settle=True)
            t_dw = event_time_ms(lambda: ops.sdd(dy, xin, Wq, out=dw), 10, settle=True)
            bw[name] = {"repack_w_and_wt_us": t_rq * 1e3, "dx_us": t_dx * 1e3, "dx_tflops": fl / (t_dx * 1e-3) / 1e12,
                        "dw_us": t_dw * 1e3, "dw_tflops": fl / (t_dw * 1e-3) / 1e12}
            tot += t_rq + t_dx + t_dw
            del Wq, Wt, vals, xin, dy, dx, dw
        # the whole MLP as a module in values-ternary QAT: forward + backward of one training step (re-pack of both
        # matrices and their transposes, 3 SpMMs forward-type, 2 dW products, SwiGLU and its derivative)
        qmlp = synth.qat_mlp_module(spec, dev)
        xq = x.clone().requires_grad_(True)
        gy = torch.randn(TOKENS, D_MODEL, device=dev).to(torch.bfloat16)

        def train_step():
            for p_ in qmlp.parameters():
                p_.grad = None
            xq.grad = None
            qmlp(xq).backward(gy)
            with torch.no_grad():                       # stand-in for the optimiser: the values change every step
                qmlp.gate_up._cms.mortar_data.add_(1e-6)
                qmlp.down._cms.mortar_data.add_(1e-6)
        t_train = event_time_ms(train_step, 5, 2, settle=True)
        bw["qat_train_step_ms"] = t_train
        bw["qat_train_tokens_per_s"] = TOKENS / (t_train * 1e-3)
        del qmlp, xq, gy
        bw["backward_ms_per_mlp"] = tot
        bw["backward_over_forward"] = tot / (ms_gu + ms_dn)
        bw["note"] = ("per-matrix figures are the backward's matrix products; qat_train_step is forward + backward of the "
                      "MLP module with trainable block values (re-pack, SpMMs, SwiGLU and its derivative, dW), "
                      "4096 tokens; dW sums fp32 over the tokens and rounds to bf16")
        out["training_backward"] = bw

    # A plain device-to-device copy of known size: the yardstick for the FETCH_SIZE / WRITE_SIZE counters when this
    # command runs under `rocprofv3 --pmc` (counter KiB per byte copied), and a practical HBM bandwidth figure.
    cal_src = torch.empty(64 << 20, dtype=torch.uint8, device=dev).fill_(1)
    cal_dst = torch.empty_like(cal_src)
    t_cal = event_time_ms(lambda: cal_dst.copy_(cal_src), 10, 2)
    out["copy_calibration"] = {"bytes_read": cal_src.numel(), "bytes_written": cal_dst.numel(), "ms": t_cal,
                               "GBps_read_plus_write": 2 * cal_src.numel() / (t_cal * 1e-3) / 1e9}

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(spec, args.cpu_tokens)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
