#!/usr/bin/env python3
"""Throughput of the per-layer MoE hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--ops-only]

One step = one pass of the hot path over the serving batch of BASELINE config 3: 32 sequences x 912 tokens
(880 VL + 32 action per sequence, seeded per-token mask), hidden 2048, VL expert 11008, action expert 1024,
bf16: token partition -> row permute (into the K-tiled activation layout) -> gate/up GEMM + SwiGLU (both experts, one launch) -> down GEMM (both
experts, one launch) -> row unpermute.  Inputs are resident in HBM before the timed region.

Prints ONE JSON line.  `value` = algorithmic FFN FLOPs (6*H*(m0*I0 + m1*I1)) / whole-step time, i.e. the
permute and unpermute passes are inside the timed step.  `roofline` is the dominant kernel (gate/up + SwiGLU)
timed by itself with HIP events on its stream.  `cpu_baseline` is the CPU oracle (a restatement of the
reference's PyTorch path) on a bounded sample of the same batch, on this box's host cores.
"""

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "wall-x_amd"))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--ops-only", action="store_true", help="skip the side measurements (M-RoPE, index builders)")
    ap.add_argument("--no-prefill", action="store_true", help="skip the config 5 prefill measurement (36-layer decoder)")
    ap.add_argument("--prefill-mask", default="action_block", choices=["action_block", "action_block_dense", "causal"],
                    help="config 5 attention mask: the reference's causal + bidirectional action block (as two "
                         "maskless attention calls, the action tokens being the last 32 of every row; or through a "
                         "dense mask), or plain causal")
    ap.add_argument("--cpu-seqs", type=int, default=32, help="sequences of the batch the CPU baseline runs (32 = all)")
    ap.add_argument("--kernel-loop", default=None,
                    choices=["gate_up", "down", "down_unpermute", "permute", "permute_plain", "unpermute", "partition", "copy",
                             "layer_one_launch", "mrope", "mrope_packed", "mrope_copy", "config2_index"],
                    help="profiling aid: run only this kernel --steps times (no JSON line); 'layer_one_launch' is "
                         "permute, gate/up and down as the one launch a denoise step gets (three launches at config "
                         "3, where it does not apply); 'copy' is a plain "
                         "device-to-device copy of the [T, H] activations, the known-size yardstick for HBM counters; "
                         "'mrope' / 'mrope_packed' are the M-RoPE apply at config 2 from the two tables / from the "
                         "packed table, 'mrope_copy' a device copy of q and k of the same shape, 'config2_index' the "
                         "three index builders and the packed-table builder at config 2")
    ap.add_argument("--kernel-data", default="normal", choices=["normal", "zeros"],
                    help="with --kernel-loop: the benchmark's normally distributed activations and weights, or all-zero "
                         "ones (same launches and cycle counts, far less switching activity: the pair shows which clock "
                         "the chip holds under each)")
    ap.add_argument("--kernel-shape", default="config3", choices=["config3", "denoise"],
                    help="with --kernel-loop: the batch the kernel runs on -- config 3 (29184 tokens, 28160 VL + 1024 "
                         "action) or config 4's denoise step (2048 action tokens, VL group empty)")
    return ap.parse_args()


def event_ms(fn, iters, warm=10, batch=1):
    """(median, mean) duration of one fn() in ms from HIP events on the current stream.  batch > 1 times that many
    back-to-back calls per event pair, which keeps launch gaps out of the figure for kernels of a few tens of us."""
    import torch

    for _ in range(warm):
        fn()
    times = []
    for _ in range(iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(batch):
            fn()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b) / batch)
    return statistics.median(times), sum(times) / len(times)


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this hot path has no cross-GPU step and every box here has a single "
              "MI355X; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (torch.cuda.is_available() is False)", file=sys.stderr)
        sys.exit(1)
    from wallx_mi355 import _lib, native, workloads as wl

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.kernel_loop in ("mrope", "mrope_packed", "mrope_copy", "config2_index"):
        config2_kernel_loop(dev, args.kernel_loop, args.steps)
        return
    H, I0, I1 = wl.HIDDEN, wl.INTER_VL, wl.INTER_ACT
    B, S, NA = 32, 912, 32
    T = B * S

    # ---- synthetic inputs, resident in HBM ----------------------------------------------------------
    x_cpu, types_cpu, w_cpu = wl.config3()
    if args.kernel_loop and args.kernel_shape == "denoise":
        T = 2048
        x_cpu = wl.randn((1, T, H), 1.0, torch.bfloat16, torch.Generator().manual_seed(4))
        types_cpu = torch.ones(1, T, dtype=torch.bool)
    x = x_cpu.view(T, H).to(dev)
    types = types_cpu.view(T).to(dev)
    weights = [w.to(dev).as_tuple() for w in w_cpu]
    (g0, u0, d0), (g1, u1, d1) = weights
    m1 = int(types_cpu.sum())
    m0 = T - m1
    ffn_flops = 6.0 * H * (m0 * I0 + m1 * I1)
    gate_up_flops = 4.0 * H * (m0 * I0 + m1 * I1)
    down_flops = 2.0 * H * (m0 * I0 + m1 * I1)
    row_bytes = 2.0 * T * H * 2 + 8.0 * T  # read + write of [T, H] bf16 plus the index traffic

    rows_pad = native.padded_sorted_rows(T)
    hmid = torch.empty(rows_pad * max(I0, I1), dtype=torch.bfloat16, device=dev)
    x_sorted = torch.empty_like(x)
    x_tiled = torch.empty(rows_pad * H, dtype=torch.bfloat16, device=dev)
    y_sorted = torch.empty_like(x)
    # expert weights in the K-tiled layout the MFMA kernels read (packed once, outside the timed region)
    pg0, pu0, pd0, pg1, pu1, pd1 = (native.pack_weight(w) for w in (g0, u0, d0, g1, u1, d1))
    y = torch.empty_like(x)
    ws = None
    stream = torch.cuda.current_stream().cuda_stream

    row_id_map, offsets, inverse, ws = native.partition(types, 2, 0, ws, want_sorted=True)

    def partition():  # straight through the C ABI into the buffers above, like the other launches of a step
        _lib.call("wx_partition_build", types.data_ptr(), _lib.WX_U8, T, 1, 2, 0, row_id_map.data_ptr(),
                  inverse.data_ptr(), offsets.data_ptr(), ws[1].data_ptr(), ws[0].data_ptr(), ws[0].numel(), stream)

    def permute():  # the layer's permute: rows go straight into the K-tiled activation matrix
        _lib.call("wx_permute_rows_tiled", x.data_ptr(), x_tiled.data_ptr(), row_id_map.data_ptr(),
                  inverse.data_ptr(), offsets.data_ptr(), T, H, stream)

    def permute_plain():  # the stand-alone op of the reference API (row-major output)
        _lib.call("wx_permute_rows", x.data_ptr(), x_sorted.data_ptr(), row_id_map.data_ptr(), T, 1, H,
                  _lib.WX_BF16, stream)

    def gate_up():
        _lib.call("wx_dual_swiglu_gate_up", x_tiled.data_ptr(), hmid.data_ptr(), offsets.data_ptr(), pg0.data_ptr(),
                  pu0.data_ptr(), pg1.data_ptr(), pu1.data_ptr(), T, H, I0, I1, None, stream)

    def down():  # on its own: rows come out in sorted order
        _lib.call("wx_dual_down_proj", hmid.data_ptr(), y_sorted.data_ptr(), offsets.data_ptr(), pd0.data_ptr(),
                  pd1.data_ptr(), T, H, I0, I1, None, None, stream)

    def down_unpermute():  # the layer's form: every row is stored at its token's position, no separate unpermute
        _lib.call("wx_dual_down_proj", hmid.data_ptr(), y.data_ptr(), offsets.data_ptr(), pd0.data_ptr(),
                  pd1.data_ptr(), T, H, I0, I1, None, inverse.data_ptr(), stream)

    def down_residual():  # ... and the decoder layer's closing residual add in the same stores (here: + x)
        _lib.call("wx_dual_down_proj_residual", hmid.data_ptr(), y.data_ptr(), x.data_ptr(), offsets.data_ptr(),
                  pd0.data_ptr(), pd1.data_ptr(), T, H, I0, I1, None, inverse.data_ptr(), stream)

    def unpermute():
        _lib.call("wx_unpermute_rows", y_sorted.data_ptr(), y.data_ptr(), row_id_map.data_ptr(), None, T, 1, H,
                  _lib.WX_BF16, stream)

    counters = torch.zeros(_lib.load().wx_ffn_fused_workspace_bytes() // 4, dtype=torch.int32, device=dev)

    def layer_one_launch():  # permute, gate/up and down as one launch where the shape allows it (a denoise step)
        _lib.call("wx_dual_swiglu_ffn_fused", x.data_ptr(), x_tiled.data_ptr(), y.data_ptr(), None, offsets.data_ptr(),
                  pg0.data_ptr(), pu0.data_ptr(), pd0.data_ptr(), pg1.data_ptr(), pu1.data_ptr(), pd1.data_ptr(),
                  hmid.data_ptr(), T, H, I0, I1, _lib.i64x2((m0, m1)), inverse.data_ptr(), counters.data_ptr(), stream)

    def step():  # partition -> permute -> gate/up + SwiGLU -> down with the unpermute in its stores
        partition()
        permute()
        gate_up()
        down_unpermute()

    if args.kernel_loop:
        if args.kernel_data == "zeros":
            for t in (x, pg0, pu0, pd0, pg1, pu1, pd1):
                t.zero_()
        permute(); gate_up(); down()
        fn = {"gate_up": gate_up, "down": down, "down_unpermute": down_unpermute, "permute": permute,
              "permute_plain": permute_plain, "layer_one_launch": layer_one_launch,
              "unpermute": unpermute, "partition": partition,
              "copy": lambda: x_sorted.copy_(x)}[args.kernel_loop]
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return

    # ---- the dominant launches by themselves (HIP events on the launch stream) ---------------------------
    # They come first: a process that has just started finds the chip in its idle power state, and the clock it
    # settles at under this load is reached after some tens of milliseconds of continuous work (with nothing before
    # them, 5 warm-up steps of 3 ms leave the timed steps 2 % slower than the same steps after 30).  After these
    # launches the step loop below measures the steady state.
    iters = max(50, args.steps)  # >= 50 timed launches after the warm-ups, median (and mean for the roofline)
    permute()
    t_gate_up, t_gate_up_avg = event_ms(gate_up, iters, warm=40)  # the first loop also carries the clock ramp
    t_down, _ = event_ms(down, iters)
    t_down_unp, _ = event_ms(down_unpermute, iters)

    # ---- the timed region ----------------------------------------------------------------------------
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    tflops = ffn_flops / (elapsed / args.steps) / 1e12

    # ---- the other launches of a step, and the stand-alone movers ---------------------------------------
    # (left out of --ops-only runs, whose kernel trace should hold the step's own two forms of the down launch only)
    t_down_res = None if args.ops_only else event_ms(down_residual, iters)[0]
    t_perm, _ = event_ms(permute, iters, batch=10)
    t_perm_plain, _ = event_ms(permute_plain, iters, batch=10)
    t_unperm, _ = event_ms(unpermute, iters, batch=10)
    t_part, _ = event_ms(partition, iters)
    # the caller fusions: RMSNorm inside the tiled permute, residual add inside the unpermute
    norm_w = torch.ones(H, dtype=torch.bfloat16, device=dev)

    def norm_permute():
        _lib.call("wx_rmsnorm_permute_rows_tiled", x.data_ptr(), norm_w.data_ptr(), 1e-6, x_tiled.data_ptr(),
                  inverse.data_ptr(), offsets.data_ptr(), T, H, stream)

    def unpermute_add():
        _lib.call("wx_unpermute_rows_add", y_sorted.data_ptr(), x.data_ptr(), y.data_ptr(), row_id_map.data_ptr(), T, H,
                  stream)

    normed = torch.empty_like(y)

    def unpermute_add_norm():
        _lib.call("wx_unpermute_rows_add_rmsnorm", y_sorted.data_ptr(), x.data_ptr(), y.data_ptr(), normed.data_ptr(),
                  norm_w.data_ptr(), 1e-6, row_id_map.data_ptr(), T, H, stream)

    t_np, _ = event_ms(norm_permute, iters, batch=10)
    t_ua, _ = event_ms(unpermute_add, iters, batch=10)
    t_uan, _ = event_ms(unpermute_add_norm, iters, batch=10)
    permute()  # x_tiled back to the plain permute's contents for anything that runs after this
    gate_up_tflops = gate_up_flops / (t_gate_up_avg * 1e-3) / 1e12

    extra = {
        "gate_up_swiglu_ms": round(t_gate_up, 4), "gate_up_tflops": round(gate_up_flops / t_gate_up / 1e9, 1),
        "down_ms": round(t_down, 4), "down_tflops": round(down_flops / t_down / 1e9, 1),
        "down_with_unpermute_ms": round(t_down_unp, 4),  # what the step runs: rows stored at their token positions
        "down_with_unpermute_and_residual_ms": None if t_down_res is None else round(t_down_res, 4),
        "ffn_kernels_tflops": round(ffn_flops / (t_gate_up + t_down) / 1e9, 1),
        "permute_ms": round(t_perm, 4), "permute_GBps": round(row_bytes / t_perm / 1e6, 1),
        "permute_rowmajor_ms": round(t_perm_plain, 4), "permute_rowmajor_GBps": round(row_bytes / t_perm_plain / 1e6, 1),
        "unpermute_ms": round(t_unperm, 4), "unpermute_GBps": round(row_bytes / t_unperm / 1e6, 1),
        "permute_frac_hbm_peak": round(row_bytes / t_perm / 1e6 / PEAK_HBM_GBS, 4),
        "partition_us": round(t_part * 1e3, 2),
        "rmsnorm_permute_ms": round(t_np, 4), "rmsnorm_permute_GBps": round(row_bytes / t_np / 1e6, 1),
        "unpermute_residual_ms": round(t_ua, 4),
        "unpermute_residual_GBps": round((row_bytes + 2.0 * T * H) / t_ua / 1e6, 1),  # one more [T, H] read
        "unpermute_residual_rmsnorm_ms": round(t_uan, 4),  # ... and one more [T, H] write (the next reader's norm)
        "unpermute_residual_rmsnorm_GBps": round((row_bytes + 4.0 * T * H) / t_uan / 1e6, 1),
    }

    # Side measurements: none of them enters `value`.  One that fails (out of memory on a smaller card, say) is
    # reported in its place and must not cost the line its contract fields.
    def side(name, fn, *fargs):
        try:
            out = fn(*fargs)
        except Exception as exc:  # noqa: BLE001 - the message goes into the report
            out = {"error": f"{type(exc).__name__}: {exc}"[:300]}
        if name is None:
            extra.update(out)
        else:
            extra[name] = out

    if not args.ops_only:
        side(None, side_measurements, dev, iters)
        side("cold_hbm", cold_measurements, dev, x, row_id_map, T, H, row_bytes, iters)
        side("config4", config4_measurement, dev, weights)
        side("asym_dual_gmm_op", backward_measurement, dev, x, weights, m0)
        side("block_training_step", training_step_measurement, dev, x, types, weights)
        side("ceilings", ceiling_measurements, dev, x, weights, m0)
    if not args.ops_only and not args.no_prefill:
        del x_tiled, hmid, x_sorted, y_sorted, y
        # the harness as it stands: q / k / v projection with bias and M-RoPE in one launch of this library's GEMM, the
        # o projection with its residual add on the same kernel
        side("prefill", prefill_measurement, dev, args.prefill_mask, True)
        # the same forward with both projections on the vendor GEMM (F.linear / addmm) and M-RoPE as its own pass
        side("prefill_vendor_projections", prefill_measurement, dev, args.prefill_mask, False)

    traffic, traffic_source = measured_traffic("gate_up")
    result = {
        "metric": "dual_expert_ffn_tflops",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "config 3 (BASELINE.json configs[2]): dual-expert FFN layer, 32 seq x 912 tokens, hidden 2048, "
                        "VL expert 11008 on 28160 tokens, action expert 1024 on 1024 tokens; "
                        "partition + permute + gate/up+SwiGLU + down + unpermute",
            "tokens": T, "vl_tokens": m0, "action_tokens": m1, "hidden": H, "inter_vl": I0, "inter_action": I1,
            "flops_per_step": ffn_flops,
        },
        "frac_mfma_peak": round(tflops / PEAK_BF16_TFLOPS, 4),
        "roofline": {
            "kernel": "dual_gemm_kernel<swiglu> (gate/up GEMM + SwiGLU, both experts)",
            "bound": "mfma",
            "achieved": round(gate_up_tflops, 2),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(gate_up_tflops / PEAK_BF16_TFLOPS, 4),
            "flops_per_launch": gate_up_flops,
            "avg_launch_ms": round(t_gate_up_avg, 4),
            "traffic": traffic,
            "traffic_source": traffic_source,
        },
        "extra": extra,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(x_cpu, types_cpu, w_cpu, args.cpu_seqs, H, I0, I1)
        if not args.ops_only:
            try:  # the config 2 ops (M-RoPE apply and the index builders) on the host cores, beside their GPU figures
                extra["cpu_baseline_config2"] = cpu_baseline_config2()
            except Exception as exc:  # noqa: BLE001 - the message goes into the report
                extra["cpu_baseline_config2"] = {"error": f"{type(exc).__name__}: {exc}"[:300]}
        if isinstance(extra.get("prefill"), dict) and "tokens_per_s" in extra["prefill"]:
            # the same prefill priced on the host cores (a bounded sample: one layer timed, 36 charged)
            try:
                extra["prefill"]["cpu_baseline"] = cpu_prefill_baseline()
            except Exception as exc:  # noqa: BLE001 - the message goes into the report
                extra["prefill"]["cpu_baseline"] = {"error": f"{type(exc).__name__}: {exc}"[:300]}
    print(json.dumps(result), flush=True)


def _sha256(path):
    import hashlib

    with open(path, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()


def measured_traffic(kernel):
    """(bytes, source) -- HBM-side bytes per launch of `kernel` from the committed rocprofv3 --pmc summary
    (FETCH_SIZE + WRITE_SIZE, each scaled by what the same counter reads for a plain copy of known size).  Counters
    need profiler runs of their own, so a bench.py run READS this figure; `source` says from where, and the figure is
    withheld (None) when the kernel source has changed since the counters were taken."""
    rel = os.path.join("profiles", "config3_hbm_traffic.json")
    try:
        with open(os.path.join(ROOT, rel)) as f:
            doc = json.load(f)
        k = doc["kernels"][kernel]
    except (OSError, KeyError, ValueError):
        return None, f"{rel} absent: not measured"
    want = doc.get("kernel_source_sha256")
    have = _sha256(os.path.join(ROOT, "wall-x_amd", "csrc", "dual_gemm.hip"))
    if want != have:
        return None, (f"{rel} was taken on another version of wall-x_amd/csrc/dual_gemm.hip (recorded sha256 "
                      f"{str(want)[:12]}, current {have[:12]}): stale, withheld")
    return round(k["read_bytes"] + k["write_bytes"]), (
        f"read from {rel} (rocprofv3 --pmc runs of bench.py --kernel-loop {kernel}, taken at commit "
        f"{doc.get('commit', 'unknown')} on dual_gemm.hip sha256 {have[:12]}); not measured in this run")


def side_measurements(dev, iters):
    """M-RoPE bandwidth and index-builder latencies at BASELINE config 2 shapes (reported, not part of `value`)."""
    import torch
    from wallx_mi355 import native, workloads as wl
    from wallx_mi355.fusions import ops

    out = {}
    ids_cpu, grid_cpu = wl.config2_tokens()
    ids, grid = ids_cpu.to(dev), grid_cpu.to(dev)
    grid32 = grid.to(torch.int32)
    args = (2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2)
    pos, _ = ops.get_rope_index(ids, *args, image_grid_thw=grid)
    t, _ = event_ms(lambda: ops.get_rope_index(ids, *args, image_grid_thw=grid), iters)
    out["rope_index_us"] = round(t * 1e3, 2)
    inv_v = wl.vision_inv_freq().to(dev)
    t, _ = event_ms(lambda: native.rot_pos_emb(inv_v, grid, 2, grid_thw_host=grid_cpu), iters)
    out["rot_pos_emb_us"] = round(t * 1e3, 2)
    t, _ = event_ms(lambda: native.get_window_index(grid32, 2, 4, 14, 4, grid_thw_host=grid_cpu), iters)
    out["window_index_us"] = round(t * 1e3, 2)

    # M-RoPE at B = 16, S = 896: q [14336, 16, 128], k [14336, 2, 128] bf16, cos/sin from the positions above
    B, S, D = ids.shape[0], ids.shape[1], wl.HEAD_DIM
    inv = wl.text_inv_freq().to(dev)
    freqs = pos.float()[..., None] * inv
    emb = torch.cat((freqs, freqs), -1)
    cos, sin = emb.cos().to(torch.bfloat16), emb.sin().to(torch.bfloat16)
    q = torch.randn(B, S, wl.N_Q_HEADS, D, device=dev).to(torch.bfloat16).transpose(1, 2)
    k = torch.randn(B, S, wl.N_KV_HEADS, D, device=dev).to(torch.bfloat16).transpose(1, 2)
    qo = torch.empty(B, wl.N_Q_HEADS, S, D, dtype=torch.bfloat16, device=dev)
    ko = torch.empty(B, wl.N_KV_HEADS, S, D, dtype=torch.bfloat16, device=dev)
    sec2 = [2 * v for v in wl.MROPE_SECTION]
    t, _ = event_ms(lambda: native.rope(q, k, cos, sin, qo, ko, sec2), iters, batch=10)
    tokens = B * S
    rope_bytes = 2.0 * 2 * tokens * D * (wl.N_Q_HEADS + wl.N_KV_HEADS) + 2.0 * 2 * tokens * D
    out["mrope_us"] = round(t * 1e3, 2)
    out["mrope_GBps"] = round(rope_bytes / t / 1e6, 1)
    out["mrope_frac_hbm_peak"] = round(rope_bytes / t / 1e6 / PEAK_HBM_GBS, 4)
    # the same rotation with cos/sin evaluated in the kernel from position_ids and inv_freq: no tables are read
    # (algorithmic bytes: q and k in and out plus the three int64 position planes), and the PyTorch ops that build
    # the tables once per forward disappear
    t, _ = event_ms(lambda: native.rope_from_positions(q, k, pos, inv, qo, ko, sec2), iters, batch=10)
    pos_bytes = 2.0 * 2 * tokens * D * (wl.N_Q_HEADS + wl.N_KV_HEADS) + 3.0 * 8 * tokens
    out["mrope_from_positions_us"] = round(t * 1e3, 2)
    out["mrope_from_positions_GBps"] = round(pos_bytes / t / 1e6, 1)
    # ... and with cos/sin read from the packed table (256 bytes per token, built once per forward for all layers)
    table = native.mrope_table(pos, inv, wl.MROPE_SECTION)
    t, _ = event_ms(lambda: native.rope_from_table(q, k, table, qo, ko, sec2), iters, batch=10)
    tab_bytes = 2.0 * 2 * tokens * D * (wl.N_Q_HEADS + wl.N_KV_HEADS) + 4.0 * tokens * (D // 2)
    out["mrope_from_packed_table_us"] = round(t * 1e3, 2)
    out["mrope_from_packed_table_GBps"] = round(tab_bytes / t / 1e6, 1)
    t, _ = event_ms(lambda: native.mrope_table(pos, inv, wl.MROPE_SECTION), iters)
    out["mrope_table_build_us"] = round(t * 1e3, 2)

    def build_tables():
        fr = pos.float()[..., None] * inv
        e = torch.cat((fr, fr), -1)
        return e.cos().to(torch.bfloat16), e.sin().to(torch.bfloat16)

    t, _ = event_ms(build_tables, iters)
    out["cos_sin_tables_torch_us"] = round(t * 1e3, 2)
    return out


def config2_inputs(dev):
    """The config 2 tensors on the device: token ids and grids, position ids, cos / sin tables, q / k as [B, H, S, D]
    views of token-major memory, contiguous outputs, the packed rotary table."""
    import torch
    from wallx_mi355 import native, workloads as wl
    from wallx_mi355.fusions import ops

    ids_cpu, grid_cpu = wl.config2_tokens()
    ids, grid = ids_cpu.to(dev), grid_cpu.to(dev)
    args = (2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2)
    pos, _ = ops.get_rope_index(ids, *args, image_grid_thw=grid)
    B, S, D = ids.shape[0], ids.shape[1], wl.HEAD_DIM
    inv = wl.text_inv_freq().to(dev)
    freqs = pos.float()[..., None] * inv
    emb = torch.cat((freqs, freqs), -1)
    cos, sin = emb.cos().to(torch.bfloat16), emb.sin().to(torch.bfloat16)
    q = torch.randn(B, S, wl.N_Q_HEADS, D, device=dev).to(torch.bfloat16).transpose(1, 2)
    k = torch.randn(B, S, wl.N_KV_HEADS, D, device=dev).to(torch.bfloat16).transpose(1, 2)
    qo = torch.empty(B, wl.N_Q_HEADS, S, D, dtype=torch.bfloat16, device=dev)
    ko = torch.empty(B, wl.N_KV_HEADS, S, D, dtype=torch.bfloat16, device=dev)
    table = native.mrope_table(pos, inv, wl.MROPE_SECTION)
    return dict(ids_cpu=ids_cpu, grid_cpu=grid_cpu, ids=ids, grid=grid, args=args, pos=pos, inv=inv, cos=cos, sin=sin,
                q=q, k=k, qo=qo, ko=ko, table=table, sec2=[2 * v for v in wl.MROPE_SECTION])


def config2_kernel_loop(dev, which, steps):
    """--kernel-loop for the config 2 kernels (profiling aid, no JSON line)."""
    import torch
    from wallx_mi355 import native, workloads as wl
    from wallx_mi355.fusions import ops

    c = config2_inputs(dev)
    grid32 = c["grid"].to(torch.int32)
    inv_v = wl.vision_inv_freq().to(dev)
    torch.cuda.synchronize()
    for _ in range(steps):
        if which == "mrope":
            native.rope(c["q"], c["k"], c["cos"], c["sin"], c["qo"], c["ko"], c["sec2"], layout="hf")
        elif which == "mrope_packed":
            native.rope_from_table(c["q"], c["k"], c["table"], c["qo"], c["ko"], c["sec2"])
        elif which == "mrope_copy":  # the same q / k bytes through the runtime's copy: the yardstick for the counters
            c["qo"].copy_(c["q"])
            c["ko"].copy_(c["k"])
        else:
            ops.get_rope_index(c["ids"], *c["args"], image_grid_thw=c["grid"])
            native.rot_pos_emb(inv_v, c["grid"], 2, grid_thw_host=c["grid_cpu"])
            native.get_window_index(grid32, 2, 4, 14, 4, grid_thw_host=c["grid_cpu"])
            native.mrope_table(c["pos"], c["inv"], wl.MROPE_SECTION)
    torch.cuda.synchronize()


def cpu_baseline_config2():
    """The config 2 ops on the host cores, beside the GPU figures of `extra`: the oracle's restatements of
    apply_multimodal_rotary_pos_emb (vl.py:731-773, eager bf16 like the reference), get_rope_index (act.py:929-1149),
    rot_pos_emb and get_window_index (vl.py:473-547) at the full config 2 sizes.  Median of 5 runs after a warm-up, on
    the threads torch uses on this box (the index builders are Python / single-threaded torch code either way)."""
    import torch
    import oracle
    from wallx_mi355 import workloads as wl

    def med_us(fn, runs=5):
        fn()
        ts = []
        for _ in range(runs):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return round(statistics.median(ts) * 1e6, 1)

    ids, grid = wl.config2_tokens()
    args = (2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2)
    pos, _ = oracle.rope_index_ref(ids, *args, image_grid_thw=grid)
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), torch.bfloat16)
    q, k = wl.qk_inputs(ids.shape[0], ids.shape[1])
    qt, kt = q.transpose(1, 2), k.transpose(1, 2)
    sec = list(wl.MROPE_SECTION)
    inv_v = wl.vision_inv_freq()
    tokens, D = ids.numel(), wl.HEAD_DIM
    rope_bytes = 2.0 * 2 * tokens * D * (wl.N_Q_HEADS + wl.N_KV_HEADS) + 2.0 * 2 * tokens * D
    t_rope = med_us(lambda: oracle.mrope_apply_ref(qt, kt, cos, sin, sec))
    return {
        "mrope_us": t_rope, "mrope_GBps": round(rope_bytes / t_rope / 1e3, 2),
        "cos_sin_tables_us": med_us(lambda: oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), torch.bfloat16)),
        "rope_index_us": med_us(lambda: oracle.rope_index_ref(ids, *args, image_grid_thw=grid)),
        "rot_pos_emb_us": med_us(lambda: oracle.rot_pos_emb_ref(inv_v, grid, 2)),
        "window_index_us": med_us(lambda: oracle.window_index_ref(grid, 112, 2, 14, 4)),
        "cores": torch.get_num_threads(), "kind": "port",
        "sample": "the oracle's functions at the full config 2 sizes (16 x 896 tokens, 48 grids of 1 x 32 x 32, q "
                  "[14336, 16, 128] and k [14336, 2, 128] bf16), median of 5 runs after a warm-up",
    }


def cold_measurements(dev, x, row_id_map, T, H, row_bytes, iters):
    """The bandwidth kernels with operands that are NOT resident in the 256 MB memory-side cache: each call works
    on the next of several buffer sets whose total size is above 1 GB, so every byte comes from and goes to HBM.
    (The per-kernel figures elsewhere in this report reuse one buffer set, which that cache largely holds.)  A
    plain device copy of the same size, timed the same way, is the reference for what HBM sustains."""
    import torch
    from wallx_mi355 import _lib

    stream = torch.cuda.current_stream().cuda_stream
    sets = 5
    xs = [x.clone() for _ in range(sets)]
    outs = [torch.empty_like(x) for _ in range(sets)]
    state = {"i": 0}

    def nxt():
        state["i"] = (state["i"] + 1) % sets
        return state["i"]

    def permute_cold():
        i = nxt()
        _lib.call("wx_permute_rows", xs[i].data_ptr(), outs[i].data_ptr(), row_id_map.data_ptr(), T, 1, H,
                  _lib.WX_BF16, stream)

    def unpermute_cold():
        i = nxt()
        _lib.call("wx_unpermute_rows", xs[i].data_ptr(), outs[i].data_ptr(), row_id_map.data_ptr(), None, T, 1, H,
                  _lib.WX_BF16, stream)

    def copy_cold():
        i = nxt()
        outs[i].copy_(xs[i])

    out = {}
    for name, fn in (("permute_rowmajor", permute_cold), ("unpermute", unpermute_cold), ("device_copy", copy_cold)):
        t, _ = event_ms(fn, iters, warm=sets, batch=sets)
        out[f"{name}_GBps"] = round(row_bytes / t / 1e6, 1)
    out["note"] = f"{sets} buffer sets of {2 * T * H * 2 / 1e6:.0f} MB each, used round-robin; bytes counted as for the warm figures"
    return out


def config4_measurement(dev, weights):
    """BASELINE config 4, the skewed / empty-group regime, through the layer entry point (partition, tiled permute,
    both FFN launches, unpermute) with no retuning between shapes: (i) a denoise step of 2048 action tokens with the
    VL group empty, (ii) a prefill of 4096 VL tokens plus n action tokens.  Activations N(0, 1); the weights are
    the benchmark's N(0, 0.02) tensors (timing does not depend on the weight scale)."""
    import torch
    from wallx_mi355 import moe, native

    H = weights[0][0].shape[1]
    I0, I1 = weights[0][0].shape[0], weights[1][0].shape[0]
    g = torch.Generator(device=dev).manual_seed(4)
    out = {}
    from types import SimpleNamespace
    cfg = SimpleNamespace(experts=[dict(hidden_size=H, intermediate_size=i, hidden_act="silu") for i in (I0, I1)])
    block = moe.SparseMoeBlock(cfg, 2).to(dev).to(torch.bfloat16)
    with torch.no_grad():
        for e, ws in enumerate(weights):
            for prm, w in zip(block.experts[e].weights(), ws):
                prm.copy_(w)
    block.pack_for_inference(free_dense=True)
    cases = [("denoise_2048_action", 0, 2048)] + [(f"prefill_4096_vl_plus_{n}_action", 4096, n) for n in (0, 1, 8, 32, 64)]
    for name, n_vl, n_act in cases:
        T = n_vl + n_act
        x = torch.randn(T, H, device=dev, generator=g).to(torch.bfloat16)
        types = torch.cat([torch.zeros(n_vl, dtype=torch.bool), torch.ones(n_act, dtype=torch.bool)]).to(dev)
        t, _ = event_ms(lambda: moe.moe_layer_forward(x, types, weights), 20, warm=5)
        # the same with the per-expert row counts handed over from the host, as the reference's caller has them
        th, _ = event_ms(lambda: moe.moe_layer_forward(x, types, weights, host_rows=(n_vl, n_act)), 20, warm=5)
        flops = 6.0 * H * (n_vl * I0 + n_act * I1)
        out[name] = {"us": round(t * 1e3, 1), "tflops": round(flops / t / 1e9, 1),
                     "us_with_host_row_counts": round(th * 1e3, 1)}
        # the two figures above are one call between two events on an idle GPU (launch latency included); the same
        # calls queued back to back, 50 per event pair, as a serving loop issues them
        tq, _ = event_ms(lambda: moe.moe_layer_forward(x, types, weights), 6, warm=1, batch=50)
        tqh, _ = event_ms(lambda: moe.moe_layer_forward(x, types, weights, host_rows=(n_vl, n_act)), 6, warm=1, batch=50)
        out[name]["us_per_call_50_calls_queued"] = round(tq * 1e3, 1)
        out[name]["us_per_call_50_calls_queued_with_host_row_counts"] = round(tqh * 1e3, 1)
        # the drop-in module called the way the reference's decoder calls it: every layer gets the same token-type
        # tensor and the CPU row ranges (act.py:257-261, 1274-1283), so the partition is shared between the layers
        x3, types2 = x.view(1, T, H), types.view(1, T)
        start, end = torch.tensor([0, n_vl]), torch.tensor([n_vl, T])
        with torch.no_grad():
            tb, _ = event_ms(lambda: block(x3, types2, start, end), 20, warm=5)
            tbb, _ = event_ms(lambda: block(x3, types2, start, end), 20, warm=5, batch=36)
            # ... and by a caller that passes no CPU row ranges: the cached partition's own asynchronous read-back of
            # expert_offsets supplies the row counts once it has landed
            tbn, _ = event_ms(lambda: block(x3, types2), 20, warm=5, batch=36)
        out[name]["us_drop_in_block_same_token_types"] = round(tb * 1e3, 1)            # one call, GPU idle before it
        out[name]["us_per_layer_drop_in_block_36_calls_back_to_back"] = round(tbb * 1e3, 1)  # as a decoder issues them
        out[name]["us_per_layer_drop_in_block_36_calls_without_row_ranges"] = round(tbn * 1e3, 1)
        if n_vl == 0:
            out[name]["kernels_us"] = denoise_kernel_times(dev, x, types, weights)
            # the denoise loop repeats this shape 10 x 36 times per action chunk: record 36 layers once into a HIP
            # graph (the entry points neither allocate nor synchronise) and time its replays
            layers = 36
            routing = moe.moe_layer_forward(x, types, weights, host_rows=(n_vl, n_act))[1]

            def stack():
                h = x
                for _ in range(layers):
                    h = moe.moe_layer_forward(h, types, weights, routing=routing, host_rows=(n_vl, n_act))[0]
                return h

            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                stack()
            torch.cuda.current_stream().wait_stream(side)
            te, _ = event_ms(stack, 5, warm=2)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                stack()
            tg, _ = event_ms(graph.replay, 10, warm=3)
            out[name]["us_per_layer_eager_shared_routing"] = round(te * 1e3 / layers, 1)
            out[name]["us_per_layer_hip_graph_replay"] = round(tg * 1e3 / layers, 1)
            # the same graph with the layer as its three launches (permute, gate/up, down) instead of one
            native.set_one_launch_ffn(False)
            try:
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    stack()
                torch.cuda.current_stream().wait_stream(side)
                graph3 = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph3):
                    stack()
                tg3, _ = event_ms(graph3.replay, 10, warm=3)
            finally:
                native.set_one_launch_ffn(True)
            out[name]["us_per_layer_hip_graph_replay_three_launches"] = round(tg3 * 1e3 / layers, 1)
            del graph3
            # the same replay with an action expert of its own in every layer, as the model has them: 36 x 12.6 MB of
            # weights no longer stay in the caches between layers, every layer streams its expert from HBM
            (g0, u0, d0), (g1, u1, d1) = weights
            per_layer = [((g0, u0, d0), tuple(w.clone() for w in (g1, u1, d1))) for _ in range(layers)]

            def stack_distinct():
                h = x
                for wl_ in per_layer:
                    h = moe.moe_layer_forward(h, types, wl_, routing=routing, host_rows=(n_vl, n_act))[0]
                return h

            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                stack_distinct()  # packs the 36 action experts outside the capture
            torch.cuda.current_stream().wait_stream(side)
            graph2 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph2):
                stack_distinct()
            tg2, _ = event_ms(graph2.replay, 10, warm=3)
            out[name]["us_per_layer_hip_graph_replay_36_distinct_action_experts"] = round(tg2 * 1e3 / layers, 1)
            del graph2
            native.set_one_launch_ffn(False)
            try:
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    stack_distinct()
                torch.cuda.current_stream().wait_stream(side)
                graph4 = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph4):
                    stack_distinct()
                tg4, _ = event_ms(graph4.replay, 10, warm=3)
            finally:
                native.set_one_launch_ffn(True)
            out[name]["us_per_layer_hip_graph_replay_36_distinct_action_experts_three_launches"] = round(tg4 * 1e3 / layers, 1)
            del graph4, per_layer
    return out


def denoise_kernel_times(dev, x, types, weights):
    """The launches of one denoise layer by themselves (HIP events, 20 back-to-back launches per event pair): tiled
    permute, gate/up + SwiGLU, down with the unpermute in its stores, the host handing over the row counts (one
    dispatch each), and what fraction of the bf16 MFMA peak the two GEMM launches reach."""
    import torch
    from wallx_mi355 import _lib, native

    T, H = x.shape
    (g0, u0, d0), (g1, u1, d1) = weights
    I0, I1 = g0.shape[0], g1.shape[0]
    packed = [native.pack_weight(w) for w in (g0, u0, d0, g1, u1, d1)]
    rmap, off, inv, _ = native.partition(types, 2, 0, None, want_sorted=True)
    rows_pad = native.padded_sorted_rows(T)
    x_tiled = torch.empty(rows_pad * H, dtype=torch.bfloat16, device=dev)
    hmid = torch.empty(rows_pad * max(I0, I1), dtype=torch.bfloat16, device=dev)
    y = torch.empty_like(x)
    n_act = int(types.sum())
    rows = _lib.i64x2((T - n_act, n_act))
    stream = torch.cuda.current_stream().cuda_stream
    p = [t.data_ptr() for t in packed]

    def permute():
        _lib.call("wx_permute_rows_tiled", x.data_ptr(), x_tiled.data_ptr(), rmap.data_ptr(), inv.data_ptr(),
                  off.data_ptr(), T, H, stream)

    def gate_up():
        _lib.call("wx_dual_swiglu_gate_up", x_tiled.data_ptr(), hmid.data_ptr(), off.data_ptr(), p[0], p[1], p[3], p[4],
                  T, H, I0, I1, rows, stream)

    def down():
        _lib.call("wx_dual_down_proj", hmid.data_ptr(), y.data_ptr(), off.data_ptr(), p[2], p[5], T, H, I0, I1, rows,
                  inv.data_ptr(), stream)

    counters = torch.zeros(_lib.load().wx_ffn_fused_workspace_bytes() // 4, dtype=torch.int32, device=dev)

    def one_launch():  # the three of them as one launch: gate/up tiles read the token rows, down tiles wait for them
        _lib.call("wx_dual_swiglu_ffn_fused", x.data_ptr(), x_tiled.data_ptr(), y.data_ptr(), None, off.data_ptr(), p[0],
                  p[1], p[2], p[3], p[4], p[5], hmid.data_ptr(), T, H, I0, I1, rows, inv.data_ptr(), counters.data_ptr(),
                  stream)

    permute(); gate_up(); down(); one_launch()
    t_p, _ = event_ms(permute, 20, warm=3, batch=20)
    t_g, _ = event_ms(gate_up, 20, warm=3, batch=20)
    t_d, _ = event_ms(down, 20, warm=3, batch=20)
    t_1, _ = event_ms(one_launch, 20, warm=3, batch=20)
    f_g, f_d = 4.0 * H * n_act * I1, 2.0 * H * n_act * I1
    return {"permute_tiled": round(t_p * 1e3, 2), "gate_up_swiglu": round(t_g * 1e3, 2),
            "down_with_unpermute": round(t_d * 1e3, 2),
            "gate_up_frac_mfma_peak": round(f_g / t_g / 1e9 / PEAK_BF16_TFLOPS, 3),
            "down_frac_mfma_peak": round(f_d / t_d / 1e9 / PEAK_BF16_TFLOPS, 3),
            "permute_gate_up_down_as_one_launch": round(t_1 * 1e3, 2),
            "one_launch_frac_mfma_peak": round((f_g + f_d) / t_1 / 1e9 / PEAK_BF16_TFLOPS, 3),
            "one_launch_wait_ran_into_its_bound": int(counters[-1].item())}


def backward_measurement(dev, x, weights, m0):
    """The reference's own op, `asym_dual_gmm` on row-major operands (ops.py:6-165), at the gate projection's
    config 3 shapes: the forward (x @ W^T for both experts in one launch, nn.Linear weights read in place) and the
    two backward GEMMs of ops.py:78-144, dX = dY @ W and dW = dY^T @ X, whose K-major operands the same kernel
    transposes between LDS and the registers (no transposed copies)."""
    import torch
    from wallx_mi355 import native

    H = x.shape[1]
    (g0, _, _), (g1, _, _) = weights
    I0, I1 = g0.shape[0], g1.shape[0]
    m1 = x.shape[0] - m0
    gen = torch.Generator(device=dev).manual_seed(2)
    dy0 = torch.randn(m0, I0, device=dev, generator=gen).to(torch.bfloat16)
    dy1 = torch.randn(m1, I1, device=dev, generator=gen).to(torch.bfloat16)
    x0, x1 = x[:m0].contiguous(), x[m0:].contiguous()
    dx0, dx1 = torch.empty_like(x0), torch.empty_like(x1)
    dw0, dw1 = torch.empty_like(g0), torch.empty_like(g1)
    flops = 2.0 * H * (m0 * I0 + m1 * I1)
    y0, y1 = torch.empty_like(dy0), torch.empty_like(dy1)
    t_fw, _ = event_ms(lambda: native.asym_dual_gmm(x0, x1, g0, g1, y0, y1, False, True), 20, warm=5)
    t_dx, _ = event_ms(lambda: native.asym_dual_gmm(dy0, dy1, g0, g1, dx0, dx1, False, False), 20, warm=5)
    t_dw, _ = event_ms(lambda: native.asym_dual_gmm(dy0, dy1, x0, x1, dw0, dw1, True, False), 20, warm=5)
    return {"forward_nt_ms": round(t_fw, 3), "forward_nt_tflops": round(flops / t_fw / 1e9, 1),
            "dx_ms": round(t_dx, 3), "dx_tflops": round(flops / t_dx / 1e9, 1),
            "dw_ms": round(t_dw, 3), "dw_tflops": round(flops / t_dw / 1e9, 1)}


def training_step_measurement(dev, x, token_types, weights):
    """Forward + backward of the drop-in SparseMoeBlock (wallx_mi355/moe.py) on the config 3 batch: the fused forward
    (which keeps the gate / up projections), then the block's own backward (SwiGLU derivative in one elementwise
    kernel, dX and dW of all three projections of both experts as dual GEMMs in their K-major layouts).  FLOPs
    counted as 3 x forward.  Also timed with the VL expert frozen, the reference's freeze_vlm fine-tuning mode
    (qwen_vl_act_trainer.py:530-536): its three weight gradients leave the launches."""
    import torch
    from types import SimpleNamespace
    from wallx_mi355 import moe

    H = x.shape[1]
    inters = [w[0].shape[0] for w in weights]
    cfg = SimpleNamespace(experts=[dict(hidden_size=H, intermediate_size=i, hidden_act="silu") for i in inters])
    block = moe.SparseMoeBlock(cfg, 2).to(dev).to(torch.bfloat16)
    with torch.no_grad():
        for e, (gw, uw, dw) in enumerate(weights):
            block.experts[e].gate_proj.weight.copy_(gw)
            block.experts[e].up_proj.weight.copy_(uw)
            block.experts[e].down_proj.weight.copy_(dw)
    xb = x.detach().clone().view(1, -1, H).requires_grad_(True)
    tb = token_types.view(1, -1)
    dy = torch.randn(xb.shape, device=dev).to(torch.bfloat16)
    routing = block.route(tb)

    def fwd():
        with torch.no_grad():
            block(xb, tb, routing=routing)

    def step():
        for prm in block.parameters():
            prm.grad = None
        xb.grad = None
        block(xb, tb, routing=routing).backward(dy)

    t_f, _ = event_ms(fwd, 5, warm=2)
    t_s, _ = event_ms(step, 5, warm=2)
    m1 = int(token_types.sum())
    flops = 6.0 * H * ((x.shape[0] - m1) * inters[0] + m1 * inters[1])
    out = {"forward_ms": round(t_f, 3), "forward_backward_ms": round(t_s, 3),
           "tflops_counting_3x_forward": round(3 * flops / t_s / 1e9, 1)}
    for prm in block.experts[0].parameters():
        prm.requires_grad_(False)
    t_fz, _ = event_ms(step, 5, warm=2)
    out["forward_backward_ms_vl_expert_frozen"] = round(t_fz, 3)
    del block, xb, dy
    torch.cuda.empty_cache()
    return out


def ceiling_measurements(dev, x, weights, m0):
    """What bounds an MFMA kernel on THIS data, measured on the same GPU in the same run (reported, not part of
    `value`): (1) back-to-back bf16 MFMA instructions with operands held in registers, on zeros and on values
    drawn like the benchmark's activations and weights -- the sustained MFMA rate depends on the operand values
    (switching activity moves the clock the chip holds), so the nominal 2.5 PFLOP/s is not reachable on random
    data; (2) the vendor GEMM (torch.matmul -> hipBLASLt) on the VL expert's two GEMM shapes with the benchmark's
    own tensors, without the SwiGLU epilogue or the second expert."""
    import ctypes
    import torch

    out = {}
    # the probe is a benchmark-only library of its own (wall-x_amd/csrc/probe.hip), not part of the product ABI
    probe = ctypes.CDLL(os.path.join(ROOT, "wall-x_amd", "wallx_mi355", "libwallx_probe.so"))
    probe.wxprobe_mfma_operand_bytes.restype = ctypes.c_size_t
    probe.wxprobe_mfma_rate.restype = ctypes.c_int
    probe.wxprobe_mfma_rate.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    n = probe.wxprobe_mfma_operand_bytes() // 2
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    flops = ctypes.c_double(0.0)
    stream = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device=dev).manual_seed(1)
    data = torch.randn(n, device=dev, generator=g)
    data[n // 2:] *= 0.02  # half the fragments look like activations N(0, 1), half like weights N(0, 0.02)
    for name, ops in (("zeros", torch.zeros(n, dtype=torch.bfloat16, device=dev)), ("normal", data.to(torch.bfloat16))):
        def run():
            if probe.wxprobe_mfma_rate(ops.data_ptr(), 4000, sink.data_ptr(), ctypes.byref(flops), stream) != 0:
                raise RuntimeError("wxprobe_mfma_rate failed")
        t, _ = event_ms(run, 5, warm=2)
        out[f"mfma_only_{name}_operands_tflops"] = round(flops.value / t / 1e9, 1)
    (g0, u0, d0) = weights[0]
    H, I0 = g0.shape[1], g0.shape[0]
    xv = x[:m0]
    wgu = torch.cat((g0, u0), 0)
    o = torch.empty(m0, 2 * I0, dtype=torch.bfloat16, device=dev)
    t, _ = event_ms(lambda: torch.matmul(xv, wgu.t(), out=o), 10)
    out["hipblaslt_gate_up_shape_tflops"] = round(4.0 * m0 * I0 * H / t / 1e9, 1)
    hm = o[:, :I0].contiguous()
    del o
    o2 = torch.empty(m0, H, dtype=torch.bfloat16, device=dev)
    t, _ = event_ms(lambda: torch.matmul(hm, d0.t(), out=o2), 10)
    out["hipblaslt_down_shape_tflops"] = round(2.0 * m0 * I0 * H / t / 1e9, 1)
    del o2, hm
    # the denoise step of config 4 (2048 action tokens on the 1024-wide expert): gate and up as one 2048 x 2048 x 2048
    # product, down as 2048 x 2048 x 1024, on the action expert's tensors; many launches per event pair, so that
    # launch gaps stay out of a figure of a few tens of microseconds
    (g1, u1, d1) = weights[1]
    I1 = g1.shape[0]
    xa = x[:2048].contiguous()
    wgu1 = torch.cat((g1, u1), 0)
    oa = torch.empty(2048, 2 * I1, dtype=torch.bfloat16, device=dev)
    t, _ = event_ms(lambda: torch.matmul(xa, wgu1.t(), out=oa), 20, batch=20)
    out["hipblaslt_denoise_gate_up_shape_us"] = round(t * 1e3, 2)
    out["hipblaslt_denoise_gate_up_shape_tflops"] = round(4.0 * 2048 * I1 * H / t / 1e9, 1)
    ha = oa[:, :I1].contiguous()
    ob = torch.empty(2048, H, dtype=torch.bfloat16, device=dev)
    t, _ = event_ms(lambda: torch.matmul(ha, d1.t(), out=ob), 20, batch=20)
    out["hipblaslt_denoise_down_shape_us"] = round(t * 1e3, 2)
    out["hipblaslt_denoise_down_shape_tflops"] = round(2.0 * 2048 * I1 * H / t / 1e9, 1)
    out["note"] = ("same GPU, same run; hipBLASLt numbers are plain GEMMs on the benchmark's tensors (no SwiGLU, one "
                   "expert, rows already contiguous): the VL expert's two shapes at config 3 (28160 rows), and the "
                   "action expert's two shapes at config 4's denoise step (2048 rows)")
    return out


def prefill_measurement(dev, mask, native_projections=True):
    """BASELINE config 5: one prefill of 16 x 912 tokens through a randomly initialised 36-layer decoder of the
    Qwen2.5-VL-3B shape with the dual-expert FFN in every layer; attention on PyTorch, the projections on this
    library's GEMM (native_projections) or the vendor's."""
    import torch
    from wallx_mi355 import harness

    model = harness.PrefillHarness(device=dev, mask="causal" if mask == "causal" else "action_block",
                                   fuse_qkv_rope=native_projections, o_proj_native=native_projections)
    ids, grid, types = harness.config5_inputs(16, dev)
    suffix = 32 if mask == "action_block" else None  # config 5: the 32 action tokens close every row
    if suffix is not None and not (bool(types[:, -suffix:].all()) and not bool(types[:, :-suffix].any())):
        raise RuntimeError("config 5 layout changed: the action tokens are not the last 32 of every row")
    for _ in range(2):
        model.forward(ids, grid, types, action_suffix=suffix)
    torch.cuda.synchronize()
    reps = 5
    t0 = time.perf_counter()
    for _ in range(reps):
        model.forward(ids, grid, types, action_suffix=suffix)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / reps
    timer = harness.OpTimer()
    model.forward(ids, grid, types, timer, action_suffix=suffix)
    split = timer.report_ms()
    total = sum(split.values())
    del model
    torch.cuda.empty_cache()
    return {
        "projections": "this library's GEMM: q / k / v with bias and M-RoPE in its epilogue (wx_qkv_rope_proj), o with "
                       "the residual add in its epilogue (wx_dual_gemm_add)" if native_projections
                       else "vendor GEMM (F.linear, addmm); M-RoPE as its own kernel",
        "workload": "config 5 (BASELINE.json configs[4]): 36 layers, hidden 2048, 16 q / 2 kv heads x 128, experts "
                    "11008 / 1024, 16 x 912 tokens (32 action each), bf16, random init, rms eps 1e-6, mask " +
                    {"action_block": "causal + bidirectional action block (act.py:616-637) as two maskless attention calls",
                     "action_block_dense": "causal + bidirectional action block through a dense mask",
                     "causal": "plain causal"}[mask],
        "tokens_per_s": round(ids.numel() / dt, 1),
        "ms_per_forward": round(dt * 1e3, 3),
        "op_split_ms": {k: round(v, 3) for k, v in sorted(split.items(), key=lambda kv: -kv[1])},
        "op_split_total_ms": round(total, 3),
        "ours_ms": round(sum(v for k, v in split.items() if not k.endswith("_torch")), 3),
    }


def physical_cores():
    """Physical cores of the host from /proc/cpuinfo (distinct (physical id, core id) pairs); None if unreadable."""
    try:
        pairs, cur = set(), {}
        with open("/proc/cpuinfo") as f:
            for line in f:
                if ":" in line:
                    key, val = (t.strip() for t in line.split(":", 1))
                    cur[key] = val
                elif cur:
                    pairs.add((cur.get("physical id", "0"), cur.get("core id", cur.get("processor"))))
                    cur = {}
        if cur:
            pairs.add((cur.get("physical id", "0"), cur.get("core id", cur.get("processor"))))
        return len(pairs) or None
    except OSError:
        return None


def cpu_baseline(x_cpu, types_cpu, w_cpu, n_seq, H, I0, I1):
    """The CPU oracle (a restatement of the reference's PyTorch path) on the first n_seq sequences of the same batch,
    fp32 math on the bf16-valued inputs: median of 5 runs after 2 warm-ups on the threads torch uses on this box,
    and the single-thread figure on one sequence for scale."""
    import torch
    import oracle

    weights = [w.as_tuple() for w in w_cpu]
    w32 = [tuple(t.float() for t in w) for w in weights]  # upcast once, outside the timed region

    def timed(n, warm, runs):
        xs, ts = x_cpu[:n].float(), types_cpu[:n]
        m1 = int(ts.sum())
        flops = 6.0 * H * ((ts.numel() - m1) * I0 + m1 * I1)
        for _ in range(warm):
            oracle.sparse_moe_block_ref(xs, ts, w32, eager_rounding=False)
        times = []
        for _ in range(runs):
            t0 = time.perf_counter()
            oracle.sparse_moe_block_ref(xs, ts, w32, eager_rounding=False)
            times.append(time.perf_counter() - t0)
        return flops, statistics.median(times), ts.numel()

    threads = torch.get_num_threads()
    flops, best, tokens = timed(n_seq, 2, 5)
    torch.set_num_threads(1)
    try:
        flops1, best1, tokens1 = timed(1, 1, 3)
    finally:
        torch.set_num_threads(threads)
    return {
        "value": round(flops / best / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": threads,
        "physical_cores_of_host": physical_cores(),
        "logical_cpus_of_host": os.cpu_count(),
        "single_thread_value": round(flops1 / best1 / 1e12, 4),
        "kind": "port",
        "sample": f"first {n_seq} of 32 sequences of the same batch ({tokens} tokens, {flops / 1e12:.3f} TFLOP), "
                  f"fp32 math on bf16-valued inputs, {threads} threads (the CPU share torch is given on this box), "
                  f"median of 5 runs after 2 warm-ups, {best * 1e3:.0f} ms per run; single_thread_value: first "
                  f"sequence ({tokens1} tokens), 1 thread, median of 3 runs after 1 warm-up, {best1 * 1e3:.0f} ms per run",
    }


def cpu_prefill_baseline(n_layers_timed=2):
    """The config 5 prefill on the host cores, for scale next to `extra.prefill`: the CPU oracle's pieces (RMSNorm,
    M-RoPE, the dual-expert block) with torch's CPU linear layers and attention between them, fp32, at the full
    16 x 912 batch.  A bounded sample: ONE decoder layer is timed n_layers_timed times after a warm-up and the forward
    is priced as 36 such layers (embedding lookup and the last-token head are left out, well under 1 %)."""
    import torch
    import torch.nn.functional as F
    import oracle
    from wallx_mi355 import workloads as wl

    g = torch.Generator().manual_seed(0)
    H, nq, nkv, D, inter = wl.HIDDEN, wl.N_Q_HEADS, wl.N_KV_HEADS, wl.HEAD_DIM, (wl.INTER_VL, wl.INTER_ACT)
    ids, grid = wl.config2_tokens(batch=16, tail_text=96)
    types = ids == wl.ACTION_TOKEN_ID
    B, S = ids.shape
    pos, _ = oracle.rope_index_ref(ids, 2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2,
                                   image_grid_thw=grid)
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(D), torch.float32)
    w = lambda *shape: torch.randn(*shape, generator=g) * 0.02  # noqa: E731
    ln = torch.ones(H)
    wqkv, bqkv, wo = w((nq + 2 * nkv) * D, H), w((nq + 2 * nkv) * D), w(H, nq * D)
    experts = [(w(i, H), w(i, H), w(H, i)) for i in inter]
    causal = torch.ones(S, S, dtype=torch.bool).tril()
    mask = causal[None, None] | (types[:, None, :, None] & types[:, None, None, :])  # act.py:616-637
    h = torch.randn(B, S, H, generator=g)

    def layer(h):
        x = oracle.rms_norm_ref(h, ln, 1e-6)
        q, k, v = F.linear(x, wqkv, bqkv).split([nq * D, nkv * D, nkv * D], dim=-1)
        q, k, v = (t.view(B, S, -1, D).transpose(1, 2) for t in (q, k, v))
        q, k = oracle.mrope_apply_ref(q, k, cos, sin, list(wl.MROPE_SECTION))
        rep = nq // nkv
        a = F.scaled_dot_product_attention(q, k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1), attn_mask=mask)
        h = h + F.linear(a.transpose(1, 2).reshape(B, S, nq * D), wo)
        return h + oracle.sparse_moe_block_ref(oracle.rms_norm_ref(h, ln, 1e-6), types, experts, eager_rounding=False)

    with torch.no_grad():
        layer(h)
        times = []
        for _ in range(n_layers_timed):
            t0 = time.perf_counter()
            layer(h)
            times.append(time.perf_counter() - t0)
    per_layer = statistics.median(times)
    return {"tokens_per_s": round(B * S / (36 * per_layer), 1), "cores": torch.get_num_threads(),
            "sample": f"one decoder layer at the full 16 x 912 batch (fp32, dense boolean attention mask), median of "
                      f"{n_layers_timed} runs after a warm-up: {per_layer * 1e3:.0f} ms; the forward priced as 36 layers"}


if __name__ == "__main__":
    main()
