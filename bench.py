#!/usr/bin/env python3
"""Benchmark of the equivariant message-passing hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

Prints ONE JSON line.  The default workload is BASELINE.json configs[2]: one
PaiNN message-passing layer (Message + Update, n = 128, 16 radial functions) on
16 polymer chains x 1024 beads in a periodic 80 A box with an 8 A cutoff; the
metric is directed edges per second per layer.  A step is one forward pass of
the layer with all inputs (positions, features, weights, edge list) resident in
HBM.  Other workloads (reported under "other_workloads" and selectable with
--workload): configs[1] neighbour search, configs[0] tensor-product trio.

roofline: the kernel that dominates the step, timed on its own with HIP events
on the launch stream: algorithmic FLOPs (or bytes) per launch / mean launch time.
cpu_baseline: the CPU oracle (a port of the reference's math, not the
reference's code) on a bounded sample of the same workload on the host cores.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
PEAK_FP32_MFMA_TFLOPS = 157.3  # MI355X dense fp32 matrix
PEAK_BF16_MFMA_TFLOPS = 2500.0  # MI355X dense bf16 matrix


def measured_traffic(kernel, summary="painn_layer_configs2_traffic.json"):
    """HBM bytes per launch of a kernel from a committed rocprofv3 --pmc summary under profiles/ (None if absent)."""
    path = os.path.join(ROOT, "profiles", summary)
    try:
        with open(path) as f:
            return json.load(f).get(kernel, {}).get("traffic_bytes")
    except (OSError, ValueError):
        return None


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="painn_layer",
                    choices=["painn_layer", "neighbour", "products", "denoiser", "stress", "polymer", "meanflow_painn",
                             "gemm_power", "painn_train", "denoiser_train", "meanflow_train"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip the other workloads")
    ap.add_argument("--no-comparisons", action="store_true",
                    help="painn_layer: skip the stand-alone timings of the kernels the layer no longer runs; "
                         "stress: skip the timing of the fp32-storage stack")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (yardstick for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    return ap.parse_args()


def event_time(torch, fn, iters, warmup=2):
    """Mean seconds per call, HIP events on the current (launch) stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / iters


def timed_steps(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


# ------------------------------------------------------------------ inputs
def polymer_positions(torch, chains, beads, box, seed):
    g = torch.Generator().manual_seed(seed)
    steps = torch.randn(chains, beads, 3, generator=g)
    steps = 3.8 * steps / steps.norm(dim=-1, keepdim=True)
    origin = torch.rand(chains, 1, 3, generator=g) * box
    return (steps.cumsum(1) + origin).reshape(1, chains * beads, 3).contiguous()


def mlp_weights(mlp):
    L = mlp.layers
    return {"W1": L[0].weight.detach().cpu(), "b1": L[0].bias.detach().cpu(),
            "W2": L[2].weight.detach().cpu(), "b2": L[2].bias.detach().cpu(),
            "W3": L[4].weight.detach().cpu(), "b3": L[4].bias.detach().cpu()}


# --------------------------------------------------------------- workloads
def bench_painn_layer(torch, args):
    ops = importlib.import_module("learned-dynamics_amd.ops")
    painn = importlib.import_module("learned-dynamics_amd.painn")
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    n, n_rbf, r0, box_len = 128, 16, 8.0, 80.0
    box = (box_len,) * 3
    seed = 0x947 + 3
    torch.manual_seed(seed)
    pos = polymer_positions(torch, 16, 1024, box_len, seed)
    block = painn.Block(r0, n, n_rbf=n_rbf).cuda().eval()
    g = torch.Generator().manual_seed(seed + 1)
    x_a = torch.randn(1, 16384, n, generator=g)
    x_v = torch.randn(1, 16384, n, 3, generator=g) / 3 ** 0.5
    pos_d, x_a_d, x_v_d = pos.cuda(), x_a.cuda(), x_v.cuda()

    with torch.no_grad():
        graph, r_ij = gl.graph_setup(r0, box, pos_d, neighbours_max=512, celllist_max=128)
        E, N = int(graph.src.numel()), 16384

        def step():
            return block((pos_d, graph, r_ij, None, None, x_a_d, x_v_d, box))

        sec = timed_steps(torch, step, args.steps, args.warmup)

        actv = block.message.mlp_actv(x_a_d.reshape(N, n))
        xv_flat, xa_flat = x_v_d.reshape(N, n, 3), x_a_d.reshape(N, n)
        t_graph = event_time(torch, lambda: gl.graph_setup(r0, box, pos_d, neighbours_max=512, celllist_max=128), 5)
        breakdown = {"graph_build_ms_not_in_step": t_graph * 1e3}
        # the same step recorded into a HIP graph and replayed (every launch of the layer, nothing cached between replays)
        ro = importlib.import_module("learned-dynamics_amd.rollout")
        graphed = ro.GraphedCall(lambda xa, xv: block((pos_d, graph, r_ij, None, None, xa, xv, box))[5:7], x_a_d, x_v_d)
        breakdown["layer_ms_replayed_from_a_hip_graph"] = event_time(torch, graphed.graph.replay, 20) * 1e3
        roofline, roofline_hbm = None, None
        comparisons = not getattr(args, "no_comparisons", False)
        if comparisons:
            # the kernels of the path with the filter MLP evaluated on every edge, timed alone for comparison
            # --- dominant kernel: the 4n x 4n filter GEMM over E rows (fp32 MFMA)
            h = torch.randn(E, 4 * n, device="cuda")
            lin = block.message.mlp_dist.layers[2]
            out = torch.empty(E, 4 * n, device="cuda")
            mode = ops.get_linear_mode()
            if mode == ops.LINEAR_F16X2:
                # as the layer runs it: row bounds carried over from the previous layer's weight norms
                bound = ops.linear_out_bound(block.message.mlp_dist.layers[0].weight, block.message.mlp_dist.layers[0].bias,
                                             None)
                t_gemm = event_time(torch, lambda: ops.tensor_linear_f16x2(lin.weight, h, bound, bias=lin.bias,
                                                                           act=ops.ACT_SILU, out=out), 10)
            else:
                t_gemm = event_time(torch, lambda: ops.tensor_linear_fwd(0, lin.weight, h, bias=lin.bias, act=ops.ACT_SILU,
                                                                         out=out), 10)
            flops = 2.0 * E * (4 * n) * (4 * n)
            split = mode == ops.LINEAR_BF16X3
            if mode == ops.LINEAR_F16X2:
                # operands split into 2 fp16 pieces, 3 fp16 MFMAs per fp32 product, fp32 accumulate
                roofline = {"kernel": "linear_rows_f16x2_kernel<8 waves, 256 columns> (filter MLP layer, E x 512 x 512, bias+SiLU fused)",
                            "bound": "mfma", "achieved": 3 * flops / t_gemm / 1e12, "peak": PEAK_BF16_MFMA_TFLOPS,
                            "unit": "TFLOP/s", "frac": 3 * flops / t_gemm / 1e12 / PEAK_BF16_MFMA_TFLOPS,
                            "traffic": measured_traffic("linear_rows_f16x2_kernel"),
                            "note": "achieved counts the executed fp16 MFMA FLOPs (3 per fp32 multiply-add pair) against "
                                    "the fp16 dense peak; fp32-equivalent rate and its ratio to the fp32 MFMA peak alongside",
                            "fp32_equivalent_tflops": flops / t_gemm / 1e12,
                            "fp32_equivalent_over_fp32_mfma_peak": flops / t_gemm / 1e12 / PEAK_FP32_MFMA_TFLOPS}
            elif split:
                # operands split into 3 bf16 pieces, 6 bf16 MFMAs per fp32 product, fp32 accumulate
                roofline = {"kernel": "linear_rows_bf16x3_wide_kernel (filter MLP layer, E x 512 x 512, bias+SiLU fused)",
                            "bound": "mfma", "achieved": 6 * flops / t_gemm / 1e12, "peak": PEAK_BF16_MFMA_TFLOPS,
                            "unit": "TFLOP/s", "frac": 6 * flops / t_gemm / 1e12 / PEAK_BF16_MFMA_TFLOPS,
                            "traffic": measured_traffic("linear_rows_bf16x3_wide_kernel"),
                            "note": "achieved counts the executed bf16 MFMA FLOPs (6 per fp32 multiply-add pair); "
                                    "fp32-equivalent rate and its ratio to the fp32 MFMA peak are given alongside",
                            "fp32_equivalent_tflops": flops / t_gemm / 1e12,
                            "fp32_equivalent_over_fp32_mfma_peak": flops / t_gemm / 1e12 / PEAK_FP32_MFMA_TFLOPS}
            else:
                roofline = {"kernel": "linear_rows_kernel (fp32 MFMA, filter MLP layer, E x 512 x 512, bias+SiLU fused)",
                            "bound": "mfma", "achieved": flops / t_gemm / 1e12, "peak": PEAK_FP32_MFMA_TFLOPS,
                            "unit": "TFLOP/s", "frac": flops / t_gemm / 1e12 / PEAK_FP32_MFMA_TFLOPS, "traffic": None}
            del h, out

            # --- HBM-bound edge kernel: fused gather-product-scatter
            filt = block.message.filters(r_ij)
            t_edge = event_time(torch, lambda: ops.painn_message(graph.row_ptr, graph.dst32, r_ij, filt, actv, xv_flat,
                                                                 0.1, xa_flat, xv_flat, node_order=graph.cell_order), 20)
            t_edge_index_order = event_time(torch, lambda: ops.painn_message(graph.row_ptr, graph.dst32, r_ij, filt, actv,
                                                                             xv_flat, 0.1, xa_flat, xv_flat), 20)
            edge_bytes = E * (16 * n + 4 + 12) + N * (16 * n + 16 * n)
            roofline_hbm = {"kernel": "painn_message_kernel (fused gather-product-scatter)", "bound": "hbm",
                            "achieved": edge_bytes / t_edge / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                            "frac": edge_bytes / t_edge / 1e9 / PEAK_HBM_GBS,
                            "traffic": measured_traffic("painn_message_kernel"),
                            "bytes_per_launch": edge_bytes, "ms": t_edge * 1e3,
                            "ms_rows_in_index_order": t_edge_index_order * 1e3}
            breakdown.update({"filter_gemm_512x512_ms": t_gemm * 1e3, "edge_kernel_ms": t_edge * 1e3})
            del filt
            if ops.painn_filter_message_supported(n, 4 * n, E):
                # as the layer runs it: the filter MLP's last layer inside the edge kernel (the largest kernel of
                # the step); the stand-alone GEMM above is the MLP's middle layer, the second largest
                msg = block.message
                first, second = msg.mlp_dist.layers[0], msg.mlp_dist.layers[2]
                b1 = ops.linear_out_bound(first.weight, first.bias, None)
                if ops.painn_filter_hidden_supported(n_rbf, 4 * n, E):
                    # encoding + first + second layer of the filter MLP in one kernel (the second largest kernel)
                    hidden_fn = lambda: ops.painn_filter_hidden(r_ij, r0, first.weight, first.bias, second.weight,
                                                                second.bias, b1)
                    t_hidden = event_time(torch, hidden_fn, 10)
                    h2, b2 = hidden_fn(), ops.linear_out_bound(second.weight, second.bias, b1)
                    breakdown["filter_encode_plus_two_layers_ms"] = t_hidden * 1e3
                    hidden_flops = 3 * (flops + 2.0 * E * 16 * 4 * n)
                    roofline = {"kernel": "painn_filter_hidden_kernel (radial encoding, E x 16 x 512 and E x 512 x 512 "
                                          "split-fp16 GEMMs, bias + SiLU; the first layer's output stays in registers)",
                                "bound": "mfma", "achieved": hidden_flops / t_hidden / 1e12, "peak": PEAK_BF16_MFMA_TFLOPS,
                                "unit": "TFLOP/s", "frac": hidden_flops / t_hidden / 1e12 / PEAK_BF16_MFMA_TFLOPS,
                                "traffic": measured_traffic("painn_filter_hidden_kernel"),
                                "fp32_equivalent_tflops": hidden_flops / 3 / t_hidden / 1e12,
                                "stand_alone_gemm_for_comparison": roofline}
                else:
                    h1, _ = msg._hidden(r_ij)
                    h2, b2 = painn._linear(h1, second, ops.ACT_SILU, b1)
                    del h1
                W3, b3 = msg._permuted_last()
                t_fused = event_time(torch, lambda: ops.painn_filter_message(
                    W3, b3, h2, b2, graph.row_ptr, graph.src32, graph.dst32, r_ij, actv, xv_flat, 0.1, xa_flat, xv_flat), 10)
                del h2
                breakdown["filter_last_layer_plus_edge_kernel_ms"] = t_fused * 1e3
                roofline_gemm = roofline
                roofline = {"kernel": "painn_filter_message_kernel (E x 512 x 512 split-fp16 GEMM whose epilogue gathers, "
                                      "multiplies and row-sums the messages) + painn_message_finish_kernel (about 1 % of the time)",
                            "bound": "mfma", "achieved": 3 * flops / t_fused / 1e12, "peak": PEAK_BF16_MFMA_TFLOPS,
                            "unit": "TFLOP/s", "frac": 3 * flops / t_fused / 1e12 / PEAK_BF16_MFMA_TFLOPS,
                            "traffic": measured_traffic("painn_filter_message_kernel"),
                            "note": "achieved counts the executed fp16 MFMA FLOPs of the GEMM part (3 per fp32 multiply-add "
                                    "pair) against the fp16 dense peak; the message arithmetic and gathers in the epilogue "
                                    "count as overhead",
                            "fp32_equivalent_tflops": flops / t_fused / 1e12,
                            "second_kernel": roofline_gemm}
                roofline_hbm["note"] = ("the stand-alone edge kernel (filter read from memory); this workload runs the fused "
                                        "kernel above instead, the stand-alone one serves channel counts that are not a "
                                        "multiple of 64 and the other GEMM modes")
        msg = block.message
        rows = msg.table_rows() if msg.use_table else 0
        if rows and E >= 4 * rows:
            # as the layer runs it now: the filter interpolated from a grid over the edge length inside the edge
            # kernel; the two GEMM kernels above are the path taken when the grid is rejected for a set of weights
            table = msg.filter_table(rows)
            t_build = event_time(torch, lambda: msg.filter_table(rows), 20)
            sliced = msg.use_sliced and rows <= ops.PAINN_SLICED_MAX_ROWS and n % ops.PAINN_SLICE == 0
            if sliced:
                actv_s = actv[:, ops.painn_slice_permutation(n, "cuda")].contiguous()
                # the kernel alone, called as the layer calls it: rows in cell order, the per-edge records (grid row,
                # interpolation weights, direction: 32 bytes per edge) written by their own small kernel
                rec = ops.painn_edge_records(r_ij, rows, 2 * r0, 0.1)
                t_rec = event_time(torch, lambda: ops.painn_edge_records(r_ij, rows, 2 * r0, 0.1), 20)
                t_table = event_time(torch, lambda: ops.painn_table_message_sliced(
                    graph.row_ptr, graph.dst32, r_ij, table, 2 * r0, actv_s, xv_flat, 0.1, xa_flat, xv_flat,
                    node_order=graph.cell_order, records=rec), 20)
                breakdown["edge_records_ms"] = t_rec * 1e3
                if comparisons:
                    msg.use_sliced = False
                    sec_cached_grid = timed_steps(torch, step, max(3, args.steps // 4), 2)
                    msg.use_sliced = True
                    breakdown["layer_ms_with_the_grid_read_through_the_caches"] = sec_cached_grid * 1e3
            else:
                t_table = event_time(torch, lambda: ops.painn_table_message(
                    graph.row_ptr, graph.dst32, r_ij, table, 2 * r0, actv, xv_flat, 0.1, xa_flat, xv_flat), 20)
            if comparisons:
                msg.use_table = False
                sec_exact = timed_steps(torch, step, max(3, args.steps // 4), 2)
                breakdown["layer_ms_with_filter_mlp_per_edge"] = sec_exact * 1e3
                # and with every linear of the layer in true fp32 matrix arithmetic (v_mfma_f32_32x32x2_f32)
                prev_mode = ops.get_linear_mode()
                ops.set_linear_mode(ops.LINEAR_FP32_MFMA)
                try:
                    sec_fp32 = timed_steps(torch, step, 3, 1)
                finally:
                    ops.set_linear_mode(prev_mode)
                breakdown["layer_ms_with_filter_mlp_per_edge_fp32_mfma"] = sec_fp32 * 1e3
                msg.use_table = True
            hbm_bytes = E * (36 if sliced else 16) + N * (16 * n + 12 * n) + 2 * N * 16 * n + rows * 16 * n
            gather_bytes = E * (16 * n + 12 * n + 16)
            grid_bytes = E * 4 * 16 * n
            cache_bytes = gather_bytes + (0 if sliced else grid_bytes)
            l1_fill_peak = 256 * 64 * 2.4                     # GB/s: 256 CUs x 64 B per clock x 2.4 GHz
            flop = E * n * (4 * 4 * 2 + 4 + 9 + 18 + 1)       # interpolation, products, cross product, accumulation
            breakdown["filter_grid_evaluation_ms"] = t_build * 1e3
            breakdown["table_edge_kernel_ms"] = t_table * 1e3
            kernel = ("painn_table_message_lds_kernel (a workgroup keeps 16 channels of the %d-row filter grid in LDS; per "
                      "edge: 4 grid rows interpolated, node rows gathered, products, sums over the edges of a node)" % rows
                      if sliced else
                      "painn_message_kernel<table> (per edge: 4 rows of the %d-row filter grid interpolated, node rows "
                      "gathered, products, sums over the edges of a node)" % rows)
            roofline = {"kernel": kernel, "bound": "fp32_vector", "achieved": flop / t_table / 1e12,
                        "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": flop / t_table / 1e12 / PEAK_FP32_MFMA_TFLOPS,
                        "traffic": measured_traffic("painn_table_message_lds_kernel" if sliced else "painn_message_kernel<true>"),
                        "flop_per_launch": flop, "ms": t_table * 1e3,
                        "peak_note": "157.3 TFLOP/s is the published fp32 vector peak and needs packed fp32 instructions, "
                                     "which are compiled out here; 78.65 TFLOP/s is reachable without them",
                        "hbm": {"bytes_per_launch": hbm_bytes, "achieved": hbm_bytes / t_table / 1e9, "peak": PEAK_HBM_GBS,
                                "unit": "GB/s", "frac": hbm_bytes / t_table / 1e9 / PEAK_HBM_GBS},
                        "cache_to_cu": {"bytes_per_launch": cache_bytes, "achieved": cache_bytes / t_table / 1e9,
                                        "peak": l1_fill_peak, "unit": "GB/s",
                                        "frac": cache_bytes / t_table / 1e9 / l1_fill_peak},
                        "lds_reads": {"bytes_per_launch": grid_bytes if sliced else 0,
                                      "achieved": (grid_bytes if sliced else 0) / t_table / 1e9, "unit": "GB/s"},
                        "note": "every operand of the kernel is cache resident (node-sized arrays and the filter grid): "
                                "the kernel is bound by vector arithmetic and by the gathers of node rows from L2 "
                                "(cache_to_cu, against 64 B per clock per CU), not by HBM (hbm)",
                        "filter_mlp_per_edge_path": roofline}
            # The three ways the layer can run, side by side.  The filter MLP's FLOPs (2 E (16 x 512 + 2 x 512^2)) are
            # only executed when the MLP runs on every edge; with the grid they are replaced by 512 rows of the same MLP.
            mlp_flops = 2.0 * E * (n_rbf * 4 * n + 2 * (4 * n) * (4 * n))
            kept = None
            if comparisons:
                msg.keep_table = True
                try:
                    sec_kept = timed_steps(torch, step, args.steps, 2)
                finally:
                    msg.keep_table = False
                kept = {"value": E / sec_kept, "unit": "edges/s", "ms_per_step": sec_kept * 1e3,
                        "note": "Message.keep_table: the filter grid, a function of the weights alone, kept from one "
                                "forward to the next instead of being evaluated in each (not what `value` measures)"}
            variants = {"filter_grid": {"value": E / sec, "unit": "edges/s", "ms_per_step": sec * 1e3,
                                        "dominant_kernel": "painn_table_message_lds_kernel" if sliced else "painn_message_kernel<true>",
                                        "bound": "fp32_vector", "frac": roofline["frac"], "traffic": roofline["traffic"],
                                        "grid_rows": rows}}
            if comparisons:
                per_edge = breakdown["layer_ms_with_filter_mlp_per_edge"] * 1e-3
                fused = roofline["filter_mlp_per_edge_path"]
                variants["filter_mlp_per_edge"] = {
                    "value": E / per_edge, "unit": "edges/s", "ms_per_step": per_edge * 1e3,
                    "dominant_kernel": "painn_filter_message_kernel + painn_filter_hidden_kernel",
                    "bound": "mfma", "peak": PEAK_BF16_MFMA_TFLOPS, "unit_roofline": "TFLOP/s",
                    # executed fp16 matrix work of the whole layer step (3 per fp32 multiply-add) against the fp16 peak
                    "achieved": 3 * mlp_flops / per_edge / 1e12, "frac": 3 * mlp_flops / per_edge / 1e12 / PEAK_BF16_MFMA_TFLOPS,
                    "fp32_equivalent_tflops": mlp_flops / per_edge / 1e12,
                    "fp32_equivalent_over_fp32_mfma_peak": mlp_flops / per_edge / 1e12 / PEAK_FP32_MFMA_TFLOPS,
                    "kernel_frac": None if fused is None else fused.get("frac"),
                    "traffic": None if fused is None else fused.get("traffic"),
                    "note": "the path every set of weights takes whose grid is refused, and every forward whose "
                            "positions are differentiated"}
                fp32 = breakdown["layer_ms_with_filter_mlp_per_edge_fp32_mfma"] * 1e-3
                variants["filter_mlp_per_edge_fp32_mfma"] = {
                    "value": E / fp32, "unit": "edges/s", "ms_per_step": fp32 * 1e3,
                    "dominant_kernel": "linear_rows_kernel (v_mfma_f32_32x32x2_f32) + painn_message_kernel",
                    "bound": "mfma", "peak": PEAK_FP32_MFMA_TFLOPS, "unit_roofline": "TFLOP/s",
                    "achieved": mlp_flops / fp32 / 1e12, "frac": mlp_flops / fp32 / 1e12 / PEAK_FP32_MFMA_TFLOPS,
                    "traffic": None,
                    "note": "mg_set_linear_mode(0): 24-bit significand products on the fp32 matrix cores in every linear "
                            "of the layer; the price of strict fp32 arithmetic (the filter is stored, E x 4n floats)"}
            if kept is not None:
                variants["filter_grid_kept_between_forwards"] = kept
            roofline["layer_variants"] = variants
        del actv

    cpu = None
    if not args.no_cpu:
        cpu = cpu_painn_layer(torch, block, n, n_rbf, r0, box_len, seed)
    per_edge_ms = breakdown.get("layer_ms_with_filter_mlp_per_edge")
    result = {
        "metric": "message-passing edges/sec per layer", "value": E / sec, "unit": "edges/s",
        "ms_per_step": sec * 1e3,
        "dtype": "f32 storage and accumulation; products of the wide linears as split-fp16 MFMA (2 x 11 significand bits)",
        "value_note": "the filter MLP of the layer is evaluated on a 512-point grid over the edge length and "
                      "interpolated per edge (a grid is accepted per set of weights when its interpolation error, "
                      "measured in float64, is below 1e-7 + 1e-6 |filter| for every filter element); "
                      "roofline.layer_variants holds the same layer with the MLP evaluated on every edge, in "
                      "split-fp16 and in true fp32 matrix arithmetic",
        "value_filter_mlp_per_edge": None if per_edge_ms is None else E / (per_edge_ms * 1e-3),
        "ms_per_step_filter_mlp_per_edge": per_edge_ms,
        "config": {"workload": "BASELINE configs[2]: one PaiNN layer (Message + Update, residuals), 16 chains x 1024 "
                               "beads, box 80 A, cutoff 8 A, n=128 scalar+128 vector channels, 16 radial functions",
                   "edges": E, "atoms": N, "graph": "prebuilt (positions fixed); build time reported in breakdown"},
        "roofline": roofline, "roofline_hbm": roofline_hbm, "breakdown": breakdown, "cpu_baseline": cpu,
    }
    return result


def cpu_painn_layer(torch, block, n, n_rbf, r0, box_len, seed):
    """Oracle (port of the reference math) on 2 of the 16 chains, host cores."""
    from oracle import layers as OL
    from oracle import neighbour as ON
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    box = (box_len,) * 3
    pos = polymer_positions(torch, 2, 1024, box_len, seed)
    Nc = pos.shape[1]
    g = torch.Generator().manual_seed(seed + 2)
    x_a = torch.randn(1, Nc, n, generator=g)
    x_v = torch.randn(1, Nc, n, 3, generator=g) / 3 ** 0.5
    ref = ON.edges(pos.numpy(), r0, box)
    src, dst = torch.from_numpy(ref["src"]).long(), torch.from_numpy(ref["dst"]).long()
    r_ij = torch.from_numpy(ON.edge_vectors(pos.numpy(), ref["src"], ref["dst"], box))
    w_dist, w_actv = mlp_weights(block.message.mlp_dist), mlp_weights(block.message.mlp_actv)
    w_upd = {"W_l": block.update.lin_l.W.detach().cpu(), "W_r": block.update.lin_r.W.detach().cpu(),
             "W_v": block.update.lin_v.W.detach().cpu(), "mlp": mlp_weights(block.update.mlp),
             "gn_gamma": block.update.gn.gamma.detach().cpu(), "gn_beta": block.update.gn.beta.detach().cpu()}

    def layer():
        da, dv = OL.painn_message(src, dst, 1, Nc, x_a, x_v, r_ij, w_dist, w_actv, r0, n, n_rbf)
        xa, xv = x_a + da, x_v + dv
        ua, uv = OL.painn_update(xa, xv, w_upd, n)
        return xa + ua, xv + uv

    with torch.no_grad():
        layer()
        times = []
        t_all = time.perf_counter()
        while len(times) < 3 or (time.perf_counter() - t_all < 10 and len(times) < 20):
            t0 = time.perf_counter()
            layer()
            times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": len(src) / med, "unit": "edges/s", "cores": cores, "kind": "port",
            "sample": f"2 of the 16 chains ({Nc} atoms, {len(src)} edges), same layer and weights, "
                      f"median of {len(times)} runs, PyTorch CPU fp32"}


def bench_neighbour(torch, args, with_cpu=True):
    ops = importlib.import_module("learned-dynamics_amd.ops")
    g = torch.Generator().manual_seed(0x947 + 2)
    pos = (torch.rand(8, 16384, 3, generator=g) * 55).contiguous()
    pos_d = pos.cuda()
    box = (55., 55., 55.)

    def step():
        search = ops.NeighbourSearch(pos_d, 5.0, box)
        return search.fill()     # includes the device->host copy of E, as get_edges does

    src, _ = step()
    E = int(src.numel())
    sec = timed_steps(torch, step, args.steps, args.warmup)
    alg_bytes = 12 * 8 * 16384 + 8 * E + 4 * 8
    search = ops.NeighbourSearch(pos_d, 5.0, box)
    t_fill = event_time(torch, lambda: search.fill(E), 10)
    t_count = event_time(torch, lambda: ops.NeighbourSearch(pos_d, 5.0, box), 10)
    # the same search into caller-sized arrays, edge count left on the device: no host synchronisation, so it can be
    # recorded into a HIP graph together with the layers that use the edges
    capacity = (E + 4095) // 4096 * 4096
    bufs = ops.neighbour_edges(pos_d, 5.0, box, capacity)
    t_capacity = event_time(torch, lambda: ops.neighbour_edges(pos_d, 5.0, box, capacity, out=bufs), 20)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.neighbour_edges(pos_d, 5.0, box, capacity, out=bufs)
    t_replay = event_time(torch, graph.replay, 20)
    if int(bufs["stats"][0]) != E or not torch.equal(bufs["src"][:E], src):
        raise RuntimeError("capacity-mode search disagrees with the exact-size search")
    out = {"metric": "neighbour search edges/sec", "value": E / sec, "unit": "edges/s", "ms_per_step": sec * 1e3,
           "dtype": "f32+int32",
           "config": {"workload": "BASELINE configs[1]: 8 boxes x 16384 atoms, box 55 A, cutoff 5 A", "edges": E},
           "roofline": {"kernel": "whole search (bin, sort, count, scan_sums, scan_apply, fill)",
                        "bound": "hbm", "achieved": alg_bytes / sec / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                        "frac": alg_bytes / sec / 1e9 / PEAK_HBM_GBS,
                        "traffic": measured_traffic("whole_search", "neighbour_search_configs1_traffic.json")},
           "breakdown": {"count_phase_ms": t_count * 1e3, "fill_phase_ms": t_fill * 1e3,
                         "capacity_mode_ms": t_capacity * 1e3, "capacity_mode_replayed_ms": t_replay * 1e3,
                         "note": "ms_per_step is the exact-size search (edge count read back by the host between "
                                 "the count and fill phases); the capacity-mode figures include the cell-order "
                                 "kernel (7 launches) and no host synchronisation"}}
    if with_cpu:
        from oracle import neighbour as ON
        one = pos[:1].numpy()
        t0 = time.perf_counter()
        ref = ON.edges(one, 5.0, box)
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": len(ref["src"]) / dt, "unit": "edges/s", "cores": 1, "kind": "port",
                               "sample": "1 of the 8 boxes, C cell list (oracle/neighbour_oracle.c), count+fill passes"}
    return out


def _board_sample():
    """(socket power in W, shader clock in MHz) as amd-smi / rocm-smi report them right now; None where unavailable."""
    import subprocess
    power = clock = None
    try:
        out = subprocess.run(["amd-smi", "metric", "-p", "--json"], capture_output=True, text=True, timeout=10).stdout
        data = json.loads(out)
        gpu = (data.get("gpu_data") or data)[0] if isinstance(data, dict) else data[0]
        power = float(gpu["power"]["socket_power"]["value"])
    except Exception:
        pass
    try:
        out = subprocess.run(["rocm-smi", "--showclocks", "--json"], capture_output=True, text=True, timeout=10).stdout
        card = next(iter(json.loads(out).values()))
        text = next(v for k, v in card.items() if k.startswith("sclk clock speed"))
        clock = float("".join(ch for ch in text if ch.isdigit() or ch == "."))
    except Exception:
        pass
    return power, clock


def bench_gemm_power(torch, args):
    """The split-fp16 row GEMM at E x 512 x 512 on random and on all-zero operands, with the board's socket power and
    shader clock sampled while it runs: what limits the kernel is the 1400 W socket power, which the chip holds by
    lowering its clock."""
    import statistics
    import threading
    ops = importlib.import_module("learned-dynamics_amd.ops")
    E, K, N = 1046456, 512, 512
    g = torch.Generator(device="cuda").manual_seed(0x947 + 9)
    W = torch.randn(N, K, device="cuda", generator=g) * K ** -0.5
    b = torch.randn(N, device="cuda", generator=g)
    y = torch.empty(E, N, device="cuda")
    out = {}
    for name in ("random", "zeros"):
        x = torch.randn(E, K, device="cuda", generator=g) if name == "random" else torch.zeros(E, K, device="cuda")
        xm = ops.row_absmax(x).reshape(E, 1) if name == "random" else torch.ones(E, 1, device="cuda")
        call = lambda: ops.tensor_linear_f16x2(W, x, xm, bias=b, act=ops.ACT_NONE, out=y)
        samples, stop = [], threading.Event()

        def sampler():
            while not stop.is_set():
                samples.append(_board_sample())
                time.sleep(0.1)

        th = threading.Thread(target=sampler, daemon=True)
        for _ in range(20):
            call()
        torch.cuda.synchronize()
        th.start()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n, t0 = 0, time.perf_counter()
        try:
            s.record()
            while time.perf_counter() - t0 < 5.0:
                for _ in range(50):
                    call()
                n += 50
                torch.cuda.synchronize()
            e.record()
            torch.cuda.synchronize()
        finally:
            stop.set()
            th.join()
        ms = s.elapsed_time(e) / n
        steady = samples[len(samples) // 3:]               # the first samples see the ramp
        pw = [p for p, _ in steady if p is not None]
        ck = [c for _, c in steady if c is not None]
        out[name] = {"ms": ms, "executed_TFLOP/s": 3 * 2 * E * K * N / ms / 1e9, "logical_TFLOP/s": 2 * E * K * N / ms / 1e9,
                     "socket_power_W_median": statistics.median(pw) if pw else None,
                     "socket_power_W_max": max(pw) if pw else None,
                     "shader_clock_MHz_median": statistics.median(ck) if ck else None, "samples": len(steady)}
        del x, xm
    r = out["random"]
    return {"metric": "split-fp16 row GEMM, E x 512 x 512, executed fp16 matrix FLOP/s", "unit": "TFLOP/s",
            "value": r["executed_TFLOP/s"], "ms_per_step": r["ms"], "dtype": "f32 storage/accumulate, split-fp16 MFMA products",
            "config": {"workload": "E = 1046456 rows, K = 512, N = 512, bias, no activation; 5 s of back-to-back calls per case"},
            "detail": out,
            "note": "socket power from `amd-smi metric -p`, shader clock from `rocm-smi --showclocks`, sampled every 0.1 s "
                    "by a thread of this process while the GPU runs the loop; the published board power of MI355X is 1400 W"}


def bench_painn_train(torch, args):
    """Forward + backward of one PaiNN block (Message + Update) at BASELINE configs[2] through the differentiable path
    (every adjoint a kernel of this library: tensor_linear input / weight gradients, gather / segment-sum adjoints,
    the filter's grid interpolation and the message's elementwise middle with their adjoints); gradients for all
    parameters and both inputs."""
    painn = importlib.import_module("learned-dynamics_amd.painn")
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    n, n_rbf, r0, box_len = 128, 16, 8.0, 80.0
    box = (box_len,) * 3
    seed = 0x947 + 3
    torch.manual_seed(seed)
    pos_d = polymer_positions(torch, 16, 1024, box_len, seed).cuda()
    block = painn.Block(r0, n, n_rbf=n_rbf).cuda().train()
    g = torch.Generator().manual_seed(seed + 1)
    x_a = torch.randn(1, 16384, n, generator=g).cuda().requires_grad_(True)
    x_v = (torch.randn(1, 16384, n, 3, generator=g) / 3 ** 0.5).cuda().requires_grad_(True)
    with torch.no_grad():
        graph, r_ij = gl.graph_setup(r0, box, pos_d, neighbours_max=512, celllist_max=128)
    E = int(graph.src.numel())
    params = [p for p in block.parameters() if p.requires_grad]

    def step():
        out = block((pos_d, graph, r_ij, None, None, x_a, x_v, box))
        loss = out[5].square().mean() + out[6].square().mean()
        grads = torch.autograd.grad(loss, [x_a, x_v] + params, allow_unused=True)
        return loss, grads

    loss, grads = step()
    finite = all(bool(torch.isfinite(gr).all()) for gr in grads if gr is not None)
    sec = timed_steps(torch, step, args.steps, args.warmup)
    with torch.no_grad():
        t_fwd = event_time(torch, lambda: block((pos_d, graph, r_ij, None, None, x_a, x_v, box)), 10)
    return {"metric": "PaiNN block training step (forward + backward) edges/sec", "unit": "edges/s", "value": E / sec,
            "ms_per_step": sec * 1e3, "dtype": "f32",
            "config": {"workload": "BASELINE configs[2]: 16384 atoms, n = 128, 16 radial functions; gradients for the "
                                   "parameters, x_a and x_v", "edges": E},
            "detail": {"loss": float(loss.detach()), "gradients_finite": finite,
                       "parameters_with_gradient": sum(gr is not None for gr in grads[2:]),
                       "inference_forward_ms_same_inputs": t_fwd * 1e3},
            "note": "the differentiable path: the filter through its 512-row grid (the MLP is differentiated on the grid's "
                    "rows, each edge interpolates; per-edge evaluation when the grid test rejects the weights); the "
                    "message's forward pass is the inference kernel, its backward pass one kernel that interpolates the "
                    "filter again and sums the gradients of the node operands per destination, plus the scatter into "
                    "the grid; split-fp16 GEMMs and weight gradients for the node-sized MLPs"}


def bench_denoiser_train(torch, args):
    """Forward + backward of a 2-block rank-0/1/2 denoiser (Messages + SelfTensProds per block) on 4 systems of 2048
    atoms through the differentiable path: gradients for every parameter and for the noised positions."""
    den = importlib.import_module("learned-dynamics_amd.denoiser")
    seed = 0x947 + 4
    torch.manual_seed(seed)
    B, N, box_len, r0 = 4, 2048, 70.0, 6.0
    dims = dict(dim_a=256, dim_v=64, dim_d=16, chan=256, blocks=2)
    box = (box_len,) * 3
    x1 = chain_positions(torch, B, N, box_len, seed)
    g = torch.Generator().manual_seed(seed + 1)
    x0 = (x1 + torch.randn(B, N, 3, generator=g)).cuda().requires_grad_(True)
    one_hot = torch.nn.functional.one_hot(torch.randint(0, 20, (B, N), generator=g), 20).float().cuda()
    s, t = torch.zeros(B).cuda(), torch.rand(B, generator=g).cuda()
    x1 = x1.cuda()
    model = den.Denoiser(r0, **dims).cuda().train()
    params = [p for p in model.parameters() if p.requires_grad]

    def step():
        out = model((s, t), x0, x1, one_hot, box)
        loss = out.square().mean()
        return loss, torch.autograd.grad(loss, [x0] + params, allow_unused=True)

    loss, grads = step()
    finite = all(bool(torch.isfinite(gr).all()) for gr in grads if gr is not None)
    sec = timed_steps(torch, step, args.steps, args.warmup)
    with torch.no_grad():
        t_fwd = event_time(torch, lambda: model((s, t), x0, x1, one_hot, box), 5)
    return {"metric": "rank-0/1/2 denoiser training step (forward + backward) atoms/sec", "unit": "atoms/s",
            "value": B * N / sec, "ms_per_step": sec * 1e3, "dtype": "f32",
            "config": {"workload": "2 x [Messages + SelfTensProds], 4 systems x 2048 atoms, box 70 A, cutoff 6 A, 256 scalar "
                                   "+ 64 vector + 16 rank-2 channels, chan 256; gradients for the parameters and x0"},
            "detail": {"loss": float(loss.detach()), "gradients_finite": finite,
                       "parameters_with_gradient": sum(gr is not None for gr in grads[1:]), "parameters": len(params),
                       "inference_forward_ms_same_inputs": t_fwd * 1e3}}


def bench_products(torch, args):
    ops = importlib.import_module("learned-dynamics_amd.ops")
    out = {}
    for rows in (4096, 262144):
        g = torch.Generator().manual_seed(0x947 + 1)
        x = torch.randn(rows, 64, generator=g).cuda()
        v = torch.randn(rows, 64, 3, generator=g).cuda()
        t = event_time(torch, lambda: ops.tensor_prods_avd(x, v, v), 50, warmup=5)
        nbytes = rows * 64 * (4 + 12 + 4 + 12 + 36)
        out[f"rows_{rows}"] = {"us": t * 1e6, "nodes_per_s": rows / t, "bytes": nbytes,
                               "GB/s": nbytes / t / 1e9, "frac_of_hbm_peak": nbytes / t / 1e9 / PEAK_HBM_GBS}
    # the same three products as the reference module runs them: TensorProds(l, r, o) = lin_o(prod(lin_l, lin_r))
    tp = importlib.import_module("learned-dynamics_amd.tensor_products")
    torch.manual_seed(0x947 + 1)
    mods = [tp.TensorProds(1, 1, 0, 64, 64, 64, 64).cuda(), tp.TensorProds(0, 1, 1, 64, 64, 64, 64).cuda(),
            tp.TensorProds(1, 1, 2, 64, 64, 64, 64).cuda()]
    for rows in (4096, 262144):
        g = torch.Generator().manual_seed(0x947 + 1)
        x = torch.randn(rows, 64, generator=g).cuda()
        v = torch.randn(rows, 64, 3, generator=g).cuda()
        with torch.no_grad():
            t = event_time(torch, lambda: (mods[0](v, v), mods[1](x, v), mods[2](v, v)), 30, warmup=5)
        flop = 2 * rows * 64 * 64 * ((3 + 3 + 1) + (1 + 3 + 3) + (3 + 3 + 9))
        out[f"rows_{rows}"]["with_linears"] = {"us": t * 1e6, "GFLOP": flop / 1e9, "TFLOP/s": flop / t / 1e12,
                                               "frac_of_fp32_mfma_peak": flop / t / 1e12 / PEAK_FP32_MFMA_TFLOPS,
                                               "launches": 3}
    return {"metric": "fused tensor-product trio (v.v, x v, v(x)v), BASELINE configs[0]", "unit": "nodes/s",
            "value": out["rows_4096"]["nodes_per_s"], "detail": out,
            "note": "includes allocation of the three outputs; 4096 rows (17.8 MB) is launch-latency bound"}


def bench_polymer(torch, args, with_cpu=True):
    """The chain generator that feeds the models (polymer_sim(SimId.REPEL5, ...), the reference's own test shape
    extensions/polymer_sims_cuda/test.py:9-17 scaled up to fill the GPU: one workgroup per chain)."""
    ops = importlib.import_module("learned-dynamics_amd.ops")
    out = {}
    for batch, n, nsteps in ((32, 200, 100), (4096, 64, 100), (2048, 200, 100)):
        g = torch.Generator().manual_seed(0x947 + 6)
        steps = torch.randn(batch, n, 3, generator=g)
        x = (0.8 * steps / steps.norm(dim=-1, keepdim=True)).cumsum(1).cuda()
        v = torch.zeros(batch, n, 3).cuda()
        drag = torch.ones(n).cuda()
        t = event_time(torch, lambda: ops.repel5_sim(x, v, drag, 1.0, 0.01, nsteps, 7), 5, warmup=2)
        pairs = batch * n * max(n - 3, 0) * (nsteps + 1)
        out[f"batch{batch}_n{n}"] = {"ms": t * 1e3, "bead_steps_per_s": batch * n * nsteps / t,
                                     "pair_forces_per_s": pairs / t, "fp32_vector_tflops": pairs * 19 / t / 1e12,
                                     "frac_of_fp32_vector_peak": pairs * 19 / t / 1e12 / (PEAK_FP32_MFMA_TFLOPS / 2)}
    res = {"metric": "chain generator bead-steps/sec (repel5, 100 steps per call)", "unit": "bead-steps/s",
           "value": out["batch2048_n200"]["bead_steps_per_s"], "ms_per_step": out["batch2048_n200"]["ms"],
           "detail": out,
           "note": "19 flop per pair force (3 sub, 5 for |d|^2 + eps, 3 mul for the 6th power, 1 division counted as 1, "
                   "6 for the scaled accumulate); the peak is the fp32 vector rate without packed instructions; "
                   "32 chains occupy 32 of 256 CUs, which is all the parallelism the reference's test shape has"}
    if with_cpu:
        import numpy as np
        OPY = importlib.import_module("oracle.polymer")
        batch, n, nsteps = 8, 200, 10
        rng = np.random.default_rng(0)
        x0 = np.cumsum(rng.normal(size=(batch, n, 3)) * 0.46, axis=1).astype(np.float32)
        normals = OPY.philox_normals(7, batch, n, 0, nsteps + 1)
        t0 = time.perf_counter()
        OPY.repel5_sim(x0, np.zeros_like(x0), np.ones(n, np.float32), 1.0, 0.01, nsteps, normals)
        dt = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": batch * n * nsteps / dt, "unit": "bead-steps/s", "cores": 1, "kind": "port",
                               "sample": f"{batch} chains x {n} beads x {nsteps} steps, numpy oracle"}
    return res


def chain_positions(torch, systems, atoms, box, seed, noise=1.0):
    g = torch.Generator().manual_seed(seed)
    steps = torch.randn(systems, atoms, 3, generator=g)
    steps = 3.8 * steps / steps.norm(dim=-1, keepdim=True)
    pos = steps.cumsum(1) + torch.rand(systems, 1, 3, generator=g) * box
    return (pos + noise * torch.randn(systems, atoms, 3, generator=g)).contiguous()


def edge_kernel_roofline(torch, msg, graph, r_ij, rows, bf16=False):
    """The fused rank-0/1/2 edge kernel of one Messages layer timed alone (HIP events): algorithmic bytes =
    per edge 3 chan outputs + indices, encoding and direction; per node 13 chan inputs read once and 60 chan
    sums written (4 bytes each, 2 with bf16 storage)."""
    ops = importlib.import_module("learned-dynamics_amd.ops")
    chan = int(msg.lin_enc.weight.shape[0])
    dev = r_ij.device
    dt = torch.bfloat16 if bf16 else torch.float32
    g = torch.Generator(device="cuda").manual_seed(1)
    La = torch.randn(rows, chan, device=dev, generator=g).to(dt)
    Lv = torch.randn(rows, 3, chan, device=dev, generator=g).to(dt)
    Ld = torch.randn(rows, 9, chan, device=dev, generator=g).to(dt)
    enc, rhat = ops.bee_edge_geometry(r_ij.contiguous(), msg.r0)
    order = getattr(graph, "cell_order", None)
    if bf16:
        fn = lambda: ops.bee_message_bf16(graph.row_ptr, graph.dst32, rhat, enc, La, Lv, Ld, msg.lin_enc.weight,
                                          msg.lin_enc.bias, node_order=order)
    else:
        # as the layer calls it: with few rank-2 output channels the kernel applies that output linear to its node
        # sums itself (and then does not store them)
        bl = importlib.import_module("learned-dynamics_amd.bee_layers")
        Y2 = msg._cat_Y(bl.LABELS_2, 0.1)
        fused = ops.bee_rank2_supported(chan, Y2.shape[0])
        fn = lambda: ops.bee_message(graph.row_ptr, graph.dst32, rhat, enc, La, Lv, Ld, msg.lin_enc.weight,
                                     msg.lin_enc.bias, node_order=order, want_node_max=True, Y2=Y2 if fused else None)
    t = event_time(torch, fn, 10)
    E = int(graph.src.numel())
    w = 2 if bf16 else 4
    # algorithmic bytes: the 13 node components read once and the 63 per-channel product sums written once per node,
    # plus index and edge vector per edge.  The three scalar products the kernel also stores per edge (the input of the
    # per-edge MLP) are not compulsory traffic and are listed on their own.
    nbytes = rows * (13 + 63) * chan * w + E * 16
    p0_bytes = E * 3 * chan * w
    return {"kernel": "bee_message_kernel (gathers, 13 products, edge sums; one Messages layer"
                      + ("; the rank-2 output linear applied to the node sums in the kernel)" if not bf16 and fused else ")"),
            "bound": "hbm",
            "achieved": nbytes / t / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": nbytes / t / 1e9 / PEAK_HBM_GBS,
            "traffic": measured_traffic("bee_message_kernel", "stress_configs4_traffic.json" if bf16
                                        else "denoiser_configs3_traffic.json"),
            "bytes_per_launch": nbytes, "ms": t * 1e3,
            "per_edge_scalar_products_stored_bytes": p0_bytes,
            "frac_counting_the_stored_scalar_products": (nbytes + p0_bytes) / t / 1e9 / PEAK_HBM_GBS,
            # the 13 products are 167 flop per (edge, channel), the 60 running sums another 60
            "fp32_vector_tflops": E * chan * 227 / t / 1e12,
            "fp32_vector_frac_of_peak": E * chan * 227 / t / 1e12 / PEAK_FP32_MFMA_TFLOPS,
            "note": "gathered node rows are served by L2 and counted once per node; the fp32 vector peak is the "
                    "published 157.3 TFLOP/s, which needs packed fp32 instructions (compiled out here: 78.65 reachable)"}


def single_system_latency(torch, model, dev, box, r0, atoms):
    """One system of the denoiser workload: the 8 blocks on a prebuilt neighbour graph, run eagerly and replayed
    from a captured HIP graph (the neighbour search stays outside the capture)."""
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    ro = importlib.import_module("learned-dynamics_amd.rollout")
    with torch.no_grad():
        one = [v[:1].contiguous() for v in dev]
        g1, _ = gl.graph_setup(r0, box, one[3], neighbours_max=256, celllist_max=64)

        def layers(s_, t_, x0_, x1_):
            return model.forward_on_graph((s_, t_), x0_, x1_, one[4], g1, gl.edge_vectors(g1, x1_, box))
        t_eager = event_time(torch, lambda: layers(*one[:4]), 10)
        captured = ro.GraphedCall(layers, *one[:4])
        t_graph = event_time(torch, lambda: captured(*one[:4]), 10)
    return {"atoms": atoms, "edges": int(g1.src.numel()), "layers_eager_ms": t_eager * 1e3,
            "layers_hip_graph_replay_ms": t_graph * 1e3,
            "note": "8 blocks on a prebuilt neighbour graph, one system; the replay includes the copies into the "
                    "capture's static inputs; inside a capture the independent pieces of a layer run on side streams"}


def bench_denoiser(torch, args, with_cpu=True):
    """BASELINE configs[3]: 8-block rank-0/1/2 denoiser forward, 32 systems x 2048 atoms."""
    den = importlib.import_module("learned-dynamics_amd.denoiser")
    seed = 0x947 + 4
    torch.manual_seed(seed)
    B, N, box_len, r0 = 32, 2048, 70.0, 6.0
    dims = dict(dim_a=256, dim_v=64, dim_d=16, chan=256, blocks=8)
    box = (box_len,) * 3
    x1 = chain_positions(torch, B, N, box_len, seed)
    g = torch.Generator().manual_seed(seed + 1)
    x0 = x1 + torch.randn(B, N, 3, generator=g)
    types = torch.randint(0, 20, (B, N), generator=g)
    one_hot = torch.nn.functional.one_hot(types, 20).float()
    s, t = torch.zeros(B), torch.rand(B, generator=g)
    model = den.Denoiser(r0, **dims).cuda().eval()
    dev = [v.cuda() for v in (s, t, x0, x1, one_hot)]

    with torch.no_grad():
        def step():
            return model((dev[0], dev[1]), dev[2], dev[3], dev[4], box)
        step()
        sec = timed_steps(torch, step, args.steps, args.warmup)
        gl = importlib.import_module("learned-dynamics_amd.graph_layers")
        graph, _ = gl.graph_setup(r0, box, dev[3], neighbours_max=256, celllist_max=64)
        E = int(graph.src.numel())
        edge_roof = edge_kernel_roofline(torch, model.messages[0], graph, gl.edge_vectors(graph, dev[3], box), B * N)
    single = None if getattr(args, "no_extras", False) else single_system_latency(torch, model, dev, box, r0, N)
    out = {"metric": "denoiser forward atoms/sec", "value": B * N / sec, "unit": "atoms/s", "ms_per_step": sec * 1e3,
           "dtype": "f32",
           "config": {"workload": "BASELINE configs[3]: 8 x [Messages + SelfTensProds] rank-0/1/2 denoiser forward "
                                  "(assembled from reference modules), 32 systems x 2048 atoms, box 70 A, cutoff 6 A, "
                                  "256 scalar + 64 vector + 16 rank-2 channels, chan 256, graph rebuilt every forward",
                      "edges": E, "atoms": B * N},
           "roofline": edge_roof, "single_system": single}
    if with_cpu:
        out["cpu_baseline"] = cpu_denoiser_block(torch, model, x1[:1], r0, box, dims)
    return out


def bench_meanflow_painn(torch, args):
    """The PaiNN meanflow denoiser (archs/meanflow_painn8.py:185-217 with a one-hot atom embedding): 2 + 5 blocks, each a
    radius-graph message, a bond message and an update; 16384 atoms at the density of configs[2] (80 A box, n = 128)
    on a jittered lattice with the cutoff at 5 A, which keeps every atom inside the reference's default caps (64
    neighbours, 32 atoms per cell; the model calls graph_setup with them); bonds join lattice neighbours in chains of
    1024; both radius graphs are rebuilt inside the forward."""
    mf = importlib.import_module("learned-dynamics_amd.meanflow_painn")
    n, r0, box_len, chains, atoms = 128, 5.0, 80.0, 16, 1024
    box = (box_len,) * 3
    seed = 0x947 + 7
    torch.manual_seed(seed)
    N = chains * atoms
    g = torch.Generator().manual_seed(seed + 1)
    side = 26                                                      # 26^3 >= 16384 lattice sites, 3.08 A apart
    k = torch.arange(N)
    sites = torch.stack([k % side, (k // side) % side, k // (side * side)], dim=1).float() * (box_len / side)
    x1 = (sites + 0.5 * torch.randn(N, 3, generator=g)).reshape(1, N, 3).contiguous()
    x0 = x1 + 0.3 * torch.randn(1, N, 3, generator=g)
    one_hot = torch.nn.functional.one_hot(torch.randint(0, 20, (N,), generator=g), 20).float()
    idx = torch.arange(N - 1)
    idx = idx[(idx + 1) % atoms != 0]                              # bonds along each chain, both directions
    topo = mf.Topology(one_hot.cuda(), torch.cat([idx, idx + 1]).cuda(), torch.cat([idx + 1, idx]).cuda())
    model = mf.SE3ITO(r0, n, N).cuda().eval()
    s, t = torch.zeros(1).cuda(), torch.rand(1, generator=g).cuda()
    x0_d, x1_d = x0.cuda(), x1.cuda()
    with torch.no_grad():
        def step():
            return model((s, t), x0_d, x1_d, box, topo)
        step()
        sec = timed_steps(torch, step, args.steps, args.warmup)
    return {"metric": "PaiNN meanflow denoiser forward atoms/sec", "value": N / sec, "unit": "atoms/s",
            "ms_per_step": sec * 1e3, "dtype": "f32 storage and accumulation",
            "config": {"workload": "SE3ITO forward (2 + 5 PaiNN blocks with bond messages, n = 128), 16384 atoms on a jittered "
                                   "lattice, box 80 A, cutoff 5 A, radius graphs rebuilt in the forward", "atoms": N}}


def bench_meanflow_train(torch, args):
    """The reference's training step for the PaiNN meanflow denoiser (archs/meanflow_painn8.py:274-296): the
    Jacobian-vector product of the model along (v, 1), the target v - (t - s) jvp, the model's value at the same
    point, the squared error, and its gradient for every parameter.  Timed in two formulations with the same result:
    the jvp in forward mode (differentiable.jvp) and, as the reference writes it, out of nested backward passes.  4 systems of 1024 atoms (jittered lattice, cutoff 5 A), n = 128, 1 + 2
    blocks, positions that move."""
    mf = importlib.import_module("learned-dynamics_amd.meanflow_painn")
    n, r0, box_len, B, N = 128, 5.0, 32.0, 4, 1024
    box = (box_len,) * 3
    seed = 0x947 + 11
    torch.manual_seed(seed)
    g = torch.Generator().manual_seed(seed + 1)
    side = 11                                                      # 11^3 >= 1024 lattice sites, 2.9 A apart
    k = torch.arange(N)
    sites = torch.stack([k % side, (k // side) % side, k // (side * side)], dim=1).float() * (box_len / side)
    x_prev = (sites[None] + 0.4 * torch.randn(B, N, 3, generator=g)).contiguous().cuda()
    z_0 = (x_prev.cpu() + 0.2 * torch.randn(B, N, 3, generator=g)).cuda()
    z_1 = (x_prev.cpu() + 0.5 * torch.randn(B, N, 3, generator=g)).cuda()
    one_hot = torch.nn.functional.one_hot(torch.randint(0, 20, (N,), generator=g), 20).float()
    idx = torch.arange(N - 1)
    topo = mf.Topology(one_hot.cuda(), torch.cat([idx, idx + 1]).cuda(), torch.cat([idx + 1, idx]).cuda())
    model = mf.SE3ITO(r0, n, N, blks_0=1, blks_1=2, mutate_pos=True).cuda().train()
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("lin_push_pos.W"):
                p.mul_(0.05)
    params = [p for p in model.parameters() if p.requires_grad]
    t, s_ = torch.rand(B, generator=g).cuda(), torch.zeros(B).cuda()

    diff = importlib.import_module("learned-dynamics_amd.differentiable")

    def step(forward_mode=True):
        z_t = t[:, None, None] * z_1 + (1 - t[:, None, None]) * z_0
        v = z_1 - z_0
        f = lambda zz, tt: model((s_, tt), x_prev, zz, box, topo)
        if forward_mode:
            # one pass gives the model's value at (z_t, t), which is v_pred, and its derivative along (v, 1)
            v_pred, jvp = diff.jvp(f, (z_t, t), (v, torch.ones_like(t)))
        else:
            # as the reference writes it: the derivative out of two nested backward passes, then the model again
            _, jvp = torch.autograd.functional.jvp(f, (z_t, t), (v, torch.ones_like(t)), create_graph=True)
            v_pred = model((s_, t), x_prev, z_t, box, topo)
        v_target = v - (t - s_)[:, None, None] * jvp
        loss = ((v_pred - v_target) ** 2).mean()
        return loss, torch.autograd.grad(loss, params, allow_unused=True)

    loss, grads = step()
    finite = all(bool(torch.isfinite(gr).all()) for gr in grads if gr is not None)
    sec = timed_steps(torch, step, args.steps, args.warmup)
    nested = {}
    if not getattr(args, "no_comparisons", False):
        loss_nested, grads_nested = step(forward_mode=False)
        # the two formulations give the same gradients: largest difference relative to the largest entry of each
        worst = max(float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))
                    for a, b in zip(grads, grads_nested) if a is not None and b is not None)
        sec_nested = timed_steps(torch, lambda: step(forward_mode=False), args.steps, args.warmup)
        nested = {"nested_backward_ms_per_step": sec_nested * 1e3,
                  "nested_backward": "torch.autograd.functional.jvp(create_graph=True), a second forward, backward: "
                                     "the reference's formulation (archs/meanflow_painn8.py:274-296)",
                  "loss_nested_backward": float(loss_nested.detach()),
                  "parameters_with_gradient_nested_backward": sum(gr is not None for gr in grads_nested),
                  "largest_relative_gradient_difference_between_the_two": worst}
    with torch.no_grad():
        t_fwd = event_time(torch, lambda: model((s_, t), x_prev, z_1, box, topo), 5)
    return {"metric": "PaiNN meanflow training step (jvp + loss gradient) atoms/sec", "unit": "atoms/s",
            "value": B * N / sec, "ms_per_step": sec * 1e3, "dtype": "f32",
            "config": {"workload": "SE3ITO, 1 + 2 blocks with bond messages, n = 128, positions that move; 4 systems x 1024 "
                                   "atoms, box 32 A, cutoff 5 A; the jvp in forward mode (one pass gives v_pred and the "
                                   "jvp) + backward"},
            "detail": {"loss": float(loss.detach()), "gradients_finite": finite,
                       "parameters_with_gradient": sum(gr is not None for gr in grads), "parameters": len(params),
                       **nested, "inference_forward_ms_same_inputs": t_fwd * 1e3}}


def bench_stress(torch, args, with_cpu=True):
    """BASELINE configs[4]: 65536 atoms uniform in a periodic cube at 0.1 atoms/A^3, cutoff 6 A,
    4 x [Messages + SelfTensProds] with 128 channels per rank, features stored as bf16 with fp32
    accumulation, neighbour rebuild inside the step.  The fp32-storage path on the same problem is
    timed beside it."""
    bee = importlib.import_module("learned-dynamics_amd.bee_layers")
    b16 = importlib.import_module("learned-dynamics_amd.bee_layers_bf16")
    gl = importlib.import_module("learned-dynamics_amd.graph_layers")
    seed = 0x947 + 5
    torch.manual_seed(seed)
    N, r0, C, layers = 65536, 6.0, 128, 4
    L = (N / 0.1) ** (1.0 / 3.0)
    box = (L, L, L)
    g = torch.Generator().manual_seed(seed)
    pos = (torch.rand(1, N, 3, generator=g) * L).cuda()
    x_a = torch.randn(1, N, C, generator=g).cuda()
    x_v = (torch.randn(1, N, C, 3, generator=g) / 3 ** 0.5).cuda()
    x_d = (torch.randn(1, N, C, 3, 3, generator=g) / 3.0).cuda()
    msgs = [bee.Messages(r0, C, C, C, C).cuda().eval() for _ in range(layers)]
    prods = [bee.SelfTensProds(C, C, C, C).cuda().eval() for _ in range(layers)]
    edges = [0]

    with torch.no_grad():
        def step_f32():
            graph, r_ij = gl.graph_setup(r0, box, pos, neighbours_max=256, celllist_max=64)
            edges[0] = int(graph.src.numel())
            a, v, d = x_a, x_v, x_d
            for m, p in zip(msgs, prods):
                da, dv, dd = m(graph, r_ij, a, v, d)
                a, v, d = a + da, v + dv, d + dd
                a, v, d = p(a, v, d, residual=True)
            return a

        def step_bf16():
            graph, r_ij = gl.graph_setup(r0, box, pos, neighbours_max=256, celllist_max=64)
            edges[0] = int(graph.src.numel())
            return b16.stack_forward(msgs, prods, graph, r_ij, x_a, x_v, x_d)

        ref = step_f32()
        out = step_bf16()[0]
        rel = float((out - ref).abs().max() / ref.abs().max())
        sec16 = timed_steps(torch, step_bf16, args.steps, args.warmup)
        sec32 = None if getattr(args, "no_comparisons", False) else timed_steps(torch, step_f32, args.steps, args.warmup)
        graph, r_ij = gl.graph_setup(r0, box, pos, neighbours_max=256, celllist_max=64)
        edge_roof = edge_kernel_roofline(torch, msgs[0], graph, r_ij, N, bf16=True)
    E = edges[0]
    cpu = cpu_stress_layer(torch, msgs[0], prods[0], r0, C, seed) if with_cpu else None
    return {"metric": "message-passing edges/sec per layer", "value": E * layers / sec16, "unit": "edges/s",
            "roofline": edge_roof, "cpu_baseline": cpu,
            "ms_per_step": sec16 * 1e3, "dtype": "bf16 storage, f32 accumulate",
            "config": {"workload": "BASELINE configs[4]: 65536 atoms, density 0.1/A^3, cutoff 6 A, "
                                   "4 x [Messages + SelfTensProds], 128 channels per rank, bf16 storage, "
                                   "neighbour rebuild in the step",
                       "edges": E, "atoms": N, "layers": layers, "atoms_per_s": N / sec16},
            "max_abs_diff_vs_fp32_storage_over_scale": rel,
            "fp32_storage": None if sec32 is None else {"value": E * layers / sec32, "unit": "edges/s",
                                                        "ms_per_step": sec32 * 1e3}}


def _bee_weights(msg, prod):
    """Weights of one Messages + SelfTensProds pair as the oracle takes them."""
    from oracle import products as OP
    dd = lambda p: p.detach().cpu()
    Lm = msg.mlp_a.layers
    w = {"L0": dd(msg.L0.W), "L1": dd(msg.L1.W), "L2": dd(msg.L2.W),
         "Y": {lab: dd(getattr(msg, f"Y_{lab}").W) for lab in OP.BEE_ORDER},
         "enc_W": dd(msg.lin_enc.weight), "enc_b": dd(msg.lin_enc.bias),
         "mlp_a": {"W_direct": dd(msg.mlp_a.lin_direct.weight), "W1": dd(Lm[0].weight), "b1": dd(Lm[0].bias),
                   "W2": dd(Lm[2].weight), "b2": dd(Lm[2].bias), "W3": dd(Lm[4].weight), "b3": dd(Lm[4].bias)}}
    ws = {k: dd(getattr(prod, k).W) for k in ("L0", "R0", "L1", "R1", "L2", "R2")}
    ws["Y"] = {lab: dd(getattr(prod, f"Y_{lab}").W) for lab in OP.BEE_ORDER}
    ws.update(gn_a=dd(prod.gn_a.gamma), gn_v=dd(prod.gn_v.gamma), gn_d=dd(prod.gn_d.gamma))
    return w, ws


def cpu_stress_layer(torch, msg, prod, r0, C, seed):
    """Oracle (fp32 PyTorch CPU port of the reference math): ONE layer (Messages + SelfTensProds, 128 channels per
    rank) on 1024 atoms at the density of configs[4] (1/64 of its atoms; the per-edge rank-2 tensors of the
    reference formulation, 13 of size edges x 128 x 9, do not fit the host for more)."""
    from oracle import layers as OL
    from oracle import neighbour as ON
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    N = 1024
    L = (N / 0.1) ** (1.0 / 3.0)
    box = (L, L, L)
    g = torch.Generator().manual_seed(seed + 7)
    pos = (torch.rand(1, N, 3, generator=g) * L).contiguous()
    ref = ON.edges(pos.numpy(), r0, box)
    src, dst = torch.from_numpy(ref["src"]).long(), torch.from_numpy(ref["dst"]).long()
    r_ij = torch.from_numpy(ON.edge_vectors(pos.numpy(), ref["src"], ref["dst"], box))
    w, ws = _bee_weights(msg, prod)
    x_a = torch.randn(1, N, C, generator=g)
    x_v = torch.randn(1, N, C, 3, generator=g) / 3 ** 0.5
    x_d = torch.randn(1, N, C, 3, 3, generator=g) / 3.0

    def layer():
        d = OL.bee_messages(src, dst, 1, N, r_ij, x_a, x_v, x_d, w, r0)
        return OL.self_tens_prods(x_a + d[0], x_v + d[1], x_d + d[2], ws)

    with torch.no_grad():
        layer()
        times = []
        t_all = time.perf_counter()
        while len(times) < 3 or (time.perf_counter() - t_all < 10 and len(times) < 10):
            t0 = time.perf_counter()
            layer()
            times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": len(src) / med, "unit": "edges/s", "cores": cores, "kind": "port",
            "sample": f"{N} atoms at 0.1 / A^3 ({len(src)} edges; 1/64 of the atoms), one of the 4 layers, fp32 storage, "
                      f"median of {len(times)} runs, PyTorch CPU fp32; neighbour search not included"}


def cpu_denoiser_block(torch, model, x1, r0, box, dims):
    """Oracle (fp32 PyTorch CPU port of the reference math): ONE block (Messages + SelfTensProds) on ONE of the
    32 systems; the forward is 8 such blocks per system, so atoms/s = atoms / (8 * t_block)."""
    from oracle import layers as OL
    from oracle import neighbour as ON
    from oracle import products as OP
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    N = x1.shape[1]
    ref = ON.edges(x1.numpy(), r0, box)
    src, dst = torch.from_numpy(ref["src"]).long(), torch.from_numpy(ref["dst"]).long()
    r_ij = torch.from_numpy(ON.edge_vectors(x1.numpy(), ref["src"], ref["dst"], box))
    msg, prod = model.messages[0], model.prods[0]
    dd = lambda p: p.detach().cpu()
    Lm = msg.mlp_a.layers
    w = {"L0": dd(msg.L0.W), "L1": dd(msg.L1.W), "L2": dd(msg.L2.W),
         "Y": {lab: dd(getattr(msg, f"Y_{lab}").W) for lab in OP.BEE_ORDER},
         "enc_W": dd(msg.lin_enc.weight), "enc_b": dd(msg.lin_enc.bias),
         "mlp_a": {"W_direct": dd(msg.mlp_a.lin_direct.weight), "W1": dd(Lm[0].weight), "b1": dd(Lm[0].bias),
                   "W2": dd(Lm[2].weight), "b2": dd(Lm[2].bias), "W3": dd(Lm[4].weight), "b3": dd(Lm[4].bias)}}
    ws = {k: dd(getattr(prod, k).W) for k in ("L0", "R0", "L1", "R1", "L2", "R2")}
    ws["Y"] = {lab: dd(getattr(prod, f"Y_{lab}").W) for lab in OP.BEE_ORDER}
    ws.update(gn_a=dd(prod.gn_a.gamma), gn_v=dd(prod.gn_v.gamma), gn_d=dd(prod.gn_d.gamma))
    g = torch.Generator().manual_seed(1)
    x_a = torch.randn(1, N, dims["dim_a"], generator=g)
    x_v = torch.randn(1, N, dims["dim_v"], 3, generator=g)
    x_d = torch.randn(1, N, dims["dim_d"], 3, 3, generator=g)

    def block():
        d = OL.bee_messages(src, dst, 1, N, r_ij, x_a, x_v, x_d, w, r0)
        return OL.self_tens_prods(x_a + d[0], x_v + d[1], x_d + d[2], ws)

    with torch.no_grad():
        block()
        times = []
        t_all = time.perf_counter()
        while len(times) < 3 or (time.perf_counter() - t_all < 10 and len(times) < 10):
            t0 = time.perf_counter()
            block()
            times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": N / (dims["blocks"] * med), "unit": "atoms/s", "cores": cores, "kind": "port",
            "sample": f"1 of 32 systems ({N} atoms, {len(src)} edges), 1 of 8 blocks timed (median of {len(times)}), "
                      f"scaled by 8 blocks; PyTorch CPU fp32"}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU; independent boxes shard by batch with no communication, "
              "so there is no multi-GPU figure to report (use --gpus 1).", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)

    if args.calibrate_copy:
        a = torch.empty(1 << 28, dtype=torch.float32, device="cuda")
        b = torch.empty_like(a)
        t_copy = event_time(torch, lambda: b.copy_(a), 5)
        print(f"calibration copy: 1 GiB read + 1 GiB written in {t_copy * 1e3:.3f} ms "
              f"({2 * a.numel() * 4 / t_copy / 1e9:.0f} GB/s)", file=sys.stderr)
        del a, b
    if args.workload == "painn_layer":
        res = bench_painn_layer(torch, args)
        if not args.no_extras:
            small = argparse.Namespace(steps=20, warmup=10)
            nb = bench_neighbour(torch, small, with_cpu=not args.no_cpu)
            dn = bench_denoiser(torch, argparse.Namespace(steps=20, warmup=5), with_cpu=not args.no_cpu)
            st = bench_stress(torch, argparse.Namespace(steps=20, warmup=5, no_comparisons=False), with_cpu=not args.no_cpu)
            res["other_workloads"] = {"denoiser_forward_configs[3]": dn, "neighbour_search_configs[1]": nb,
                                      "tensor_products_configs[0]": bench_products(torch, small),
                                      "stress_configs[4]": st,
                                      "meanflow_painn_forward": bench_meanflow_painn(torch, argparse.Namespace(steps=10, warmup=3)),
                                      "painn_block_training_step": bench_painn_train(torch, argparse.Namespace(steps=5, warmup=2)),
                                      "painn_meanflow_training_step": bench_meanflow_train(torch, argparse.Namespace(steps=3, warmup=1))}
    elif args.workload == "neighbour":
        res = bench_neighbour(torch, args, with_cpu=not args.no_cpu)
    elif args.workload == "denoiser":
        res = bench_denoiser(torch, args, with_cpu=not args.no_cpu)
    elif args.workload == "stress":
        res = bench_stress(torch, args, with_cpu=not args.no_cpu)
    elif args.workload == "meanflow_painn":
        res = bench_meanflow_painn(torch, args)
    elif args.workload == "polymer":
        res = bench_polymer(torch, args, with_cpu=not args.no_cpu)
    elif args.workload == "gemm_power":
        res = bench_gemm_power(torch, args)
    elif args.workload == "painn_train":
        res = bench_painn_train(torch, args)
    elif args.workload == "denoiser_train":
        res = bench_denoiser_train(torch, args)
    elif args.workload == "meanflow_train":
        res = bench_meanflow_train(torch, args)
    else:
        res = bench_products(torch, args)
        res.setdefault("ms_per_step", res["detail"]["rows_4096"]["us"] * 1e-3)

    line = {"metric": res.pop("metric"), "value": res.pop("value"), "unit": res.pop("unit"), "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": res.pop("ms_per_step"),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": res.pop("dtype", "f32"),
            "data": "synthetic"}
    line.update(res)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
