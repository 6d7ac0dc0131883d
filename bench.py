"""Benchmark of the fixed-fan-in sparse layer on one MI355X.

One step = forward + backward (input gradient and weight gradient) of the layer over one batch of
synthetic input that is already resident in HBM, through the same C-ABI entry points the op
bindings use.  Prints ONE JSON line (metric: samples/s of forward+backward at 670,091 labels,
fan-in 32), with the roofline figures of the slowest kernel and a CPU baseline timed on this box.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2] [--layout nb|bn]
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

HBM_PEAK_GBPS = 8000.0        # MI355X published HBM3E peak
# the other two resources every multiply-add of this path uses (published figures): the gathered operand comes out
# of LDS (4 bytes per multiply-add; 256 bytes per clock per CU, 256 CUs, 2.4 GHz) and the multiply-add itself is a
# plain FP32 FMA (packed FP32 forms are not used: half of the 157.3 TFLOP/s vector peak)
LDS_PEAK_GBPS = 256 * 256 * 2.4
FP32_FMA_PEAK_TFLOPS = 157.3 / 2

PROFILE_DIR = os.path.join(ROOT, "profiles")

# GPU kernels behind each pass (one C-ABI call)
PASS_KERNELS = {
    "forward": "fwd_lane32_kernel",
    "weight_grad": "wgrad_stream_kernel",
    "input_grad": "igrad_permute_weights_kernel + igrad_tile_kernel + igrad_reduce_kernel",
}
WIDE_PASS_KERNELS = {
    "forward": "fwd_wide_kernel",
    "weight_grad": "wgrad_wide_kernel",
    "input_grad": "transpose_kernel + igrad_wide_kernel",
}


def measured_traffic(config_name):
    """HBM bytes per launch of each pass, read from the committed counter summary profiles/ffi_<config>_counters.txt
    (lines `traffic_bytes <pass> <bytes>`; rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this file, scaled by what the
    same counters read for a plain copy kernel of known size).  Returns ({pass: bytes}, source) or ({}, None)."""
    path = os.path.join(PROFILE_DIR, f"ffi_{config_name}_counters.txt")
    out, stamp = {}, None
    if os.path.exists(path):
        for line in open(path):
            f = line.split()
            if len(f) >= 3 and f[0] == "traffic_bytes":
                out[f[1]] = float(f[2])
            elif len(f) >= 2 and f[0] == "measured_at":
                stamp = " ".join(f[1:])
    return out, (f"profiles/{os.path.basename(path)}" + (f" ({stamp})" if stamp else "")) if out else None


def measured_pipe_load(config_name):
    """Per pass: VALU wavefront-instructions and LDS-busy cycles per launch, from the same counter summary (lines
    `valu_insts <pass> <n>` = SQ_INSTS_VALU, `lds_busy_cycles <pass> <n>` = SQ_LDS_IDX_ACTIVE, summed over the pass's kernels)."""
    path = os.path.join(PROFILE_DIR, f"ffi_{config_name}_counters.txt")
    out = {"valu_insts": {}, "lds_busy_cycles": {}}
    if os.path.exists(path):
        for line in open(path):
            f = line.split()
            if len(f) >= 3 and f[0] in out:
                out[f[0]][f[1]] = float(f[2])
    return out


def attainable(cfg, alg, config_name):
    """What this design would reach if, in every pass, the slowest of its three resources ran without a gap: the VALU at
    one instruction per 4 clocks and SIMD with the instruction counts the kernels have NOW (multiply-adds plus address,
    unpacking and padding overhead, SQ_INSTS_VALU), the LDS with the cycles per read it shows NOW (bank conflicts
    included, SQ_LDS_IDX_ACTIVE), HBM at its published peak.  Measured time above this is lost overlap (phases that wait
    for each other); this figure above the HBM floor is the price of the instruction mix, the padding and the conflicts."""
    load = measured_pipe_load(config_name)
    if not load["valu_insts"]:
        return None
    simds, cus, clk = 1024.0, 256.0, 2.4e9
    per_pass = {}
    for k in ("forward", "weight_grad", "input_grad"):
        if k not in load["valu_insts"] or k not in load["lds_busy_cycles"]:
            return None
        valu = load["valu_insts"][k] * 4.0 / simds / clk
        lds = load["lds_busy_cycles"][k] / cus / clk
        hbm = alg[k] / (HBM_PEAK_GBPS * 1e9)
        per_pass[k] = {"valu_ms": round(valu * 1e3, 4), "lds_ms": round(lds * 1e3, 4), "hbm_ms": round(hbm * 1e3, 4),
                       "bound_ms": round(max(valu, lds, hbm) * 1e3, 4)}
    step = sum(v["bound_ms"] for v in per_pass.values())
    return {"ms_per_step": round(step, 4), "samples_per_s": round(cfg.batch / (step * 1e-3), 1),
            "frac_of_hbm_peak": round(alg["total"] / (step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4), "per_pass": per_pass,
            "basis": f"SQ_INSTS_VALU and SQ_LDS_IDX_ACTIVE per launch from profiles/ffi_{config_name}_counters.txt, 1,024 SIMDs x 4 clocks per "
                     "instruction, 256 CUs, 2.4 GHz, HBM 8 TB/s; per pass the largest of the three"}


def rewire_costs(pkg, cfg, x, lookup, w, g, tp, stream):
    """What a rewiring step costs the backward pass (the reference rewires every `rewire_interval` steps,
    sparse/optimizer.py:68-74; tasks/amazon670k-cascade.json: 1000, also 100): the plan build alone, the first
    ffi_backward_f32 after the library's own ffi_rewire_f32 (rebuilds the plan first), and after an edit of the lookup
    by foreign code (served once by the kernels that read the lookup directly, then rebuilt).  Host-timed, each call
    bracketed by synchronisations; on a copy of the lookup."""
    import ctypes

    import torch
    B, N, L, K = cfg.batch, cfg.num_features, cfg.num_units, cfg.fan_in
    lib, check, sh = pkg._lib.lib(), pkg._lib.check, stream.cuda_stream
    ptr = lambda a: a.data_ptr()  # noqa: E731
    lookup2 = lookup.clone()
    gx, gw = torch.empty_like(x), torch.empty_like(w)

    def timed(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3

    backward = lambda: check(lib.ffi_backward_f32(ptr(x), ptr(lookup2), ptr(w), ptr(g), ptr(gx), ptr(gw), B, N, L, K, int(tp), sh))  # noqa: E731
    for _ in range(5):
        backward()
    normal = min(timed(backward) for _ in range(5))
    plan = ctypes.c_void_p()
    check(lib.ffi_plan_create(ptr(lookup2), L, K, N, B, sh, ctypes.byref(plan)))
    build = min(timed(lambda: check(lib.ffi_plan_refresh(plan, ptr(lookup2), sh))) for _ in range(3))
    check(lib.ffi_plan_destroy(plan))
    thr = torch.empty(1, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(11)

    def rewire(target=lookup2):
        check(lib.ffi_select_threshold_f32(ptr(w), L * K, (L * K) // 100, ptr(thr), sh))
        check(lib.ffi_rewire_f32(ptr(target), ptr(w), None, 0, L * K, N, ptr(thr), 12345, None, sh))

    rewire(lookup.clone())                       # (untimed, on another copy: the selection's workspace is allocated once per process)
    rewire_ms = timed(rewire)
    first_library = timed(backward)
    after_library = timed(backward)
    # (a rewired lookup has labels that list a column twice -- about 4 % of the redrawn connections land on a column their
    # label already has -- and tiles with such labels take the slower of the plan's two slot placements)
    check(lib.ffi_plan_create(ptr(lookup2), L, K, N, B, sh, ctypes.byref(plan)))
    build_rewired = min(timed(lambda: check(lib.ffi_plan_refresh(plan, ptr(lookup2), sh))) for _ in range(3))
    check(lib.ffi_plan_destroy(plan))
    pos = torch.randint(0, L * K, ((L * K) // 100,), device="cuda", generator=gen)
    lookup2.view(-1)[pos] = torch.randint(0, N, (pos.numel(),), device="cuda", generator=gen, dtype=torch.int32)
    first_foreign = timed(backward)
    second_foreign = timed(backward)
    after_foreign = timed(backward)
    out = {"backward_ms": round(normal, 4), "plan_build_ms": round(build, 4), "plan_build_after_rewire_ms": round(build_rewired, 4),
           "select_and_rewire_1pct_ms": round(rewire_ms, 4),
           "first_backward_after_rewire_ms": {"library_rewire": round(first_library, 4), "foreign_in_place_edit": round(first_foreign, 4)},
           "second_backward_after_rewire_ms": {"library_rewire": round(after_library, 4), "foreign_in_place_edit": round(second_foreign, 4)},
           "third_backward_after_foreign_edit_ms": round(after_foreign, 4),
           "note": "library route: ffi_rewire_f32 marks the cached plan outdated, the next backward rebuilds it and runs the plan-driven kernels; "
                   "foreign route: the first backward runs the kernels that read the lookup directly (the input gradient sorts every label tile by column on the fly), the second rebuilds"}
    extra_library = rewire_ms + first_library - normal
    extra_foreign = (first_foreign - normal) + (second_foreign - normal)
    out["amortised_ms_per_step"] = {f"rewire_interval_{i}": {"library_rewire": round(extra_library / i, 5), "foreign_in_place_edit": round(extra_foreign / i, 5)}
                                    for i in (100, 1000)}
    return out


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)      # (the GPU clock takes tens of milliseconds of load to settle)
    ap.add_argument("--config", default="c2", help="workload: c1..c4 forward + backward in fp32 (c2 is the headline); "
                                                   "c5 = bf16 forward with top-5 per sample (inference)")
    ap.add_argument("--layout", default="nb", choices=["nb", "bn"],
                    help="features as [N,B] (the production 'Tp' op) or [B,N]")
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--arranged", action="store_true",
                    help="reorder every label's connections with ffi_arrange_connections_f32 first (same connection sets)")
    ap.add_argument("--cpu-labels", type=int, default=0, help="labels in the CPU-baseline sample (0 = auto)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--train-step", type=float, default=0.0, metavar="DENSITY",
                    help="also time one training step of the layer (forward + squared-hinge loss gradient in one kernel, "
                         "backward over the non-zero gradients and Adam in one call) with the bias set so that this share of the loss "
                         "gradients is non-zero; reported under 'train_step' in the same JSON line")
    ap.add_argument("--preload-ms", type=float, default=150.0,
                    help="milliseconds of untimed steps in front of the warm-up: the GPU's clocks settle under load within tens of "
                         "milliseconds, and a 20-step run (14 ms) would otherwise be timed on the ramp")
    ap.add_argument("--no-rewire-costs", action="store_true", help="skip the plan-build / first-backward-after-rewiring timings")
    ap.add_argument("--sweep", nargs="?", const="all", default=None, choices=["all", "reference", "layer", "layer_k64"],
                    help="instead of the benchmark line: batch x width x labels x fan-in grids of the passes, one CSV line per "
                         "timing (file: --sweep-csv): 'reference' = the grid of the reference's testing/detailed-bench.cpp:26-112, "
                         "'layer' = the same axes around the headline workload, each pass also with the library's kernel choices overridden")
    ap.add_argument("--sweep-csv", default="sweep.csv", help="where --sweep writes its timings (relative to this file)")
    ap.add_argument("--copy-bytes", type=int, default=0,
                    help="also run one plain device copy kernel of this many bytes (read N, write N): the "
                         "known-size reference that rocprofv3 FETCH_SIZE/WRITE_SIZE readings are scaled by")
    return ap.parse_args()


def time_kernel(fn, stream, iters):
    """Average duration (ms) of `fn`, HIP events recorded on the stream the kernels run on."""
    import torch
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    # untimed calls first, with no host wait between them and the timed ones: the GPU's clocks take tens of
    # milliseconds of continuous load to settle, and a pass timed from idle reads 3-8 % slow
    for _ in range(max(1, iters // 4)):
        fn()
    start.record(stream)
    for _ in range(iters):
        fn()
    stop.record(stream)
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def cpu_baseline(cfg, layout_tp, arrays):
    """Times the CPU oracle (restatement of the reference's CPU kernels) on a bounded sample: `arrays` are the first
    labels of the very tensors the GPU leg runs on.  Returns the report and the oracle's three results."""
    import oracle

    threads = oracle.default_threads()
    x, lookup, w, g = arrays
    labels = lookup.shape[0]
    oracle.forward(x[:, :], lookup[:1024], w[:1024], transposed=layout_tp, threads=threads)   # warm-up
    best, results = None, None
    for _ in range(2):
        t0 = time.perf_counter()
        out = oracle.forward(x, lookup, w, transposed=layout_tp, threads=threads)
        gw = oracle.weight_grad(x, lookup, w, g, transposed=layout_tp, threads=threads)
        gx = oracle.input_grad(x, lookup, w, g, transposed=layout_tp, threads=threads)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
        results = (out, gx, gw)
    full_time = best * cfg.num_units / labels        # every pass is linear in the label count
    report = {
        "value": cfg.batch / full_time,
        "unit": "samples/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{labels} of {cfg.num_units} labels (same B, N, K, same tensors as the GPU leg); fwd+gW+gx in {best:.3f} s (best of 2)"
                  + ("" if labels == cfg.num_units else ", scaled linearly to the full label count"),
    }
    return report, results


def rel_err(a, ref):
    import numpy as np
    denom = float(np.abs(ref).max())
    return float(np.abs(a.astype(np.float64) - ref).max() / (denom if denom > 0 else 1.0))


def parity_check(pkg, arrays, tp, stream, reference=None):
    """The three passes on a label sample of the workload's own tensors, HIP path against the CPU oracle, before any
    timing: forward max|a-b|/max|ref| <= 1e-5, gradients <= 1e-4 (the gates of the parity tests)."""
    import numpy as np
    import oracle
    import torch

    x, lookup, w, g = arrays
    if reference is None:
        reference = (oracle.forward(x, lookup, w, transposed=tp), oracle.input_grad(x, lookup, w, g, transposed=tp),
                     oracle.weight_grad(x, lookup, w, g, transposed=tp))
    L, K = lookup.shape
    B = g.shape[0]
    N = x.shape[0] if tp else x.shape[1]
    dx, dl, dw, dg = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (x, lookup, w, g))
    out = torch.full((B, L), float("nan"), device="cuda")
    gx, gw = torch.full_like(dx, float("nan")), torch.full_like(dw, float("nan"))
    lib, check, sh = pkg._lib.lib(), pkg._lib.check, stream.cuda_stream
    check(lib.ffi_forward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), out.data_ptr(), B, N, L, K, int(tp), sh))
    check(lib.ffi_backward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx.data_ptr(), gw.data_ptr(), B, N, L, K, int(tp), sh))
    stream.synchronize()
    errs = {"forward": rel_err(out.cpu().numpy(), reference[0]), "input_grad": rel_err(gx.cpu().numpy(), reference[1]),
            "weight_grad": rel_err(gw.cpu().numpy(), reference[2])}
    gates = {"forward": 1e-5, "input_grad": 1e-4, "weight_grad": 1e-4}
    ok = all(errs[k] <= gates[k] for k in gates)
    return {"checked_before_timing": True, "labels": int(L), "against": "CPU oracle (oracle/ffi_oracle.c)",
            "rel_err": {k: float(f"{v:.3e}") for k, v in errs.items()}, "gates": gates, "pass": bool(ok)}


def bench_inference(args, pkg, synth, cfg):
    """c5: bf16 features and weights, fp32 accumulation, top-5 per sample without the score matrix."""
    import numpy as np
    import oracle
    import torch

    t = synth.make_inputs(cfg, seed=args.seed, device="cuda", transposed=True)
    x, lookup, w = t["features"].to(torch.bfloat16), t["lookup"], t["weights"].to(torch.bfloat16)
    B, N, L, K = cfg.batch, cfg.num_features, cfg.num_units, cfg.fan_in
    lib, check = pkg._lib.lib(), pkg._lib.check
    stream = torch.cuda.current_stream()
    sh = stream.cuda_stream
    vals = torch.empty((B, 5), device="cuda")
    labels = torch.empty((B, 5), dtype=torch.int32, device="cuda")

    def step():
        check(lib.ffi_forward_topk_bf16(x.data_ptr(), lookup.data_ptr(), w.data_ptr(), vals.data_ptr(), labels.data_ptr(),
                                        B, N, L, K, 5, 1, sh))

    # parity before timing: the top-5 of 8 samples against the oracle's top-5 of fp32 scores of the same bf16-rounded inputs
    step()
    stream.synchronize()
    rows = 8
    xs = x[:, :rows].float().cpu().numpy()
    ref = oracle.forward(np.ascontiguousarray(xs), lookup.cpu().numpy(), w.float().cpu().numpy(), transposed=True)
    ref_v, ref_i = oracle.topk(ref, 5)
    got_v, got_i = vals[:rows].cpu().numpy(), labels[:rows].cpu().numpy()
    same_labels = float((got_i == ref_i).mean())
    parity = {"checked_before_timing": True, "samples": rows, "against": "CPU oracle on the same bf16-rounded inputs",
              "rel_err": {"top5_scores": float(f"{rel_err(got_v, ref_v):.3e}")}, "gates": {"top5_scores": 1e-2},
              "top5_labels_equal": same_labels, "pass": bool(rel_err(got_v, ref_v) <= 1e-2)}
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kernel_ms = time_kernel(step, stream, max(3, min(args.steps, 20)))
    alg = 2 * L * K + 4 * L * K + 2 * B * N                  # bf16 W, int32 idx, bf16 x; the scores are never written
    achieved = alg / (kernel_ms * 1e-3) / 1e9
    traffic, source = measured_traffic(cfg.name)
    return {
        "metric": "ffi_bf16_fwd_top5_samples_per_s", "value": round(B / (ms * 1e-3), 1), "unit": "samples/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{cfg.name}: FFI layer forward + top-5 per sample, bf16 features and weights with fp32 accumulation, "
                               f"batch {B}, {N} inputs, {L} labels, fan-in {K} (sorted rows), features [N,B]"},
        "roofline": {"bound": "hbm", "kernel": "forward pass (fwd_bf16_topk_kernel + topk_merge_kernel)", "achieved": round(achieved, 2),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic.get("forward"), "traffic_source": source, "algorithmic_bytes": alg,
                     "kernel_ms": {"forward": round(kernel_ms, 4)},
                     "note": f"the gathers (B*L*K*2 = {B * L * K * 2 / 1e9:.1f} GB per call) are served by L2 / Infinity Cache, which is what bounds this workload"},
        "parity": parity,
        "library_bytes": int(lib.ffi_cache_bytes()),
    }


def train_step(pkg, cfg, x, lookup, w, tp, density, stream, iters):
    """One training step as the reference's loop runs it (sparse/optimizer.py:43-66): forward + loss,
    backward, Adam on weights and bias, with synthetic labels (5 per sample) and the bias chosen so that
    `density` of the squared-hinge gradients are non-zero (late in training nearly every margin is met)."""
    import ctypes

    import torch
    B, N, L, K = cfg.batch, cfg.num_features, cfg.num_units, cfg.fan_in
    lib, check, sh = pkg._lib.lib(), pkg._lib.check, stream.cuda_stream
    ptr = lambda a: a.data_ptr()  # noqa: E731
    gen = torch.Generator(device="cuda").manual_seed(7)
    scores = torch.empty((B, L), device="cuda")
    check(lib.ffi_forward_f32(ptr(x), ptr(lookup), ptr(w), ptr(scores), B, N, L, K, int(tp), sh))
    # a negative's gradient is non-zero where 1 + score + bias > 0
    sample = scores.flatten()[torch.randint(0, B * L, (1 << 20,), device="cuda", generator=gen)]
    bias = torch.full((L,), -1.0 - float(torch.quantile(sample, 1.0 - density)), device="cuda")
    rows = torch.arange(B, device="cuda").repeat_interleave(5)
    labels = torch.stack([rows, torch.randint(0, L, (B * 5,), device="cuda", generator=gen)], dim=1).contiguous()
    g = torch.empty_like(scores)
    masks = torch.empty(((B + 31) // 32, L), dtype=torch.int32, device="cuda")
    loss = torch.empty(1, device="cuda")
    gx, gw, gb = torch.empty_like(x), torch.empty_like(w), torch.empty_like(bias)
    mw, vw, mb, vb = torch.zeros_like(w), torch.zeros_like(w), torch.zeros_like(bias), torch.zeros_like(bias)
    w2, bias2 = w.clone(), bias.clone()              # Adam runs on copies: every timed step sees the same scores
    scale = ctypes.c_float(1.0 / (B * L))
    taken = ctypes.c_int(-1)
    SQH, SKIP = 2, 0x100      # squared hinge; zero gradients are not stored (the masks say where out_grad is valid)

    def fused_forward_loss():
        check(lib.ffi_forward_loss_f32(ptr(x), ptr(lookup), ptr(w), ptr(bias), ptr(labels), None, labels.shape[0], SQH | SKIP, scale,
                                       None, ptr(g), ptr(loss), ptr(masks), B, N, L, K, int(tp), sh))

    tv, ti = torch.empty((B, 5), device="cuda"), torch.empty((B, 5), dtype=torch.int32, device="cuda")

    def fused_forward_loss_topk():
        # the same pass with the top-5 of the scores as a by-product (what P@1/3/5 need), still without the score matrix
        check(lib.ffi_forward_loss_topk_f32(ptr(x), ptr(lookup), ptr(w), ptr(bias), ptr(labels), None, labels.shape[0], SQH | SKIP,
                                            scale, None, ptr(g), ptr(loss), ptr(masks), ptr(tv), ptr(ti), 5, B, N, L, K, int(tp), sh))

    def backward_sparse():
        check(lib.ffi_backward_sparse_f32(ptr(x), ptr(lookup), ptr(w), ptr(g), ptr(masks), 1, ctypes.c_float(0.0), ptr(gx), ptr(gw),
                                          ptr(gb), ctypes.byref(taken), B, N, L, K, int(tp), sh))

    def adam():
        check(lib.ffi_adam_step_f32(ptr(w2), ptr(mw), ptr(vw), ptr(gw), L * K, 1e-3, 0.9, 0.999, 1e-7, 1, sh))
        check(lib.ffi_adam_step_f32(ptr(bias2), ptr(mb), ptr(vb), ptr(gb), L, 1e-3, 0.9, 0.999, 1e-7, 1, sh))

    def unfused_forward_loss():
        check(lib.ffi_forward_bias_f32(ptr(x), ptr(lookup), ptr(w), ptr(bias), ptr(scores), B, N, L, K, int(tp), sh))
        check(lib.ffi_loss_grad_f32(ptr(scores), ptr(labels), None, labels.shape[0], SQH, scale, ptr(g), ptr(loss), None, B, L, sh))

    def backward_dense():
        check(lib.ffi_backward_bias_f32(ptr(x), ptr(lookup), ptr(w), ptr(g), ptr(gx), ptr(gw), ptr(gb), B, N, L, K, int(tp), sh))

    def backward_adam():
        # learning rate 0: all the memory traffic and arithmetic of the step, and the same scores in every timed pass;
        # flags: out_grad is valid at the masks' set bits only (1), kernels chosen from the previous call's count (2)
        check(lib.ffi_backward_sparse_adam_f32(ptr(x), ptr(lookup), ptr(w), ptr(g), ptr(masks), 1 | 2, ctypes.c_float(0.0), ptr(gx),
                                               ptr(mw), ptr(vw), ptr(bias), ptr(mb), ptr(vb), 0.0, 0.9, 0.999, 1e-7, 1,
                                               ctypes.byref(taken), B, N, L, K, int(tp), sh))

    def whole():
        fused_forward_loss()
        backward_adam()

    out = {"loss": "squared hinge, 5 labels per sample", "target_density": density}
    out["forward_loss_ms"] = round(time_kernel(fused_forward_loss, stream, iters), 4)
    g.zero_()
    fused_forward_loss()
    out["forward_loss_top5_ms"] = round(time_kernel(fused_forward_loss_topk, stream, iters), 4)
    out["gradient_density"] = round(float((g != 0).float().mean()), 6)
    out["backward_sparse_ms"] = round(time_kernel(backward_sparse, stream, iters), 4)
    out["sparse_kernels_ran"] = bool(taken.value)
    out["adam_ms"] = round(time_kernel(adam, stream, iters), 4)
    out["backward_sparse_with_adam_ms"] = round(time_kernel(backward_adam, stream, iters), 4)
    out["step_ms"] = round(time_kernel(whole, stream, iters), 4)
    out["samples_per_s"] = round(B / (out["step_ms"] * 1e-3), 1)
    # rewiring (every rewire_interval steps in the reference): threshold of the 1 % smallest magnitudes, redraw of
    # their sources, moments cleared -- on a copy of the index matrix, so the layer above is left as it is
    lookup2 = lookup.clone()
    thr = torch.empty(1, device="cuda")
    arrays = (ctypes.c_void_p * 2)(ptr(mw), ptr(vw))

    def rewire():
        check(lib.ffi_select_threshold_f32(ptr(w), L * K, (L * K) // 100, ptr(thr), sh))
        check(lib.ffi_rewire_f32(ptr(lookup2), ptr(w), arrays, 2, L * K, N, ptr(thr), 12345, None, sh))

    out["rewire_1pct_ms"] = round(time_kernel(rewire, stream, iters), 4)
    # the same step through the PyTorch binding: the fused loss as an autograd function, loss.backward() (the
    # upstream factor arrives as a device scalar), gradients left in .grad; no optimizer
    x_a, w_a, b_a = x.clone().requires_grad_(True), w.clone().requires_grad_(True), bias.clone().requires_grad_(True)
    loss_fn, y_true = pkg.SparseSquaredHingeLoss(), (labels, None)

    def autograd_step():
        x_a.grad = w_a.grad = b_a.grad = None
        loss_fn.fused(x_a, lookup, w_a, b_a, y_true, transposed=tp)[0].backward()

    out["autograd_forward_loss_backward_ms"] = round(time_kernel(autograd_step, stream, iters), 4)

    def c_abi_step():
        fused_forward_loss()
        check(lib.ffi_backward_sparse_f32(ptr(x), ptr(lookup), ptr(w), ptr(g), ptr(masks), 1 | 2, ctypes.c_float(0.0), ptr(gx), ptr(gw),
                                          ptr(gb), ctypes.byref(taken), B, N, L, K, int(tp), sh))

    out["c_abi_forward_loss_backward_ms"] = round(time_kernel(c_abi_step, stream, iters), 4)
    out["unfused_dense_route_ms"] = {"forward_bias+loss_grad": round(time_kernel(unfused_forward_loss, stream, iters), 4),
                                     "backward_dense": round(time_kernel(backward_dense, stream, iters), 4)}
    return out


# Points of --sweep.  "reference": the grid of the reference's testing/detailed-bench.cpp:26-112 (forward pass, both
# feature layouts, one axis varied around batch 32 / 32,768 inputs / 670,000 labels / fan-in 32).  "layer": the same
# four axes around the headline workload, whose narrow input takes the LDS-tile kernels: all three passes, and each
# pass also with the library's choices overridden (ffi_set_option), which is what re-checks those choices.
SWEEP_GRIDS = {
    "reference": {"base": (32, 32768, 670000, 32), "passes": ("forward",), "layouts": ("bn", "nb"), "distinct": False,
                  "axes": {"batch": [4, 8, 10, 16, 25, 32, 50, 64, 100],
                           "num_features": [768, 1024, 2048, 4096, 8192, 16384, 24576, 32768, 49152, 65536],
                           "num_units": [4000, 10000, 32000, 64000, 100000, 256000, 670000, 1000000],
                           "fan_in": [4, 8, 12, 16, 24, 32, 40, 48, 64, 80, 96, 128]}},
    "layer": {"base": (128, 768, 670091, 32), "passes": ("forward", "weight_grad", "input_grad"), "layouts": ("nb",), "distinct": True,
              "axes": {"batch": [32, 64, 96, 128, 160, 256, 512],
                       "num_features": [64, 128, 256, 384, 512, 608, 640, 768, 1024, 1216],
                       "num_units": [4000, 32000, 131072, 262144, 393216, 524288, 670091, 1000000, 3000000],
                       "fan_in": [8, 16, 32, 64, 96, 128]}},
}
# (the second narrow workload of the benchmark set: 64 connections per label = two chunks per label, 512 columns)
SWEEP_GRIDS["layer_k64"] = dict(SWEEP_GRIDS["layer"], base=(256, 512, 501070, 64),
                                axes={"batch": [64, 128, 256, 512], "num_features": [256, 512, 608, 768],
                                      "num_units": [131072, 501070, 1000000], "fan_in": [48, 64, 128]})
SWEEP_VARIANTS = {
    "forward": [("fwd_lane64", -1)],
    "weight_grad": [("wgrad_units", 3), ("wgrad_units", 4), ("wgrad_stream", -1)],
    "input_grad": [("plan_weights_in_lds", -1), ("plan_weights_in_lds", 1), ("workgroups_per_cu", 1), ("plan_sorted_columns", -1), ("plan_sorted_columns", 1)],
}


def sweep(args, pkg, synth):
    """Times the passes over SWEEP_GRIDS and writes one CSV line per (point, layout, pass, variant) to
    the file named by --sweep-csv; prints one JSON line that lists where an override beat the library's own choice."""
    import csv
    import ctypes

    import torch
    lib, check = pkg._lib.lib(), pkg._lib.check
    stream = torch.cuda.current_stream()
    sh = stream.cuda_stream
    ptr = lambda a: a.data_ptr()  # noqa: E731
    path = os.path.join(ROOT, args.sweep_csv)
    os.makedirs(os.path.dirname(path) or ".", exist_ok=True)
    rows, beaten, points = [], [], 0
    names = ("batch", "num_features", "num_units", "fan_in")
    grids = [g for g in SWEEP_GRIDS if args.sweep in ("all", g)]
    for grid in grids:
        spec = SWEEP_GRIDS[grid]
        seen = set()
        for axis, values in spec["axes"].items():
            for v in values:
                dims = list(spec["base"])
                dims[names.index(axis)] = v
                B, N, L, K = dims
                if (B, N, L, K) in seen and axis != "batch":
                    continue                      # the base point is on every axis: timed once
                seen.add((B, N, L, K))
                points += 1
                gen = torch.Generator(device="cuda").manual_seed(args.seed)
                lookup = synth.make_lookup(L, K, N, distinct=spec["distinct"], generator=gen, device="cuda")
                w = torch.randn((L, K), generator=gen, device="cuda") * K ** -0.5
                g = torch.randn((B, L), generator=gen, device="cuda") * 0.1
                out, gw = torch.empty_like(g), torch.empty_like(w)
                for layout in spec["layouts"]:
                    tp = layout == "nb"
                    x = torch.relu(torch.randn((N, B) if tp else (B, N), generator=gen, device="cuda"))
                    gx = torch.empty_like(x)
                    plan = ctypes.c_void_p()
                    iters = max(3, min(30, int(2.0e10 / (B * L * K))))

                    def settled(fn):
                        # 25 ms of the same kernel in front of the timed launches: the clocks follow the load
                        t0 = time.perf_counter()
                        while time.perf_counter() - t0 < 0.025:
                            for _ in range(iters):
                                fn()
                            torch.cuda.synchronize()
                        return time_kernel(fn, stream, iters)

                    def timed(name):
                        # the gradient passes through an explicit plan (built under the options in force), created here
                        # and destroyed after the timing
                        if name == "forward":
                            return settled(lambda: check(lib.ffi_forward_f32(ptr(x), ptr(lookup), ptr(w), ptr(out), B, N, L, K, int(tp), sh)))
                        check(lib.ffi_plan_create(ptr(lookup), L, K, N, B, sh, ctypes.byref(plan)))
                        if name == "weight_grad":
                            ms = settled(lambda: check(lib.ffi_weight_grad_planned_f32(plan, ptr(x), ptr(lookup), ptr(g), ptr(gw), B, int(tp), sh)))
                        else:
                            ms = settled(lambda: check(lib.ffi_input_grad_planned_f32(plan, ptr(w), ptr(g), ptr(gx), B, int(tp), sh)))
                        check(lib.ffi_plan_destroy(plan))
                        return ms

                    for name in spec["passes"]:
                        narrow = grid != "reference"
                        variants = [("auto", 0)] + (SWEEP_VARIANTS[name] if narrow else [])
                        # two rounds over the variants, the smaller time of each: the clocks drift by several percent
                        # with the load of the preceding milliseconds, in both directions
                        results = {}
                        for _ in range(2 if narrow else 1):
                            for option, value in variants:
                                if value:
                                    check(lib.ffi_set_option(option.encode(), value))
                                ms = timed(name)
                                if value:
                                    check(lib.ffi_set_option(option.encode(), 0))
                                label = option if not value else f"{option}={value}"
                                results[label] = min(ms, results.get(label, ms))
                        for label, ms in results.items():
                            rows.append([grid, axis, B, N, L, K, layout, name, label, f"{ms:.5f}"])
                            if label != "auto" and ms < 0.97 * results["auto"]:
                                beaten.append({"point": [B, N, L, K], "pass": name, "override": label,
                                               "auto_ms": round(results["auto"], 4), "override_ms": round(ms, 4)})
                    del x, gx
                del lookup, w, g, out, gw
                check(lib.ffi_cache_clear())
                torch.cuda.empty_cache()
                print(f"sweep: {grid} {axis}={v} done", file=sys.stderr, flush=True)
    with open(path, "w", newline="") as f:
        wr = csv.writer(f)
        wr.writerow(["grid", "axis", "batch", "num_features", "num_units", "fan_in", "layout", "pass", "variant", "ms"])
        wr.writerows(rows)
    print(json.dumps({"sweep": grids, "points": points, "timings": len(rows), "csv": os.path.relpath(path, ROOT),
                      "overrides_faster_than_the_library_by_3_percent": beaten}))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus above 1 is not supported "
              "(across GPUs the layer would shard by label: each GPU its own labels, one all-reduce of the input gradient)", file=sys.stderr)
        sys.exit(2)

    import importlib

    import torch

    pkg = importlib.import_module("ecml23-sparse_amd")
    from ecml23_sparse_amd import synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    if args.copy_bytes:
        # the process's first elementwise multiply kernel: reads N bytes, writes N bytes
        src = torch.empty(args.copy_bytes // 4, dtype=torch.float32, device="cuda").fill_(1.0)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
    if args.sweep:
        sweep(args, pkg, synth)
        return
    cfg = synth.CONFIGS[args.config]
    if cfg.name == "c5":
        print(json.dumps(bench_inference(args, pkg, synth, cfg)))
        return
    tp = args.layout == "nb"
    t = synth.make_inputs(cfg, seed=args.seed, device="cuda", transposed=tp)
    x, lookup, w, g = t["features"], t["lookup"], t["weights"], t["out_grad"]
    B, N, L, K = cfg.batch, cfg.num_features, cfg.num_units, cfg.fan_in
    if args.arranged:
        pkg.arrange_connections(lookup, w)
    # Parity first, outside the timed region: the HIP path against the CPU oracle on the first labels of these very
    # tensors (all of them when the CPU baseline's time budget allows: then the input gradient is the full one).
    # The oracle's run is also the CPU baseline.
    labels = min(L, args.cpu_labels or max(4096, int(8.0e9 / (B * K))))
    if args.no_cpu_baseline:
        labels = min(L, args.cpu_labels or 8192)
    sample = (x.cpu().numpy(), lookup[:labels].cpu().numpy(), w[:labels].cpu().numpy(),
              g[:, :labels].contiguous().cpu().numpy())
    cpu_report, cpu_results = (None, None) if args.no_cpu_baseline else cpu_baseline(cfg, tp, sample)
    parity = parity_check(pkg, sample, tp, torch.cuda.current_stream(), cpu_results)
    del sample, cpu_results
    if not parity["pass"]:
        print(f"bench.py: parity check failed, nothing is timed: {json.dumps(parity)}", file=sys.stderr)
        sys.exit(4)
    pkg._lib.lib().ffi_cache_clear()
    out = torch.empty((B, L), device="cuda")
    gx = torch.empty_like(x)
    gw = torch.empty_like(w)
    lib = pkg._lib.lib()
    check = pkg._lib.check
    stream = torch.cuda.current_stream()
    sh = stream.cuda_stream
    ptr = lambda a: a.data_ptr()  # noqa: E731

    def step():
        check(lib.ffi_forward_f32(ptr(x), ptr(lookup), ptr(w), ptr(out), B, N, L, K, int(tp), sh))
        check(lib.ffi_backward_f32(ptr(x), ptr(lookup), ptr(w), ptr(g), ptr(gx), ptr(gw), B, N, L, K, int(tp), sh))

    # untimed pre-load: steps until the GPU has been busy for --preload-ms (its clocks settle under load)
    preload_steps, t_pre = 0, time.perf_counter()
    while (time.perf_counter() - t_pre) * 1e3 < args.preload_ms:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
        preload_steps += 10
    preload_ms = (time.perf_counter() - t_pre) * 1e3
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    # spread of single steps, outside the timed region (an event between two steps costs a few microseconds)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    marks[0].record(stream)
    for i in range(args.steps):
        step()
        marks[i + 1].record(stream)
    marks[-1].synchronize()
    singles = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    step_spread = {"min": round(singles[0], 4), "median": round(singles[len(singles) // 2], 4), "max": round(singles[-1], 4),
                   "note": "per-step event timing in a second loop of the same length (includes the event records)"}

    # per-kernel durations with events on the launch stream (explicit plan: the kernel alone)
    import ctypes
    plan = ctypes.c_void_p()
    check(lib.ffi_plan_create(ptr(lookup), L, K, N, B, sh, ctypes.byref(plan)))
    iters = max(3, min(args.steps, 20))
    kernels = {
        "forward": lambda: check(lib.ffi_forward_f32(ptr(x), ptr(lookup), ptr(w), ptr(out), B, N, L, K, int(tp), sh)),
        "weight_grad": lambda: check(lib.ffi_weight_grad_planned_f32(plan, ptr(x), ptr(lookup), ptr(g), ptr(gw), B, int(tp), sh)),
        "input_grad": lambda: check(lib.ffi_input_grad_planned_f32(plan, ptr(w), ptr(g), ptr(gx), B, int(tp), sh)),
    }
    back_to_back_ms = {name: time_kernel(fn, stream, iters) for name, fn in kernels.items()}
    # What a pass costs inside a step: the three launches in the order of a step, timed as whole rounds with all three
    # and with one of them left out; a pass's figure is the difference per round.  (No event inside a round: a record
    # between two kernels opens a gap of several microseconds; and a pass launched back to back follows its own stores
    # instead of the pass it follows in a step, which the forward pass in particular feels.)
    order = ("forward", "weight_grad", "input_grad")
    rounds = max(20, min(args.steps, 100))

    def rounds_ms(names):
        for _ in range(5):
            for name in names:
                kernels[name]()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(stream)
        for _ in range(rounds):
            for name in names:
                kernels[name]()
        b.record(stream)
        b.synchronize()
        return a.elapsed_time(b) / rounds

    whole, without = [], {}
    for left_out in order:
        whole.append(rounds_ms(order))
        without[left_out] = rounds_ms(tuple(n for n in order if n != left_out))
    whole.append(rounds_ms(order))
    whole_ms = sum(whole) / len(whole)
    kernel_ms = {name: whole_ms - without[name] for name in order}
    plan_info = (ctypes.c_int64 * 8)()
    check(lib.ffi_plan_info(plan, plan_info))
    check(lib.ffi_plan_destroy(plan))
    alg = synth.algorithmic_bytes(cfg)
    dominant = max(kernel_ms, key=kernel_ms.get)
    achieved = alg[dominant] / (kernel_ms[dominant] * 1e-3) / 1e9
    traffic, traffic_source = measured_traffic(cfg.name)
    narrow = N <= 1216
    pass_kernels = dict(PASS_KERNELS if narrow else WIDE_PASS_KERNELS)
    if N <= 608 and B > 32 and (B >= 192 or (K >= 64 and B >= 128) or (K > 32 and K % 32 != 0 and K % 16 == 0)):
        pass_kernels["forward"] = "fwd_lane64_kernel"       # batch tiles of 64 where the [N][64] tile fits in LDS and pays
    if narrow and plan_info[0] and plan_info[1]:
        # the plan's tiles are small enough for the walking kernel to keep the tile's weights in LDS: no permutation kernel
        pass_kernels["input_grad"] = "igrad_tile_kernel + igrad_reduce_kernel"
    if narrow and not (N * 128 + 65536 <= 160 * 1024 and L >= 64):
        pass_kernels["weight_grad"] = "wgrad_arranged_kernel"        # no room for the out_grad slices behind the tile of x
    flops = 2.0 * B * L * K
    roofline = {
        "bound": "hbm",
        "kernel": f"{dominant} pass ({pass_kernels[dominant]})",
        "achieved": round(achieved, 2),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4),
        "traffic": traffic.get(dominant),
        "traffic_source": traffic_source,
        "algorithmic_bytes": alg[dominant],
        "kernel_ms": {k: round(v, 4) for k, v in kernel_ms.items()},
        "kernel_ms_note": f"cost of each pass inside a round of the three passes in step order: {rounds} rounds with all three minus {rounds} rounds "
                          f"without it, HIP events around the {rounds} rounds (whole round {whole_ms:.4f} ms)",
        "kernel_ms_back_to_back": {k: round(v, 4) for k, v in back_to_back_ms.items()},
        "all_kernels_gbps": {k: round(alg[k] / (v * 1e-3) / 1e9, 1) for k, v in kernel_ms.items()},
        "three_pass_gbps": round(alg["total"] / (sum(kernel_ms.values()) * 1e-3) / 1e9, 1),
        # what one pass cannot go below on the two other resources it uses for every multiply-add (published peaks):
        # 4 bytes of LDS reads (narrow inputs: the gathered operand is staged in LDS) and one plain FP32 FMA
        "other_floors_ms_per_pass": {"lds_gather": round(4.0 * B * L * K / (LDS_PEAK_GBPS * 1e9) * 1e3, 4) if narrow else None,
                                     "fp32_fma_unpacked": round(flops / (FP32_FMA_PEAK_TFLOPS * 1e12) * 1e3, 4),
                                     "hbm": round(alg[dominant] / (HBM_PEAK_GBPS * 1e9) * 1e3, 4)},
    }

    result = {
        "metric": "ffi_fwd_bwd_samples_per_s",
        "value": round(B / (ms_per_step * 1e-3), 1),
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{cfg.name}: FFI layer fwd+input-grad+weight-grad, batch {B}, {N} inputs, "
                               f"{L} labels, fan-in {K}, features [{'N,B' if tp else 'B,N'}]"
                               + (", connections of each label reordered by ffi_arrange_connections_f32" if args.arranged else ""),
                   "label_samples_per_s": round(B * L / (ms_per_step * 1e-3), 1)},
        "preload_ms": round(preload_ms, 1),
        "preload_steps": preload_steps,
        "step_ms": step_spread,
        "roofline": roofline,
        "attainable": attainable(cfg, alg, cfg.name) if narrow else None,
        "parity": parity,
        # device memory the library holds beside the caller's tensors after these steps (cached plan + workspaces),
        # and what ffi_workspace_bytes() predicts for this shape
        "library_bytes": int(lib.ffi_cache_bytes()),
        "library_bytes_estimate": int(lib.ffi_workspace_bytes(B, N, L, K, int(tp), 3)),
        "plan": {"tiled": bool(plan_info[0]), "weights_in_lds": bool(plan_info[1]), "tile_labels": int(plan_info[2]), "tiles": int(plan_info[4]),
                 "slots_per_connection": round(plan_info[5] * 64 / (L * K), 4) if plan_info[0] else None, "bytes": int(plan_info[6])},
    }
    if narrow and not args.no_rewire_costs:
        result["rewiring"] = rewire_costs(pkg, cfg, x, lookup, w, g, tp, stream)
    if args.train_step > 0:
        result["train_step"] = train_step(pkg, cfg, x, lookup, w, tp, args.train_step, stream, max(3, min(args.steps, 20)))
    if cpu_report is not None:
        result["cpu_baseline"] = cpu_report
    print(json.dumps(result))


if __name__ == "__main__":
    main()
