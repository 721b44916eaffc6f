#!/usr/bin/env python3
"""Benchmark of the MatrixFSDP hot path on one MI355X.

``python bench.py --gpus 1 --steps K --warmup W`` prints ONE JSON line.

A *step* is one pass of the flat-buffer copy path over the hidden4096
workload: for each of the 32 layer buffers (Wqkv 12288x4096, Wo 4096x4096,
W1/W3 11008x4096, W2 4096x11008, two 4096 norm vectors; bf16; 2x2
block-sharded for a simulated world of 4) one *pack* launch (full buffer ->
padded all-gather buffer, every rank's strided block) and one *unpack* launch
(gathered buffer -> full buffer).  ``value`` is the algorithmic bytes of those
64 launches (2 B read + 2 B written per element, each way) over the wall time
of the step, inputs resident in HBM.

After the timed region the same run measures, with their own clocks and
reported under ``legs``: the hidden2048 row-split workload (pack, unpack,
gradient chunk-cat with bf16->fp32 cast), the owner-rank Muon update of the
three hidden4096 matrices (ms/step and Newton-Schulz TFLOP/s by the
reference's full-GEMM flop count) and fused AdamW.  The CPU baselines time the
CPU oracle (a port of the reference's per-segment slice-copy loops and of
``torch.optim.Muon``) on a bounded sample on this host's cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E, vendor figure
BF16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, vendor figure
NS_COEFFS = (3.4445, -4.7750, 2.0315)
# Figures QUOTED from the committed rocprofv3 counter profiles (counters cannot be read from inside this process).  They
# describe the library as it was when the profile was taken (its `head` line) and are reported under keys that say so.
PROFILED_TRAFFIC = {"bytes_per_launch": 812_818_425, "source": "profiles/segment_program_hbm_traffic.md"}
PROFILED_MUON = {
    # SQ_VALU_MFMA_BUSY_CYCLES over the SIMD cycles of the dispatch (all 256 CUs), per kernel and launch shape
    "mfma_busy": {
        "gemm_nt_kernel<256,256> general product, 768 workgroups (12288x4096)": 0.565,
        "gemm_nt_kernel<256,256> general product, 688 workgroups (11008x4096)": 0.508,
        "gemm_nt_kernel<256,256> general product, 256 workgroups (4096x4096)": 0.597,
        "gemm_nt_kernel<128,128> symmetric products, one matrix at a time, 768 workgroups": 0.470,
    },
    # the dominant launch, B X on 12288 x 4096 (768 workgroups): FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, in bytes
    "traffic_bytes_per_launch": (2 * 295_250 + 176_947) * 1024,
    "source": "profiles/gemm_nt_kernel_muon_hidden4096_counters.md, profiles/gemm_nt_kernel_muon_hbm_traffic.md",
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=0, help="layer buffers of the hidden4096 workload (0 = all 32)")
    ap.add_argument("--skip-legs", action="store_true", help="only the timed pack/unpack region (used under rocprofv3)")
    ap.add_argument("--skip-mixed", action="store_true", help="skip the hidden5120 mixed-step leg")
    ap.add_argument("--legs", default="ceiling,rows,devcopy,gemm,muon,adamw,mixed",
                    help="comma list of the extra legs to run: ceiling (plain copy / read-only / write-only probes), rows (hidden2048 row split), "
                    "devcopy (the device-metadata rank-segment copy, the reference extension's own entry point), gemm (one plain 8192^3 product beside "
                    "the library's), muon, adamw, mixed")
    ap.add_argument("--muon-form", default="both", choices=("both", "serial", "side-by-side"),
                    help="which form of the Muon leg to run: one matrix at a time on the calling stream, the three side by side on side streams, "
                    "or both (serial alone makes every kernel of a rocprofv3 trace run by itself)")
    ap.add_argument("--skip-cpu", action="store_true", help="do not time the CPU baselines")
    ap.add_argument("--hold-muon-seconds", type=float, default=0.0,
                    help="after the Muon leg, keep stepping for this long (for sampling the clock beside it); reports the rate of that stretch")
    ap.add_argument("--no-launch-events", action="store_true", help="no HIP events inside the timed region (launch time from the wall clock)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain Tensor.copy_ of 1 GiB (a copy kernel of known size, to scale rocprofv3's FETCH_SIZE / WRITE_SIZE)")
    return ap.parse_args()


def median(values):
    values = sorted(values)
    return values[len(values) // 2]


def event_pair(torch):
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def time_launches(torch, fn, iters, warmup):
    """Median and mean device time of ``fn`` (HIP events on the current stream)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    pairs = [event_pair(torch) for _ in range(iters)]
    for a, b in pairs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    times = [a.elapsed_time(b) for a, b in pairs]
    return median(times), sum(times) / len(times)


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(
            "bench.py measures the per-rank hot path on ONE GPU (the world of size W is simulated in memory, no "
            f"collectives are issued); --gpus {args.gpus} is not supported.",
            file=sys.stderr,
        )
        return 2

    import torch

    import matrix_fsdp_amd  # noqa: F401
    from matrix_fsdp_amd import _lib
    from matrix_fsdp_amd.kernels.segment_program import grad_fill_program, pack_program, unpack_program
    from matrix_fsdp_amd.optim import functional as F
    from matrix_fsdp_amd.workloads import HIDDEN2048_W4, HIDDEN4096_W4_BLOCK, HIDDEN5120, HIDDEN5120_TAIL_NUMEL, MUON_HIDDEN4096_SHAPES, MUON_SEED

    if not torch.cuda.is_available():
        print("bench.py needs a HIP device.", file=sys.stderr)
        return 2
    _lib.lib()  # fail loudly when the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    host_cores = os.cpu_count() or 1
    host_threads = min(host_cores, 16)  # torch's CPU kernels stop scaling beyond that on these copies
    torch.set_num_threads(host_threads)

    # ------------------------------------------------------------------ timed region: hidden4096 2x2 block pack + unpack
    w = HIDDEN4096_W4_BLOCK
    layers = args.layers or w.layers
    plan = w.plan()
    pack = pack_program(plan, torch.bfloat16, device=dev)
    unpack = unpack_program(plan, torch.bfloat16, device=dev)
    padded_numel = w.world_size * plan.max_shard_size
    gen = torch.Generator(device=dev).manual_seed(w.seed)
    fulls = [torch.empty(w.total_numel, dtype=torch.bfloat16, device=dev).normal_(0.0, 0.02, generator=gen) for _ in range(layers)]
    gathered = [torch.empty(padded_numel, dtype=torch.bfloat16, device=dev) for _ in range(layers)]
    outs = [torch.empty(w.total_numel, dtype=torch.bfloat16, device=dev) for _ in range(layers)]
    bytes_per_launch = pack.bytes_moved
    assert unpack.bytes_moved == bytes_per_launch == 4 * w.total_numel
    launch_events = []

    def step(record: bool) -> None:
        # one pair of HIP events around the step's 2 * layers launches (on the stream they are launched on): events
        # around every single launch cost about 5 % of the throughput they are meant to measure
        if record:
            a, b = event_pair(torch)
            a.record()
        for i in range(layers):
            pack.run((fulls[i],), gathered[i])
        for i in range(layers):
            unpack.run((gathered[i],), outs[i])
        if record:
            b.record()
            launch_events.append((a, b))

    if args.calibrate_copy:
        cal_src = torch.empty(1 << 29, dtype=torch.bfloat16, device=dev).normal_()
        cal_dst = torch.empty_like(cal_src)
        cal_dst.copy_(cal_src)  # 1 GiB read + 1 GiB written by torch's element-wise copy kernel
        torch.cuda.synchronize()
        del cal_src, cal_dst
    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    record = not args.no_launch_events
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(record)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    step_bytes = 2 * layers * bytes_per_launch
    value = step_bytes / (elapsed / args.steps) / 1e9
    roundtrip_ok = all(torch.equal(o, f) for o, f in zip(outs[:2], fulls[:2]))
    if not roundtrip_ok:
        print("unpack(pack(x)) != x", file=sys.stderr)
        return 1
    if launch_events:
        avg_launch_ms = sum(a.elapsed_time(b) for a, b in launch_events) / (len(launch_events) * 2 * layers)
    else:
        avg_launch_ms = ms_per_step / (2 * layers)
    achieved = bytes_per_launch / (avg_launch_ms * 1e-3) / 1e9
    roofline = {
        "kernel": "segment_program_kernel<16,16> (pack / unpack of one hidden4096 layer buffer)",
        "bound": "hbm",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4),
        # HBM bytes per launch: not measurable from inside the run; the figure of the committed counter profile of this
        # workload (rocprofv3 FETCH_SIZE / WRITE_SIZE scaled by a plain 1 GiB copy), quoted only for the run it describes
        "traffic": PROFILED_TRAFFIC["bytes_per_launch"] if layers == w.layers else None,
        "traffic_source": (PROFILED_TRAFFIC["source"] + " (quoted, not measured by this run)") if layers == w.layers else None,
        "algorithmic_bytes_per_launch": bytes_per_launch,
        "avg_launch_ms": round(avg_launch_ms, 5),
        "launches_timed": len(launch_events) * 2 * layers,
    }
    result = {
        "metric": "pack/unpack GB/s (% HBM peak); Muon NS TFLOP/s + ms/step at hidden4096",
        "value": round(value, 1),
        "unit": "GB/s",
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
            "workload": f"{w.name}: {layers} layer buffers x {w.total_numel} bf16 elements, 2x2 block-sharded for simulated world 4, "
            "pack + unpack of every buffer per step (one launch per buffer each way)",
            "bytes_per_step": step_bytes,
            "reference_convention_GBps": round(value / 2, 1),
        },
        "pct_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "roofline": roofline,
    }
    del fulls, gathered, outs
    torch.cuda.empty_cache()

    legs = {}
    want = set() if args.skip_legs else {name for name in args.legs.split(",") if name}
    if args.skip_mixed:
        want.discard("mixed")
    if "mixed" in want:
        want |= {"muon", "adamw"}  # the mixed step reuses their set-up
    if "ceiling" in want:
        # -------------------------------------------------------------- what this part sustains: a plain contiguous copy of one
        # layer buffer's size through the library's range copy, pure reads and pure writes in the same launch shape
        import ctypes

        n_el = w.total_numel
        a_buf = torch.empty(n_el, dtype=torch.bfloat16, device=dev).normal_(0.0, 0.02)
        b_buf = torch.empty(n_el, dtype=torch.bfloat16, device=dev)
        sink = torch.zeros(4096, dtype=torch.uint8, device=dev)
        from matrix_fsdp_amd.kernels import native as N

        stream = torch.cuda.current_stream(dev).cuda_stream
        nbytes = 2 * n_el

        def probe(kind):
            _lib.check(_lib.lib().mfsdp_hbm_probe(kind, a_buf.data_ptr(), (sink if kind == 0 else b_buf).data_ptr(), nbytes, stream))

        t_copy, _ = time_launches(torch, lambda: N.copy_range(a_buf, b_buf, 0), 20, 5)
        t_read, _ = time_launches(torch, lambda: probe(0), 20, 5)
        t_write, _ = time_launches(torch, lambda: probe(1), 20, 5)
        t_torch, _ = time_launches(torch, lambda: b_buf.copy_(a_buf), 20, 5)
        read_gbps, write_gbps = nbytes / (t_read * 1e-3) / 1e9, nbytes / (t_write * 1e-3) / 1e9
        legs["hbm_ceiling_one_layer_buffer"] = {
            "plain_copy_GBps": round(2 * nbytes / (t_copy * 1e-3) / 1e9, 1),
            "read_only_GBps": round(read_gbps, 1),
            "write_only_GBps": round(write_gbps, 1),
            "equal_mix_of_both_GBps": round(2 / (1 / read_gbps + 1 / write_gbps), 1),
            "torch_copy_GBps": round(2 * nbytes / (t_torch * 1e-3) / 1e9, 1),
            "note": f"{nbytes} bytes each way, contiguous; plain copy = mfsdp_copy_range (read + written bytes counted), probes = "
            "mfsdp_hbm_probe; the equal mix is the rate at which half the bytes move at the read-only and half at the write-only rate",
        }
        result["roofline"]["frac_of_plain_copy"] = round(achieved / legs["hbm_ceiling_one_layer_buffer"]["plain_copy_GBps"], 4)
        # what the segment programs stand in for: the reference's per-segment slice copies (flat_buffer.py:1304-1316), on this
        # GPU, for ONE rank's shard of one layer buffer (a quarter of a pack), once after a warm-up pass
        rank_segments = plan.rank_segments[0]
        shard = torch.empty(plan.max_shard_size, dtype=torch.bfloat16, device=dev)

        def slice_copy_loop():
            for seg in rank_segments:
                shard[seg.local_start : seg.local_start + seg.numel].copy_(a_buf[seg.global_start : seg.global_start + seg.numel])

        slice_copy_loop()
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        slice_copy_loop()
        torch.cuda.synchronize(dev)
        t_loop = time.perf_counter() - t0
        loop_bytes = 2 * 2 * sum(seg.numel for seg in rank_segments)
        legs["reference_slice_copy_loop_same_gpu"] = {
            "segments": len(rank_segments),
            "ms_one_rank_shard": round(t_loop * 1e3, 2),
            "GBps": round(loop_bytes / t_loop / 1e9, 2),
            "note": "torch slice copy_ per layout segment, as the reference packs a rank's shard without its extension; rank 0 of one "
            "hidden4096 layer buffer, wall time including the launches",
        }
        del a_buf, b_buf, sink, shard
        torch.cuda.empty_cache()

    if "rows" in want:
        # -------------------------------------------------------------- hidden2048 row split: pack / unpack / chunk-cat + cast
        w2 = HIDDEN2048_W4
        plan2 = w2.plan()
        pack2 = pack_program(plan2, torch.bfloat16, device=dev)
        unpack2 = unpack_program(plan2, torch.bfloat16, device=dev)
        fill2 = grad_fill_program(w2.specs, plan2.shard_sizes, plan2.rank_segments, torch.bfloat16, torch.float32, device=dev)
        gen2 = torch.Generator(device=dev).manual_seed(w2.seed)
        full2 = [torch.empty(w2.total_numel, dtype=torch.bfloat16, device=dev).normal_(0.0, 0.02, generator=gen2) for _ in range(w2.layers)]
        gath2 = [torch.empty(w2.world_size * plan2.max_shard_size, dtype=torch.bfloat16, device=dev) for _ in range(w2.layers)]
        out2 = [torch.empty(w2.total_numel, dtype=torch.bfloat16, device=dev) for _ in range(w2.layers)]
        grads2 = [[torch.empty(s.numel, dtype=torch.bfloat16, device=dev).normal_(0.0, 1e-3, generator=gen2) for s in w2.specs] for _ in range(w2.layers)]
        packed32 = [torch.empty(w2.world_size * plan2.max_shard_size, dtype=torch.float32, device=dev) for _ in range(w2.layers)]

        def all_layers(fn):
            def run():
                for i in range(w2.layers):
                    fn(i)
            return run

        for name, fn, nbytes in (
            ("pack", all_layers(lambda i: pack2.run((full2[i],), gath2[i])), pack2.bytes_moved),
            ("unpack", all_layers(lambda i: unpack2.run((gath2[i],), out2[i])), unpack2.bytes_moved),
            ("chunk_cat_bf16_to_f32", all_layers(lambda i: fill2.run(grads2[i], packed32[i])), fill2.bytes_moved),
            # the same eight buffers as ONE grid (mfsdp_segment_program_run_many): launch ramp and tail paid once
            ("pack_8_buffers_one_grid", lambda: pack2.run_many([(f,) for f in full2], gath2), pack2.bytes_moved),
            ("unpack_8_buffers_one_grid", lambda: unpack2.run_many([(g,) for g in gath2], out2), unpack2.bytes_moved),
            ("chunk_cat_bf16_to_f32_8_buffers_one_grid", lambda: fill2.run_many(grads2, packed32), fill2.bytes_moved),
        ):
            med, _ = time_launches(torch, fn, 20, 5)
            legs[f"hidden2048_w4_rows.{name}"] = {
                "ms_all_8_layers": round(med, 4),
                "GBps": round(w2.layers * nbytes / (med * 1e-3) / 1e9, 1),
                "pct_hbm_peak": round(100 * w2.layers * nbytes / (med * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
            }
        assert torch.equal(out2[0], full2[0])
        del full2, gath2, out2, grads2, packed32
        torch.cuda.empty_cache()

    if "devcopy" in want:
        # -------------------------------------------------------------- the boundary function itself: copy_rank_segments_to_full with
        # DEVICE metadata (kernels/native/matrix_copy.cpp:53-83), one rank's shard of one hidden4096 layer buffer into the full buffer
        import ctypes

        from matrix_fsdp_amd.kernels import native as N
        from matrix_fsdp_amd.kernels.segment_program import local_segments_program

        segs = plan.rank_segments[0]
        n_sets = 4  # the launches rotate over four (shard, full buffer) pairs, 2 GB in all: nothing is served from a cache
        locals_dc = [torch.empty(plan.shard_sizes[0], dtype=torch.bfloat16, device=dev).normal_(0.0, 0.02) for _ in range(n_sets)]
        fulls_dc = [torch.zeros(plan.total_numel, dtype=torch.bfloat16, device=dev) for _ in range(n_sets)]
        gs, ls, ln, mx = N._segment_metadata_tensors(tuple(segs), device=dev)
        ws_dc = N.copy_rank_segments_workspace(len(segs), dev)
        moved = 2 * 2 * sum(sg.numel for sg in segs)  # bytes read + bytes written
        stream = torch.cuda.current_stream(dev).cuda_stream

        def noalloc(i):
            _lib.check(_lib.lib().mfsdp_copy_rank_segments_to_full_noalloc(
                locals_dc[i].data_ptr(), locals_dc[i].numel(), fulls_dc[i].data_ptr(), fulls_dc[i].numel(), gs.data_ptr(), ls.data_ptr(),
                ln.data_ptr(), len(segs), int(mx), 2, stream))

        prog_dc = local_segments_program(segs, locals_dc[0].numel(), plan.total_numel, torch.bfloat16, device=dev)
        leg = {"segments": len(segs), "bytes_moved": moved}
        per_batch = 8  # launches between one pair of events (a pair around every launch costs 2 us of a 35 us launch)
        for name, fn in (
            ("uniform_launch_shape", lambda i: N.copy_rank_segments_to_full(locals_dc[i], fulls_dc[i], gs, ls, ln, mx)),
            ("balanced_launch_shape", lambda i: N.copy_rank_segments_to_full(locals_dc[i], fulls_dc[i], gs, ls, ln, mx, workspace=ws_dc)),
            ("noalloc_entry_point", noalloc),
            ("compiled_segment_program_same_copy", lambda i: prog_dc.run((locals_dc[i],), fulls_dc[i])),
        ):
            def batch(fn=fn):
                for k in range(per_batch):
                    fn(k % n_sets)
            med, _ = time_launches(torch, batch, 12, 3)
            med /= per_batch
            leg[name] = {"us": round(med * 1e3, 2), "GBps": round(moved / (med * 1e-3) / 1e9, 1), "pct_hbm_peak": round(100 * moved / (med * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2)}
        want_full = torch.zeros_like(fulls_dc[1])
        prog_dc.run((locals_dc[1],), want_full)
        assert torch.equal(fulls_dc[1], want_full)
        leg["note"] = ("mfsdp_copy_rank_segments_to_full_device on rank 0's shard of one hidden4096 layer buffer (row segments of a 2x2 block shard), "
                       "metadata in device memory; uniform = one tile slot per (segment, tile index), balanced = byte-balanced grid behind two count kernels "
                       "(for layouts whose segment lengths differ widely), noalloc = balanced with the library's static scratch; time per launch "
                       "over back-to-back launches that rotate over four buffer pairs")
        legs["device_metadata_copy"] = leg
        del locals_dc, fulls_dc, ws_dc, want_full, prog_dc
        torch.cuda.empty_cache()

    if "gemm" in want:
        # -------------------------------------------------------------- one plain product through the Newton-Schulz kernel beside
        # the library's kernel for the same product (what torch.optim.Muon runs on)
        n_g = 8192
        pg = torch.empty(n_g, n_g, dtype=torch.bfloat16, device=dev).normal_()
        qg = torch.empty(n_g, n_g, dtype=torch.bfloat16, device=dev).normal_()
        cg = torch.empty(n_g, n_g, dtype=torch.bfloat16, device=dev)
        scratch_g = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
        stream = torch.cuda.current_stream(dev).cuda_stream

        def ours():
            _lib.check(_lib.lib().mfsdp_gemm_nt_bf16(pg.data_ptr(), qg.data_ptr(), cg.data_ptr(), n_g, n_g, n_g, scratch_g.data_ptr(), scratch_g.numel(), stream))

        def library():
            torch.matmul(pg, qg.T, out=cg)

        fl = 2.0 * n_g**3
        leg = {"shape": f"{n_g} x {n_g} x {n_g}, C = P Q^T, bf16, fp32 accumulation"}
        for name, fn in (("gemm_nt_kernel", ours), ("library_torch_matmul", library)):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            reps = 0
            while time.perf_counter() - t0 < 1.0:  # long enough for the clock to settle at its sustained level
                for _ in range(20):
                    fn()
                torch.cuda.synchronize()
                reps += 20
            sustained = (time.perf_counter() - t0) / reps
            med, _ = time_launches(torch, fn, 20, 2)
            leg[name] = {"us": round(med * 1e3, 1), "TFLOPs": round(fl / (med * 1e-3) / 1e12, 1),
                         "sustained_TFLOPs_over_1s": round(fl / sustained / 1e12, 1), "pct_bf16_mfma_peak": round(100 * fl / (med * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS, 2)}
        ours()
        torch.cuda.synchronize()
        check = torch.matmul(pg[:256].float(), qg[:256].float().T)
        assert torch.allclose(cg[:256, :256].float(), check, rtol=2e-2, atol=2.0)
        legs["gemm_8192_cubed"] = leg
        del pg, qg, cg, scratch_g
        torch.cuda.empty_cache()

    if "muon" in want:
        # -------------------------------------------------------------- Muon on the hidden4096 matrices
        ws = F.MuonWorkspace(dev)
        genm = torch.Generator(device=dev).manual_seed(MUON_SEED)
        mats = []
        for shape in MUON_HIDDEN4096_SHAPES:
            p = torch.empty(shape, device=dev).normal_(0.0, 0.02, generator=genm)
            g = torch.empty(shape, device=dev).normal_(0.0, 1e-3, generator=genm).bfloat16().float()  # bf16-valued grads
            buf = torch.empty(shape, device=dev).normal_(0.0, 1e-3, generator=genm)
            mats.append((p, g, buf))
        kw = dict(lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=True, ns_coefficients=NS_COEFFS, ns_steps=5, eps=1e-7)

        def muon_one_by_one():
            for p, g, buf in mats:
                F.muon_step(p, g, buf, workspace=ws, **kw)

        def muon_all():
            # the step of the optimizer: independent matrices side by side on the library's side streams, joined on this stream
            F.muon_step_many([(p, g, buf, kw) for p, g, buf in mats])

        med_one_stream = med = None
        if args.muon_form in ("both", "serial"):
            med_one_stream, _ = time_launches(torch, muon_one_by_one, 20, 5)
        if args.muon_form in ("both", "side-by-side"):
            med, _ = time_launches(torch, muon_all, 20, 5)
        if med is None:
            med = med_one_stream  # the step's time in the one form that was run
        flops = 0
        per_matrix = {}
        for (p, g, buf), shape in zip(mats, MUON_HIDDEN4096_SHAPES):
            m, n = min(shape), max(shape)
            fl = 5 * (4 * m * m * n + 2 * m**3)
            flops += fl
            if args.muon_form == "side-by-side":
                continue
            t, _ = time_launches(torch, lambda: F.muon_step(p, g, buf, workspace=ws, **kw), 20, 5)
            fl_exec = int(_lib.lib().mfsdp_muon_executed_flops(shape[0], shape[1], 5, 0))
            per_matrix[f"{shape[0]}x{shape[1]}"] = {"ms": round(t, 4), "TFLOPs_executed": round(fl_exec / (t * 1e-3) / 1e12, 1),
                                                    "TFLOPs_reference_flop_count": round(fl / (t * 1e-3) / 1e12, 1)}
        # the optimizer the reference builds for these parameters (torch.optim.Muon: hipBLASLt products, full GEMMs), same
        # GPU, same hyper-parameters, on copies of the tensors: the reference's own execution of this step, for scale
        torch_ms = None
        if hasattr(torch.optim, "Muon") and args.muon_form == "both":
            t_params = [torch.nn.Parameter(p.clone()) for p, _, _ in mats]
            t_opt = torch.optim.Muon(t_params, lr=kw["lr"], weight_decay=kw["weight_decay"], momentum=kw["momentum"], nesterov=kw["nesterov"],
                                     ns_coefficients=NS_COEFFS, eps=kw["eps"], ns_steps=kw["ns_steps"])
            for tp, (_, g, _) in zip(t_params, mats):
                tp.grad = g.clone()
            torch_ms, _ = time_launches(torch, t_opt.step, 10, 3)
            del t_opt, t_params
        tflops = flops / (med * 1e-3) / 1e12
        legs["muon_hidden4096"] = {
            "ms_per_step": round(med, 4),
            "form_timed": {"both": "side by side (muon_step_many)", "serial": "one matrix at a time", "side-by-side": "side by side (muon_step_many)"}[args.muon_form],
            "ms_per_step_one_matrix_at_a_time": None if med_one_stream is None else round(med_one_stream, 4),
            "ns_TFLOPs_reference_flop_count": round(tflops, 1),
            "pct_bf16_mfma_peak": round(100 * tflops / BF16_MFMA_PEAK_TFLOPS, 2),
            "flop_count": "5 * (4 m^2 n + 2 m^3) per matrix, full GEMMs as the reference executes them; the time is the whole "
            "update (momentum, norm, Newton-Schulz, parameter update) of the three matrices, which muon_step_many runs side by side on "
            "three streams; per_matrix times are each matrix alone",
            "dtype_variant": "fp32 params / momentum, bf16-valued fp32 grads",
            "per_matrix": per_matrix,
        }
        if torch_ms is not None:
            legs["muon_hidden4096"]["torch_optim_muon_same_gpu"] = {"ms_per_step": round(torch_ms, 4), "ns_TFLOPs_reference_flop_count": round(flops / (torch_ms * 1e-3) / 1e12, 1)}
        result["muon_ns_TFLOPs"] = round(tflops, 1)
        result["muon_ms_per_step"] = round(med, 4)
        if args.hold_muon_seconds > 0:
            t_hold, n_hold = time.perf_counter(), 0
            while time.perf_counter() - t_hold < args.hold_muon_seconds:
                for _ in range(20):
                    muon_all()
                torch.cuda.synchronize(dev)
                n_hold += 20
            held = (time.perf_counter() - t_hold) / n_hold * 1e3
            legs["muon_hidden4096"]["held"] = {"seconds": args.hold_muon_seconds, "ms_per_step": round(held, 4), "ns_TFLOPs_reference_flop_count": round(flops / (held * 1e-3) / 1e12, 1)}
        executed = sum(int(_lib.lib().mfsdp_muon_executed_flops(sh[0], sh[1], 5, 0 if args.muon_form == "serial" else _lib.MUON_SHARED_MACHINE)) for sh in MUON_HIDDEN4096_SHAPES)
        tflops_executed = executed / (med * 1e-3) / 1e12
        legs["muon_hidden4096"]["ns_TFLOPs_executed"] = round(tflops_executed, 1)
        result["roofline_muon"] = {
            "kernel": "gemm_nt_kernel (Newton-Schulz products; the whole Muon step is timed: momentum, norm, 15 products per matrix, update)",
            "bound": "mfma",
            # the reference's count: full GEMMs, 5 * (4 m^2 n + 2 m^3) per matrix
            "achieved": round(tflops, 1),
            "peak": BF16_MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(tflops / BF16_MFMA_PEAK_TFLOPS, 4),
            "frac_reference_count": round(tflops / BF16_MFMA_PEAK_TFLOPS, 4),
            # flops the kernels execute: the symmetric products X X^T and A A compute the tiles on or below the diagonal only
            "achieved_executed": round(tflops_executed, 1),
            "frac_executed": round(tflops_executed / BF16_MFMA_PEAK_TFLOPS, 4),
            "executed_over_reference_flops": round(executed / flops, 4),
            # counter figures QUOTED from the committed profiles of this leg (not measured by this run; see their `head` lines)
            "quoted_from_profiles": {"mfma_busy": PROFILED_MUON["mfma_busy"], "traffic_bytes_dominant_launch": PROFILED_MUON["traffic_bytes_per_launch"],
                                     "source": PROFILED_MUON["source"]},
        }
        del mats
        torch.cuda.empty_cache()

    if "adamw" in want:
        # -------------------------------------------------------------- fused AdamW on a flat fp32 shard
        n_adam = HIDDEN5120_TAIL_NUMEL
        pa, ga = torch.randn(n_adam, device=dev) * 0.02, torch.randn(n_adam, device=dev) * 1e-3
        ma, va = torch.zeros(n_adam, device=dev), torch.zeros(n_adam, device=dev)
        med, _ = time_launches(torch, lambda: F.adamw_step(pa, ga, ma, va, 1, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1), 20, 5)
        legs["adamw_flat_shard_41M_fp32"] = {"ms": round(med, 4), "GBps": round(28 * n_adam / (med * 1e-3) / 1e9, 1), "pct_hbm_peak": round(100 * 28 * n_adam / (med * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2)}
        del pa, ga, ma, va
        torch.cuda.empty_cache()

    if "mixed" in want:
        # -------------------------------------------------------------- hidden5120 mixed step, rank 0 of a simulated world of 4:
        # pack + unpack of the 40 rank-major owner-layout layer buffers (uneven shards, padded staging), AdamW on the fp32
        # tail shard, Muon on the 50 matrices this rank owns
        w5 = HIDDEN5120
        progs = {}
        for k in range(w5.world_size):  # the owner pattern repeats every world_size layers
            plan5 = w5.owner_layout(k)[2]
            progs[k] = (plan5, pack_program(plan5, torch.bfloat16, device=dev), unpack_program(plan5, torch.bfloat16, device=dev))
        gen5 = torch.Generator(device=dev).manual_seed(w5.seed)
        full5 = [torch.empty(w5.total_numel, dtype=torch.bfloat16, device=dev).normal_(0.0, 0.02, generator=gen5) for _ in range(w5.layers)]
        gath5 = [torch.empty(w5.world_size * progs[i % w5.world_size][0].max_shard_size, dtype=torch.bfloat16, device=dev) for i in range(w5.layers)]
        out5 = [torch.empty(w5.total_numel, dtype=torch.bfloat16, device=dev) for _ in range(w5.layers)]

        def copies5():
            for i in range(w5.layers):
                progs[i % w5.world_size][1].run((full5[i],), gath5[i])
            for i in range(w5.layers):
                progs[i % w5.world_size][2].run((gath5[i],), out5[i])

        t_copy, _ = time_launches(torch, copies5, 5, 2)
        assert torch.equal(out5[1], full5[1])
        copy_bytes = sum(progs[i % w5.world_size][1].bytes_moved + progs[i % w5.world_size][2].bytes_moved for i in range(w5.layers))
        del full5, gath5, out5, progs
        torch.cuda.empty_cache()

        owned = [s.shape for layer in range(w5.layers) for s, o in zip(w5.specs, w5.owner_ranks(layer)) if o == 0 and len(s.shape) == 2]
        mats5 = []
        for shape in owned:
            p = torch.empty(shape, device=dev).normal_(0.0, 0.02, generator=gen5)
            g = torch.empty(shape, device=dev).normal_(0.0, 1e-3, generator=gen5).bfloat16().float()
            mats5.append((p, g, torch.zeros(shape, device=dev)))
        pa = torch.empty(n_adam, device=dev).normal_(0.0, 0.02, generator=gen5)
        ga = torch.empty(n_adam, device=dev).normal_(0.0, 1e-3, generator=gen5)
        ma, va = torch.zeros(n_adam, device=dev), torch.zeros(n_adam, device=dev)

        def update5():
            F.adamw_step(pa, ga, ma, va, 1, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
            for p, g, buf in mats5:
                F.muon_step(p, g, buf, workspace=ws, **kw)

        t_upd, _ = time_launches(torch, update5, 3, 1)
        flops5 = sum(5 * (4 * min(sh) ** 2 * max(sh) + 2 * min(sh) ** 3) for sh in owned)
        legs["hidden5120_mixed_step_rank0_of_4"] = {
            "ms_per_step": round(t_copy + t_upd, 3),
            "copies_ms": round(t_copy, 4),
            "copies_GBps": round(copy_bytes / (t_copy * 1e-3) / 1e9, 1),
            "update_ms": round(t_upd, 3),
            "muon_matrices": len(owned),
            "ns_TFLOPs_reference_flop_count": round(flops5 / (t_upd * 1e-3) / 1e12, 1),
            "note": "40 owner-layout layer buffers packed and unpacked (padded staging of uneven shards, zero-filled pad "
            "tails counted as written bytes), AdamW on the 41M-element fp32 tail shard, Muon on every 4th matrix",
        }
        del mats5, pa, ga, ma, va
        torch.cuda.empty_cache()
    if legs:
        result["legs"] = legs

    # ------------------------------------------------------------------ CPU baselines (oracle port, bounded samples)
    if not args.skip_cpu:
        from oracle import copy_oracle, optim_oracle

        cpu_full = torch.empty(w.total_numel, dtype=torch.bfloat16).normal_(0.0, 0.02, generator=torch.Generator().manual_seed(w.seed))
        reps, t_cpu = 0, 0.0
        while reps < 40 and t_cpu < 12.0:
            t0 = time.perf_counter()
            padded = copy_oracle.pack_to_padded(cpu_full, plan)
            back = copy_oracle.unpack_from_padded(padded, plan)
            t_cpu += time.perf_counter() - t0
            reps += 1
        assert torch.equal(back, cpu_full)
        cpu_gbps = reps * 2 * bytes_per_launch / t_cpu / 1e9
        result["cpu_baseline"] = {
            "value": round(cpu_gbps, 3),
            "unit": "GB/s",
            "cores": host_cores,
            "threads": host_threads,
            "kind": "port",
            "sample": f"{reps} x (pack + unpack) of ONE of the 32 hidden4096 layer buffers ({w.total_numel} bf16 elements, ~85k row segments) with the "
            "oracle's per-segment slice-copy loops; same byte accounting as the GPU value",
            "seconds": round(t_cpu, 2),
        }
        if "muon" in want:
            u = torch.empty(4096, 4096).normal_(0.0, 1e-3, generator=torch.Generator().manual_seed(MUON_SEED))
            fl, t_ns, ns_reps = 0, 0.0, 0
            while ns_reps < 20 and t_ns < 10.0:
                t0 = time.perf_counter()
                optim_oracle.newton_schulz(u, NS_COEFFS, 5, 1e-7)
                t_ns += time.perf_counter() - t0
                fl += 5 * (4 * 4096**3 + 2 * 4096**3)
                ns_reps += 1
            result["cpu_baseline_muon"] = {
                "value": round(fl / t_ns / 1e12, 4),
                "unit": "TFLOP/s",
                "cores": host_cores,
                "threads": host_threads,
                "kind": "port",
                "sample": f"{ns_reps} x 5-step Newton-Schulz of one 4096x4096 matrix with the oracle (torch bf16 matmuls on the CPU)",
                "seconds": round(t_ns, 2),
            }
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
