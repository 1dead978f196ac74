#!/usr/bin/env python3
"""Headline benchmark: images/s of the u8/u8 MobileNetV2 (width 1.0, 224x224, random-init
weights, per-tensor PTQ calibrated on 32 seeded images) at batch 64 on one MI355X, running as
a resident `hip` function (one HIP-graph replay per step) with the input already in HBM.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 64]

Prints ONE JSON line.  Besides the contract fields it carries
  roofline     -- the kernel family (one kernel symbol, whatever its template arguments) with the
                  largest share of device time: algorithmic bytes of its launches / their summed
                  mean durations (HIP events on the stream the kernels run on) against the 8 TB/s
                  HBM peak; rooflines_by_family holds the same for the five largest families
  step_ms      -- min / avg / max of single, individually synchronised steps (the reference's
                  benchmark protocol, benchmark/cli.cpp:41-63)
  cpu_baseline -- the same graph executed the way nncase's CPU target executes it
                  (Dequantize -> float Conv2D -> Quantize with the loop-for-loop restatement of
                  its kernels), one thread, on a bounded number of batch-1 images.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0    # dense int8 MFMA


# Bytes that crossed the L2 <-> fabric boundary per launch (average over the launches of a kernel in
# one step) at the headline workload, blocks unfused (the default) and fused (--fuse-blocks), with whole-batch
# launches one after the other (--lanes 1 --in-flight 1), from two rocprofv3 --pmc runs
# of this script (FETCH_SIZE, then WRITE_SIZE, each scaled by what the same counter reads for the 256 MiB
# copy that --copy-probe launches: x1.9996 and x1.0000).  Counters cannot be read from inside a timed run, so the figures
# are recorded here and reported only for the configuration they were measured on: the bench line names the profile
# summary they come from, and reports no traffic at all when the kernels a run launches are not exactly the ones of
# the table (a kernel selection that has changed since the profile was taken).
MEASURED_TRAFFIC_SOURCE = {"unfused": "profiles/mobilenetv2_b64_kernels_counters.txt",
                           "fused": "profiles/mobilenetv2_b64_fused_blocks_kernels_counters.txt"}
MEASURED_TRAFFIC_B64 = {
    "unfused": {
        "dw3x3<S=1>": 19011936,
        "dw3x3<S=2>": 41883762,
        "qconv_igemm+add<T=2,RG=1,rows16>": 13054633,
        "qconv_igemm+add<T=2,RG=2,rows16>": 40563268,
        "qconv_igemm<T=1,RG=1,rows16>": 3359320,
        "qconv_igemm<T=1,RG=4,rows16>": 38602230,
        "qconv_igemm<T=12,RG=1,rows16>": 10267976,
        "qconv_igemm<T=2,RG=1,rows16>": 8930024,
        "qconv_igemm<T=2,RG=2,rows16>": 24171978,
        "qconv_igemm<T=2,RG=2,vec16>": 38626465,
        "qconv_igemm<T=5,RG=1,rows16>": 5099510,
        "qconv_igemm<T=6,RG=2,rows16>": 90023774,
        "qconv_igemm<T=8,RG=1,rows16>": 5904294,
        "qconv_igemm<T=9,RG=1,rows8>": 34301598,
        "qconv_wide+add<T=2,RG=2,rows16>": 6175918,
        "qconv_wide+add<T=4,RG=2,rows16>": 10530291,
        "qconv_wide+dequantize<T=2,RG=2,rows16>": 1710972,
        "qconv_wide<T=2,RG=2,rows16>": 4725052,
        "qconv_wide<T=4,RG=2,rows16>": 7450706,
        "qglobal_avgpool": 4238843,
        "quantize+pack": 51434794,
    },
    "fused": {
        "dw3x3<S=1>": 27882249,
        "dw3x3<S=2>": 51731083,
        "qblock+add<S=1,P=2>": 4954955,
        "qblock+add<S=1,P=4>": 2669235,
        "qblock+add<S=1,P=6>": 4553259,
        "qblock<S=1,P=6>": 3246740,
        "qblock<S=2,P=4>": 3355417,
        "qconv_igemm+add<T=2,RG=2,rows16>": 39841988,
        "qconv_igemm<T=1,RG=4,rows16>": 38602966,
        "qconv_igemm<T=12,RG=1,rows16>": 9114287,
        "qconv_igemm<T=2,RG=1,rows16>": 8914666,
        "qconv_igemm<T=2,RG=2,rows16>": 24176233,
        "qconv_igemm<T=2,RG=2,vec16>": 38614243,
        "qconv_igemm<T=5,RG=1,rows16>": 5104363,
        "qconv_igemm<T=6,RG=2,rows16>": 90039131,
        "qconv_igemm<T=9,RG=1,rows8>": 34300750,
        "qconv_wide+add<T=2,RG=2,rows16>": 5250994,
        "qconv_wide+dequantize<T=2,RG=2,rows16>": 1710205,
        "qconv_wide<T=2,RG=2,rows16>": 4714430,
        "qconv_wide<T=4,RG=2,rows16>": 8201110,
        "qglobal_avgpool": 4238971,
        "quantize+pack": 51434890,
    },
}


def op_accounting(qg, batch, model):
    """Per operator of the recorded function (one lane): (bytes, floor_bytes, macs).
    bytes is the algorithmic traffic of the graph nodes the operator computes, each counted as the
    operator of its own the reference runs: every node reads its inputs once, writes its output once and
    reads its constants once (a convolution with a table and a residual add in its epilogue, or a whole
    expand -> depthwise -> project block, is several such nodes).  floor_bytes is what the fused operator
    itself cannot avoid: the tensors that enter it, its result, its constants."""
    size = lambda j: batch * int(np.prod(qg.nodes[j].out_shape))
    nbytes, floors, macs = [], [], []
    for k, (name, members) in enumerate(zip(model.op_names, model.op_members)):
        if name.startswith("dequantize"):
            o = size(model.op_nodes[k])
            nbytes.append(o + 4 * o)
            floors.append(o + 4 * o)
            macs.append(0)
            continue
        inside = set(members)
        external = {j for m in members for j in qg.nodes[m].inputs if j not in inside}
        consts = b = m = 0
        for j in members:
            n = qg.nodes[j]
            b += sum(size(i) for i in n.inputs) + size(j)
            if n.op == "input":
                consts += 4 * size(j)            # the float32 tensor the quantize operator reads
            elif n.op == "conv":
                consts += n.weights.size + 4 * n.bias.size
                m += batch * n.macs
        nbytes.append(b + consts)
        floors.append(sum(size(j) for j in external) + size(members[-1]) + consts)
        macs.append(m)
    return nbytes, floors, macs


def time_calls(ctx, fn, warmup, steps):
    """Mean device milliseconds of fn() over `steps` back-to-back calls (wall clock, synchronised both sides)."""
    for _ in range(warmup):
        fn()
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    ctx.sync()
    return (time.perf_counter() - t0) / steps * 1e3


def step_spread(ctx, fn, steps):
    """min / avg / max milliseconds of single steps, each synchronised on its own (the reference's benchmark
    protocol, benchmark/cli.cpp:41-63: warm-up, then every run timed separately).  A step timed alone includes the
    host's launch and synchronisation latency, which back-to-back steps hide; `ms_per_step` is the back-to-back figure."""
    times = []
    for _ in range(steps):
        ctx.sync()
        t0 = time.perf_counter()
        fn()
        ctx.sync()
        times.append((time.perf_counter() - t0) * 1e3)
    return {"min": round(min(times), 5), "avg": round(sum(times) / len(times), 5), "max": round(max(times), 5), "runs": len(times)}


def side_workload(args):
    """The other BASELINE configurations' kernels at their real shapes (one JSON line each):
    --workload matmul            config 1: A[512,1024] u8 x B[1024,1024] u8 -> f32
    --workload conv_block        config 2: 1x1 64->144, dw 3x3, 1x1 144->64 on 56x56, batch 32
    --workload paged_attention   config 5: batch 32, 14 q / 2 kv heads, d 64, block 16, ctx U[512,4096], fp16
    """
    from nncase_amd import netbuilder as nb
    from nncase_amd import quant
    from nncase_amd import runtime as rt
    from nncase_amd.runtime import Context, qp

    ctx = Context(0)
    base = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "data": "synthetic"}
    if args.workload == "matmul":
        # config 1, and with --batched N the same product on N stacked A matrices (M = 512 N rows against the one
        # constant B): the steady-state form, in which the matrix cores and not the launch set the time
        rng = np.random.default_rng(0)
        rows = 512 * max(1, args.batched)
        a = rng.integers(0, 256, (rows, 1024), dtype=np.uint8)
        bq, zb, sb = quant.quantize_weights((rng.standard_normal((1024, 1024)) * 0.05).astype(np.float32))
        w = ctx.prepack_matmul(bq, None, qp(zb, sb), expected_rows=rows)
        da, dy = ctx.to_device(a), ctx.alloc(rows * 1024 * 4)
        margs = rt.MatmulArgs(rows, qp(128, 0.02), qp(0, 1.0), -rt.FLT_MAX, rt.FLT_MAX, rt.DT_F32)
        call = lambda: ctx.qmatmul(da, w, dy, margs)
        ms = time_calls(ctx, call, args.warmup, args.steps)
        ops, nbytes = 2 * rows * 1024 * 1024, rows * 1024 + 1048576 + rows * 1024 * 4
        tops = ops / (ms * 1e-3) / 1e12
        note = ("1.07 G int8-op and 3.67 MB: both roofline floors are < 0.5 us, the launch is latency-bound" if rows == 512 else
                f"{ops / 1e9:.1f} G int8-op, {nbytes / 1e6:.0f} MB (the f32 result is {rows * 4096 / 1e6:.0f} MB of it): floors "
                f"{ops / INT8_PEAK_TOPS / 1e6:.1f} us on the matrix cores, {nbytes / HBM_PEAK_GBS / 1e3:.1f} us on HBM")
        # the same product requantised to u8 (what a following quantised layer consumes): a quarter of the f32 stores
        dy8 = ctx.alloc(rows * 1024)
        sy = float(np.sqrt(1024.0) * 0.02 * 128 * sb * 0.6 / 128)
        margs8 = rt.MatmulArgs(rows, qp(128, 0.02), qp(128, sy), -rt.FLT_MAX, rt.FLT_MAX, rt.DT_U8)
        ms8 = time_calls(ctx, lambda: ctx.qmatmul(da, w, dy8, margs8), args.warmup, args.steps)
        line = dict(base, metric=f"int8 TOPS u8/u8 MatMul {rows}x1024x1024 -> f32", value=round(tops, 2), unit="TOPS",
                    u8_out={"int8_TOPS": round(ops / (ms8 * 1e-3) / 1e12, 2), "ms_per_step": round(ms8, 5),
                            "frac_of_int8_peak": round(ops / (ms8 * 1e-3) / 1e12 / INT8_PEAK_TOPS, 5)},
                    ms_per_step=round(ms, 5), dtype="u8",
                    config={"workload": "config 1: A[512,1024] u8 x B[1024,1024] u8, f32 out" +
                                        (f", batched x{args.batched} (A stacked to [{rows},1024])" if args.batched > 1 else "")},
                    roofline={"bound": "mfma", "achieved": round(tops, 2), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                              "frac": round(tops / INT8_PEAK_TOPS, 5), "traffic": None,
                              "hbm_GBps": round(nbytes / (ms * 1e-3) / 1e9, 1), "note": note},
                    step_ms=step_spread(ctx, call, args.steps))
    elif args.workload == "pack":
        # pack / unpack and the NCHW <-> NHWC relayout at sizes past the 256 MiB of memory-side cache: pure byte moves
        def moved(name, nbytes, call):
            ms = time_calls(ctx, call, max(args.warmup, 3), min(args.steps, 30))
            return {"case": name, "us": round(ms * 1e3, 1), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1), "frac_of_hbm": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        n, c, hw = 512, 256, 56
        cnt = n * c * hw * hw
        a, b = ctx.alloc(cnt), ctx.alloc(cnt)
        a.fill(1)
        cases = [moved("pack u8 NCHW [512,256,56,56] -> NC/32 HW 32", 2 * cnt, lambda: ctx.pack(a, b, 1, [n, c, hw, hw], [1], [32])),
                 moved("unpack of the same", 2 * cnt, lambda: ctx.unpack(b, a, 1, [n, c, hw, hw], [1], [32])),
                 moved("pack u8 [16384,16384] by (N: 16, K: 64) (weight tiles)", 2 * 16384 * 16384, lambda: ctx.pack(a, b, 1, [16384, 16384], [1, 0], [16, 64])),
                 moved("pack u8 NHWC [512,56,56,256] by 32 on C", 2 * cnt, lambda: ctx.pack(a, b, 1, [n, hw, hw, c], [3], [32])),
                 moved("nchw -> nhwc u8 [512,256,56,56]", 2 * cnt, lambda: ctx.nchw_to_nhwc(a, b, 1, n, c, hw, hw)),
                 moved("nhwc -> nchw u8 [512,256,56,56]", 2 * cnt, lambda: ctx.nhwc_to_nchw(b, a, 1, n, c, hw, hw)),
                 moved("nchw -> nhwc f32 [640,3,224,224]", 2 * 4 * 640 * 3 * 224 * 224, lambda: ctx.nchw_to_nhwc(a, b, 4, 640, 3, 224, 224)),
                 moved("nhwc -> nchw f32 [640,224,224,3]", 2 * 4 * 640 * 3 * 224 * 224, lambda: ctx.nhwc_to_nchw(b, a, 4, 640, 3, 224, 224)),
                 moved("copy (pack without axes) u32", 2 * cnt, lambda: ctx.pack(a, b, 4, [cnt // 4], [], []))]
        head = cases[0]
        line = dict(base, metric="GB/s pack u8 NCHW -> NC/32 HW 32", value=head["GBps"], unit="GB/s", ms_per_step=round(head["us"] / 1e3, 5), dtype="u8",
                    config={"workload": "pack / unpack / relayout of 411 MB tensors (read once, written once)"},
                    roofline={"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": head["frac_of_hbm"], "traffic": None},
                    cases=cases)
    elif args.workload == "conv_block":
        batch = 32
        rng = np.random.default_rng(1)
        qg = nb.quantize_graph(nb.conv_block(seed=1), rng.random((32, 56, 56, 64), dtype=np.float32))
        model = nb.HipModel(ctx, qg, batch, capture_graph=not args.no_graph)
        model.set_input(rng.random((batch, 56, 56, 64), dtype=np.float32))
        ms = time_calls(ctx, model.invoke, args.warmup, args.steps)
        spread = step_spread(ctx, model.invoke, args.steps)
        op_ms = model.fn.profile(10)
        nbytes = sum(op_accounting(qg, batch, model)[0])
        line = dict(base, metric="images/sec u8/u8 conv block b32", value=round(batch / (ms * 1e-3), 1), unit="images/s",
                    ms_per_step=round(ms, 5), dtype="u8",
                    config={"workload": "config 2: f32 in -> quantize -> 1x1 64->144, dw 3x3, 1x1 144->64 (ReLU6) on 56x56 -> dequantize, batch 32"},
                    roofline={"bound": "hbm", "achieved": round(nbytes / (sum(op_ms) * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": round(nbytes / (sum(op_ms) * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None},
                    step_ms=spread,
                    kernels={model.fn.op_kernel(i): round(t * 1e3, 2) for i, t in enumerate(op_ms)})
    elif args.workload == "yolov5s":
        batch, hw = 16, 640
        rng = np.random.default_rng(7)
        g = nb.yolov5s(seed=4, input_hw=hw)
        qg = nb.quantize_graph(g, rng.random((2, hw, hw, 3), dtype=np.float32), calib_batch=1)
        # copies of the function in flight, as in the headline workload
        pipe = nb.HipPipeline(0, qg, batch, depth=args.in_flight, capture_graph=not args.no_graph, lanes=args.lanes)
        model, ctx = pipe.models[0], pipe.contexts[0]
        x = rng.random((batch, hw, hw, 3), dtype=np.float32)
        pipe.set_input(x)
        for _ in range(max(args.warmup, args.in_flight)):
            pipe.submit()
        pipe.sync()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            pipe.submit()
        pipe.sync()
        ms = (time.perf_counter() - t0) / args.steps * 1e3
        spread = step_spread(ctx, model.invoke, args.steps)
        # per-kernel figures on the one-chain recording (kernels of concurrent chains have no duration of their own)
        kmodel = model if args.lanes == 1 else nb.HipModel(ctx, qg, batch, capture_graph=False)
        if kmodel is not model:
            kmodel.set_input(x)
        op_ms = kmodel.fn.profile(5)
        names = [kmodel.fn.op_kernel(i) for i in range(len(kmodel.fn))]
        macs = sum(qg.macs_per_image.values()) * batch
        groups = {}
        for nme, t in zip(names, op_ms):
            key = nme.split("<")[0]
            groups[key] = groups.get(key, 0.0) + t
        conv_ms = sum(t for nme, t in zip(names, op_ms) if nme.startswith("qconv"))
        # batch consistency: image 0 alone gives the same three head tensors
        one = nb.HipModel(ctx, qg, 1, capture_graph=False)
        one.run(x[:1])
        model.invoke()
        ctx.sync()
        for a, b in zip(model.all_outputs(), one.all_outputs()):
            if not np.array_equal(a[:1].view(np.uint32), b.view(np.uint32)):
                sys.exit("bench.py: batch-16 head outputs of image 0 differ from its batch-1 outputs")
        line = dict(base, metric="images/sec u8/u8 YOLOv5s 640x640 b16", value=round(batch / (ms * 1e-3), 1), unit="images/s",
                    ms_per_step=round(ms, 4), dtype="u8",
                    config={"workload": "config 4: YOLOv5s-style backbone + neck + head, 640x640, u8/u8 per-tensor PTQ (2 calibration "
                                        "images), batch 16, SiLU as byte tables, " + str(len(kmodel.fn)) + " operators, HIP-graph replay" +
                                        (f" as {args.lanes} concurrent chains of {batch // args.lanes} images" if args.lanes > 1 else "") +
                                        (f", {args.in_flight} copies of the function take the steps in turn (step_ms: one step at a time)"
                                         if args.in_flight > 1 else ""),
                            "in_flight": args.in_flight, "batch_consistent": True},
                    roofline={"bound": "mfma", "achieved": round(2 * macs / (conv_ms * 1e-3) / 1e12, 1), "peak": INT8_PEAK_TOPS,
                              "unit": "TOP/s", "frac": round(2 * macs / (conv_ms * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4), "traffic": None,
                              "note": "all convolutions together: int8 op count / summed conv kernel time"},
                    step_ms=spread, sum_of_kernel_ms=round(sum(op_ms), 4),
                    kernel_groups_ms={k: round(v, 4) for k, v in sorted(groups.items(), key=lambda kv: -kv[1])})
    elif args.workload == "llm_decode":
        from nncase_amd import llm
        cfg = llm.DecoderConfig()
        batch, max_ctx = 32, 4096
        rng = np.random.default_rng(5)
        weights = llm.random_weights(cfg, seed=5)
        lens = rng.integers(512, max_ctx + 1, batch).astype(np.int32)
        max_blocks = (max_ctx + args.steps + args.warmup + 64) // cfg.block_size + 1
        nblocks = batch * max_blocks
        bt = rng.permutation(nblocks).reshape(batch, max_blocks).astype(np.int32)
        # one random cache image, uploaded once per layer (every layer has its own device copy)
        kc = rng.standard_normal((nblocks, cfg.kv_heads, cfg.block_size, cfg.head_dim), dtype=np.float32).astype(np.float16)
        vc = rng.standard_normal((nblocks, cfg.kv_heads, cfg.head_dim, cfg.block_size), dtype=np.float32).astype(np.float16)
        dec = llm.HipDecoder(ctx, cfg, weights, batch, max_blocks, bt, lens, [kc] * cfg.layers, [vc] * cfg.layers,
                             capture_graph=not args.no_graph, feedback=True, lanes=args.decode_lanes)
        dec.set_tokens(rng.integers(0, cfg.vocab, batch).astype(np.int32))
        ms = time_calls(ctx, dec.step, args.warmup, args.steps)
        toks = dec.result()
        assert toks.min() >= 0 and toks.max() < cfg.vocab
        steps_done = args.warmup + args.steps
        mean_ctx = float(lens.mean()) + steps_done / 2
        kv_bytes = int(mean_ctx * batch * cfg.kv_heads * cfg.head_dim * 2 * 2 * cfg.layers)
        w_bytes = dec.weight_bytes()
        op_ms = dec.fn.profile(3)
        groups = {}
        for i, t in enumerate(op_ms):
            k_ = dec.fn.op_kernel(i)
            groups[k_] = groups.get(k_, 0.0) + t
        line = dict(base, metric="tokens/sec LLM decode step b32 (Qwen2-0.5B shape, W8A16, fp16 paged KV)", value=round(batch / (ms * 1e-3), 1),
                    unit="tokens/s", ms_per_step=round(ms, 4), dtype="f16",
                    config={"workload": "config 5: 24 layers, hidden 896, 14 q / 2 kv heads, head_dim 64, MLP 4864, vocab 151936, W8A16 per-output-channel "
                                        "weights, fp16 paged KV (block 16), batch 32, ctx U[512,4096], greedy arg-max fed back on the device, "
                                        f"{len(dec.fn)} operators in {args.decode_lanes} lane(s), one HIP-graph replay per step"},
                    roofline={"bound": "hbm", "achieved": round((kv_bytes + w_bytes) / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": round((kv_bytes + w_bytes) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                              "algorithmic_bytes_per_step": kv_bytes + w_bytes, "weight_bytes": w_bytes, "kv_bytes": kv_bytes},
                    sum_of_kernel_ms=round(sum(op_ms), 4),
                    kernel_groups_ms={k_: round(v, 4) for k_, v in sorted(groups.items(), key=lambda kv: -kv[1])})
    elif args.workload == "paged_attention":
        rng = np.random.default_rng(5)
        bsz, hq, hkv, d, blk = 32, 14, 2, 64, 16
        lens = rng.integers(512, 4097, bsz).astype(np.int32)
        max_blocks = 4096 // blk
        nblocks = bsz * max_blocks
        q = rng.standard_normal((bsz, hq, d)).astype(np.float16)
        kc = rng.standard_normal((nblocks, hkv, blk, d)).astype(np.float16)
        vc = rng.standard_normal((nblocks, hkv, d, blk)).astype(np.float16)  # V is cached d-major
        bt = rng.permutation(nblocks).reshape(bsz, max_blocks).astype(np.int32)
        dq, dk, dv, dbt, dcl = (ctx.to_device(t) for t in (q, kc, vc, bt, lens))
        dout = ctx.alloc(bsz * hq * d * 2)
        pargs = rt.PagedAttnArgs(bsz, hq, hkv, d, blk, max_blocks, nblocks, 0.125, rt.DT_F16)
        attn = lambda: ctx.paged_attention_decode(dq, dk, dv, dbt, dcl, dout, pargs)
        ms = time_calls(ctx, attn, args.warmup, args.steps)
        spread = step_spread(ctx, attn, args.steps)
        kv_bytes = int(lens.sum()) * hkv * d * 2 * 2
        line = dict(base, metric="sequence-layers/sec paged-attention decode b32", value=round(bsz / (ms * 1e-3), 1), unit="sequence-layers/s",
                    ms_per_step=round(ms, 5), dtype="f16",
                    config={"workload": "config 5 attention layer: batch 32, 14 q / 2 kv heads, head_dim 64, block 16, ctx U[512,4096], "
                                        f"{int(lens.sum())} cached tokens, fp16 KV"},
                    roofline={"bound": "hbm", "achieved": round(kv_bytes / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": round(kv_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                              "algorithmic_bytes_per_launch": kv_bytes},
                    step_ms=spread)
    else:
        sys.exit(f"unknown workload {args.workload}")
    print(json.dumps(line))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="mobilenetv2", help="mobilenetv2 (headline, default) | matmul | conv_block | yolov5s | paged_attention | llm_decode | pack")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--batched", type=int, default=1, help="--workload matmul: number of stacked A matrices (M = 512 x this)")
    ap.add_argument("--lanes", type=int, default=1,
                    help="independent chains the batch is split into and replayed concurrently (1 = one chain of "
                         "full-batch launches); results are bit-identical for every value")
    ap.add_argument("--decode-lanes", type=int, default=2,
                    help="--workload llm_decode: ranges the 32 sequences are split into, each recorded as a chain of its own that the graph replays beside the others")
    ap.add_argument("--in-flight", type=int, default=4,
                    help="copies of the function (own stream and buffers each) that take the steps in turn, so that "
                         "consecutive steps overlap on the device (1 = one step at a time)")
    ap.add_argument("--cpu-images", type=int, default=32, help="batch-1 images timed on the CPU baseline (0 = skip)")
    ap.add_argument("--profile-iters", type=int, default=10)
    ap.add_argument("--batch1-steps", type=int, default=200, help="timed batch-1 invocations (0 = skip the batch-1 figure)")
    ap.add_argument("--fuse-blocks", action="store_true",
                    help="run the inverted-residual blocks on the 28x28 and 14x14 maps as one fused kernel each (38 operators "
                         "instead of 56): shorter single steps, but more vector-ALU work in total, so fewer images per "
                         "second once steps overlap")
    ap.add_argument("--no-graph", action="store_true",
                    help="enqueue the operators one by one instead of replaying the HIP graph (used under rocprofv3 "
                         "--kernel-trace, whose tracer crashes inside hipGraphLaunch on this image)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="first launch a plain 256 MiB -> 256 MiB copy kernel three times, so that a rocprofv3 --pmc run of "
                         "this command can scale FETCH_SIZE / WRITE_SIZE by what they read for a copy of known size")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the workload is one GPU's share at its real shape); "
                 "--gpus N with N > 1 is not supported")
    if args.workload != "mobilenetv2":
        return side_workload(args)

    from nncase_amd import netbuilder as nb
    from nncase_amd.runtime import Context

    probe_ctx = Context(0)  # raises if libnncase_hip.so is missing or there is no gfx950 device
    ctx = probe_ctx
    if args.copy_probe:
        n = 64 << 20  # dwords
        src, dst = ctx.alloc(n * 4), ctx.alloc(n * 4)
        src.fill(1)
        dst.fill(0)
        for _ in range(3):
            ctx.pack(src, dst, 4, [n], [], [])  # no packed axes: the element-wise pack kernel is a plain copy (16 bytes per thread)
        ctx.sync()
        del src, dst
    graph = nb.mobilenet_v2(seed=2)
    calib = np.random.default_rng(3).random((32, 224, 224, 3), dtype=np.float32)
    qg = nb.quantize_graph(graph, calib)
    x = np.random.default_rng(4).random((args.batch, 224, 224, 3), dtype=np.float32)

    # --in-flight copies of the function, each with its own stream and buffers, take the steps in turn: step i + 1
    # is enqueued while step i runs.  Every step is still one whole pass over one batch on one copy.
    pipe = nb.HipPipeline(0, qg, args.batch, depth=args.in_flight, capture_graph=not args.no_graph, lanes=args.lanes,
                          fuse_blocks=args.fuse_blocks)
    model = pipe.models[0]
    ctx = pipe.contexts[0]
    pipe.set_input(x)  # resident in HBM before the timed region
    # Order of the measurements: the one-step-at-a-time latencies and the per-kernel times come first, the headline's
    # warm-up and timed steps last.  The device raises its clocks over the first tens of milliseconds of load (20 timed
    # steps behind 5 warm-up steps read 213 k images/s, behind 50: 221 k, behind 400: 224 k), and the headline is the
    # steady rate; the steps it counts are the --warmup untimed and the --steps timed ones either way.
    spread = step_spread(ctx, model.invoke, args.steps)  # one step at a time: the latency of a step on an idle device

    # ---- per-kernel device time (HIP events on the context's stream) --------------------------
    # Kernels of concurrently replayed chains overlap and have no duration of their own, so the per-kernel figures
    # are taken on the one-chain recording of the same operators (every launch then covers the whole batch).
    kmodel = model if args.lanes == 1 else nb.HipModel(ctx, qg, args.batch, capture_graph=False, lanes=1,
                                                        fuse_blocks=args.fuse_blocks)
    if kmodel is not model:
        kmodel.set_input(x)
        kmodel.invoke()
        ctx.sync()
        if not np.array_equal(kmodel.output().view(np.uint32), model.output().view(np.uint32)):
            sys.exit("bench.py: the one-chain and the %d-chain function disagree" % args.lanes)
    op_ms = kmodel.fn.profile(args.profile_iters)
    names = [kmodel.fn.op_kernel(i) for i in range(len(kmodel.fn))]

    # ---- the headline: --warmup untimed steps, then exactly --steps timed ones ------------------
    for _ in range(max(args.warmup, args.in_flight)):
        pipe.submit()
    pipe.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        pipe.submit()
    pipe.sync()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    images_per_s = args.batch / (dt / args.steps)
    for m in pipe.models[1:]:
        if not np.array_equal(m.output().view(np.uint32), model.output().view(np.uint32)):
            sys.exit("bench.py: the copies of the function in flight disagree")
    # every lane launches the whole operator list on its batch/lanes images (and reads the weights itself)
    lane_batch = args.batch // args.lanes
    abytes, fbytes, macs = op_accounting(qg, args.batch, kmodel)
    assert len(abytes) == len(macs) == len(names) == len(op_ms)
    groups = {}
    for name, ms, b, fb, m in zip(names, op_ms, abytes, fbytes, macs):
        g = groups.setdefault(name, {"ms": 0.0, "bytes": 0, "floor": 0, "macs": 0, "launches": 0})
        g["ms"] += ms
        g["bytes"] += b
        g["floor"] += fb
        g["macs"] += m
        g["launches"] += 1
    # Kernel families (one symbol, whatever its template arguments and fused extras): the dominant one is the family
    # with the largest share of device time.
    def family(name):
        return name.split("<")[0].split("+")[0]

    table_key = "fused" if args.fuse_blocks else "unfused"
    table = MEASURED_TRAFFIC_B64[table_key]
    live, recorded = set(groups), set(table)
    traffic_source = {"profile": MEASURED_TRAFFIC_SOURCE[table_key], "kernels_in_profile": sorted(recorded),
                      "matches_this_run": args.batch == 64 and live == recorded}
    if live != recorded:
        traffic_source["launched_but_not_profiled"] = sorted(live - recorded)
        traffic_source["profiled_but_not_launched"] = sorted(recorded - live)
    fams = {}
    for name, g in groups.items():
        f = fams.setdefault(family(name), {"ms": 0.0, "bytes": 0, "floor": 0, "macs": 0, "launches": 0, "traffic": 0, "traffic_known": True})
        for k in ("ms", "bytes", "floor", "macs", "launches"):
            f[k] += g[k]
        t = table.get(name) if traffic_source["matches_this_run"] else None
        if t is None:
            f["traffic_known"] = False
        else:
            f["traffic"] += t * g["launches"]

    def roofline_of(fname, f):
        # every operator is held to the bytes it cannot avoid (the tensors that enter it, its result, its constants);
        # where it computes several graph nodes (a block, a conv with a table or a residual add in its epilogue, the
        # quantising pack) the bytes of those nodes run one by one, as the reference runs them, are reported beside it
        own = f["floor"]
        gbs = own / (f["ms"] * 1e-3) / 1e9
        r = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
             "traffic": int(f["traffic"] / f["launches"]) if f["traffic_known"] else None,
             "kernel": fname, "images_per_launch": args.batch, "launches_per_step": f["launches"],
             "avg_launch_us": round(f["ms"] / f["launches"] * 1e3, 2),
             "algorithmic_bytes_per_launch": int(own / f["launches"]),
             "share_of_device_time": round(f["ms"] / sum(op_ms), 4),
             "int8_TOPS": round(2 * f["macs"] / (f["ms"] * 1e-3) / 1e12, 2),
             "mfma_frac": round(2 * f["macs"] / (f["ms"] * 1e-3) / 1e12 / INT8_PEAK_TOPS, 5)}
        if f["bytes"] != f["floor"]:
            r["unfused_operator_bytes_per_launch"] = int(f["bytes"] / f["launches"])
            r["unfused_credit_GBps"] = round(f["bytes"] / (f["ms"] * 1e-3) / 1e9, 1)
        return r

    ranked = sorted(fams.items(), key=lambda kv: -kv[1]["ms"])
    dom_name, dom = ranked[0]

    def klass(name):
        if name.startswith("qblock"):
            return "fused_block"
        return "dense" if name.startswith("qconv_") else ("depthwise" if name.startswith("dw") else "elementwise")

    classes = {}
    for name, g in groups.items():
        c = classes.setdefault(klass(name), {"ms": 0.0, "floor": 0, "macs": 0})
        for k in ("ms", "floor", "macs"):
            c[k] += g[k]
    class_report = {k: {"ms": round(v["ms"], 4), "hbm_GBps": round(v["floor"] / (v["ms"] * 1e-3) / 1e9, 1),
                        "hbm_frac": round(v["floor"] / (v["ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                        "int8_TOPS": round(2 * v["macs"] / (v["ms"] * 1e-3) / 1e12, 2),
                        "mfma_frac": round(2 * v["macs"] / (v["ms"] * 1e-3) / 1e12 / INT8_PEAK_TOPS, 5)}
                    for k, v in classes.items()}

    # ---- batch-1 latency (same graph, HIP-graph replay) -----------------------------------------
    b1 = None
    if args.batch1_steps > 0:
        m1 = nb.HipModel(ctx, qg, 1, capture_graph=not args.no_graph)
        m1.set_input(x[:1])
        for _ in range(20):
            m1.invoke()
        ctx.sync()
        t1 = time.perf_counter()
        for _ in range(args.batch1_steps):
            m1.invoke()
        ctx.sync()
        b1_ms = (time.perf_counter() - t1) / args.batch1_steps * 1e3
        b1 = {"ms_per_image": round(b1_ms, 4), "images_per_s": round(1e3 / b1_ms, 1), "operators": len(m1.fn)}
        # the batched run must give image 0 the very logits it gets alone (integer arithmetic: bit-exact);
        # the batch-1 graph is the one the GPU tests follow tensor by tensor against the CPU oracle
        model.invoke()
        ctx.sync()
        if not np.array_equal(model.output()[:1].view(np.uint32), m1.output().view(np.uint32)):
            sys.exit("bench.py: batch-%d logits of image 0 differ from its batch-1 logits" % args.batch)
        b1["batch_consistent"] = True

    # ---- CPU baseline: the CPU target's float chain, 1 thread, bounded sample -------------------
    cpu = None
    if args.cpu_images > 0:
        from oracle import netref
        t2 = time.perf_counter()
        for i in range(args.cpu_images):
            netref.run_float_chain(qg, x[i % args.batch:i % args.batch + 1])
        cpu_dt = time.perf_counter() - t2
        cpu = {"value": round(args.cpu_images / cpu_dt, 4), "unit": "images/s", "cores": 1, "kind": "port",
               "host_cores": os.cpu_count(),
               "sample": f"{args.cpu_images} batch-1 images of the same MobileNetV2 graph, every conv as Dequantize -> float "
                         "Conv2D(fused_clamp) -> Quantize with the restated nncase CPU-target loops, -O2, 1 thread"}

    total_macs = sum(macs)
    line = {
        "metric": "images/sec u8/u8 MobileNetV2 b64",
        "value": round(images_per_s, 1),
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": f"MobileNetV2 w1.0 224x224 u8/u8 per-tensor PTQ (32 calibration images), batch {args.batch}, "
                               "NHWC f32 input resident in HBM -> quantize -> 52 convs + 10 adds + pool + FC -> dequantize" +
                               (f"; {len(model.blocks)} expand/depthwise/project blocks fused into one kernel each" if model.blocks else ""),
                   "batch": args.batch, "lanes": args.lanes, "in_flight": args.in_flight, "ops_per_step": len(model.fn),
                   "execution": "resident hip function, " + ("eager launches" if args.no_graph else "HIP-graph replay") +
                                (f", {args.lanes} concurrent chains of {lane_batch} images" if args.lanes > 1 and not args.no_graph else "") +
                                (f"; {args.in_flight} copies of the function (own stream and buffers) take the steps in turn, so "
                                 "consecutive steps overlap on the device; step_ms is one step at a time" if args.in_flight > 1 else "")},
        "roofline": roofline_of(dom_name, dom),
        "rooflines_by_family": [roofline_of(n, f) for n, f in ranked[:5]],
        "traffic_source": traffic_source,
        "step_ms": spread,
        # the other view of the same function: one request at a time on an idle device (value has --in-flight requests overlapping)
        "one_request_at_a_time": {"images_per_s": round(args.batch / (spread["avg"] * 1e-3), 1), "ms_per_step": spread["avg"]},
        "cpu_baseline": cpu,
        "int8_TOPS_whole_net": round(2 * total_macs / (ms_per_step * 1e-3) / 1e12, 2),
        "hbm_GBps_whole_net": round(sum(fbytes) / (ms_per_step * 1e-3) / 1e9, 1),
        "hbm_GBps_whole_net_unfused_operator_bytes": round(sum(abytes) / (ms_per_step * 1e-3) / 1e9, 1),
        "sum_of_kernel_ms": round(sum(op_ms), 4),
        "kernel_classes": class_report,
        "kernels": {k: {"ms": round(v["ms"], 4), "launches": v["launches"],
                        "hbm_GBps": round(v["floor"] / (v["ms"] * 1e-3) / 1e9, 1)} for k, v in sorted(groups.items())},
        "operators": [{"kernel": n, "us": round(t * 1e3, 2)} for n, t in zip(names, op_ms)],
        "batch1": b1,
        "device": {"compute_units": ctx.compute_units, "clock_mhz": ctx.clock_khz / 1000.0},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
