"""GPU parity of whole quantised graphs run as a resident `hip` function (eager and as a HIP
graph) against the CPU oracle executing the same graph node by node: every intermediate u8
tensor and the dequantised output must be bit-identical.  The float chain the CPU target
really executes is cross-checked layer by layer (same inputs) to the <= 1 LSB bar."""
import numpy as np
import pytest

from nncase_amd import netbuilder as nb
from nncase_amd import runtime as rt
from oracle import netref
from oracle import oracle as O

pytestmark = pytest.mark.gpu
f32 = np.float32


def check_model(hip_ctx, qg, x, capture, fuse_residual=True, fuse_blocks="all", fuse_pairs=True):
    model = nb.HipModel(hip_ctx, qg, x.shape[0], capture_graph=capture, fuse_residual=fuse_residual, fuse_blocks=fuse_blocks,
                        fuse_pairs=fuse_pairs)
    y = model.run(x)
    want, outs = netref.run_integer(qg, x, keep_all=True)
    for i, ref in enumerate(outs):
        if not model.materialized(i):
            continue
        got = model.tensor(i)
        assert np.array_equal(got, ref), f"node {i} ({qg.nodes[i].name}): {(got != ref).sum()} of {ref.size} bytes differ"
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    return model, y, outs


def test_conv_block_config2(hip_ctx):
    g = nb.conv_block(seed=1)
    rng = np.random.default_rng(1)
    calib = rng.random((32, 56, 56, 64), dtype=f32)
    qg = nb.quantize_graph(g, calib)
    assert qg.macs_per_image == {"dense": 2 * 28901376, "depthwise": 4064256}
    x = rng.random((2, 56, 56, 64), dtype=f32)
    check_model(hip_ctx, qg, x, capture=False)
    model, y, outs = check_model(hip_ctx, qg, x, capture=True)
    # HIP-graph replays interleaved with eager work keep giving the same bytes
    for _ in range(3):
        model.set_input(x)
        model.invoke()
        hip_ctx.sync()
        assert np.array_equal(model.output().view(np.uint32), y.view(np.uint32))
        model.fn.invoke_one(1)
        hip_ctx.sync()


def test_conv_block_config2_at_batch_32(hip_ctx):
    """BASELINE config 2 at its larger batch: every tensor of the 32-image block equals the oracle's, unfused
    (three operators) and as HipModel fuses it, eagerly and replayed as a graph."""
    rng = np.random.default_rng(1)
    qg = nb.quantize_graph(nb.conv_block(seed=1), rng.random((32, 56, 56, 64), dtype=f32))
    x = rng.random((32, 56, 56, 64), dtype=f32)
    want, outs = netref.run_integer(qg, x, keep_all=True)
    for capture, fuse_blocks in ((False, False), (True, "all"), (True, True)):
        model = nb.HipModel(hip_ctx, qg, 32, capture_graph=capture, fuse_blocks=fuse_blocks)
        y = model.run(x)
        for i, ref in enumerate(outs):
            if model.materialized(i):
                assert np.array_equal(model.tensor(i), ref), f"node {i} ({qg.nodes[i].name}), capture={capture}, fuse={fuse_blocks}"
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32))


def test_mobilenetv2_config3(hip_ctx):
    g = nb.mobilenet_v2(seed=2)
    rng = np.random.default_rng(3)
    calib = rng.random((32, 224, 224, 3), dtype=f32)
    qg = nb.quantize_graph(g, calib)
    assert qg.macs_per_image == {"dense": 280057856, "depthwise": 20716416}
    x = rng.random((2, 224, 224, 3), dtype=f32)
    plain, _, _ = check_model(hip_ctx, qg, x, capture=False, fuse_residual=False)   # every tensor, add as its own kernel
    assert len(plain.fused_into) == 0 and len(plain.fn) == 67     # (quantize, pack of 2 x 2 pixel blocks, 52 convs, ...)
    model, y, outs = check_model(hip_ctx, qg, x, capture=True, fuse_blocks=False, fuse_pairs=False)
    assert len(model.fused_into) == 10 and len(model.fused_dequant) == 1 and len(model.fn) == 55   # residual adds folded into
    #                                                                            the convs, the output's dequantize into the classifier
    model, y, outs = check_model(hip_ctx, qg, x, capture=True, fuse_blocks=False, fuse_pairs="all")
    assert len(model.pairs) == 17 and len(model.pair_fronts) == 17 and len(model.pool_fronts) == 1 and len(model.fn) == 20   # every depthwise convolution and projection runs
    #                                                                      with the expansion behind them as one launch, the classifier with its pool
    model, y, outs = check_model(hip_ctx, qg, x, capture=True, fuse_blocks=False, fuse_pairs="nofront")
    assert 0 < len(model.pairs) < 17 and not model.pair_fronts
    model, y, outs = check_model(hip_ctx, qg, x, capture=True, fuse_blocks=False)
    assert 0 < len(model.pairs) < 17                           # ... at this batch, where the pair streams few weights
    model, y, outs = check_model(hip_ctx, qg, x, capture=True)
    assert len(model.blocks) == 16 and len(model.pool_fronts) == 1 and len(model.fn) == 22   # ... and whole blocks into one operator
    # the reference's own acceptance bar for a PTQ model: cosine >= 0.98 against the float model
    fl = nb.float_forward(g, x)[-1]
    assert O.cosine(y, fl) > 0.98
    # layer-by-layer cross-check against the CPU target's float chain on identical inputs
    for i, n in enumerate(qg.nodes):
        if n.op != "conv" or i % 5:
            continue
        src = qg.nodes[n.inputs[0]]
        chain = O.qconv2d_float_chain(outs[n.inputs[0]][:1], n.weights, n.bias, src.out_qp[0], src.out_qp[1], n.w_qp[0], n.w_qp[1],
                                      n.out_qp[0], n.out_qp[1], n.stride, n.padding, (1, 1), n.groups, n.clamp)
        d = np.abs(chain.astype(np.int32) - outs[i][:1].astype(np.int32))
        assert d.max() <= 1, f"{n.name}: float chain differs by {d.max()} LSB"
    # batch independence: image 0 alone gives the same logits (size-independent property)
    m1 = nb.HipModel(hip_ctx, qg, 1, capture_graph=False)
    assert np.array_equal(m1.run(x[:1]).view(np.uint32), y[:1].view(np.uint32))


def test_mobilenetv2_batch64_equals_small_batches(hip_ctx):
    """The headline configuration (batch 64) picks other tilings and strip lengths than the small batches
    the oracle can follow: every tensor of the batch-64 run must equal, image by image, what a batch-4 run
    of the same images gives (integer arithmetic: bit-exact), and image 0 must equal the oracle's logits."""
    g = nb.mobilenet_v2(seed=2)
    rng = np.random.default_rng(3)
    qg = nb.quantize_graph(g, rng.random((32, 224, 224, 3), dtype=f32))
    x = np.random.default_rng(4).random((64, 224, 224, 3), dtype=f32)
    for fuse in (False, True):
        big = nb.HipModel(hip_ctx, qg, 64, capture_graph=True, fuse_residual=fuse)
        y = big.run(x)
        smalls = []
        for lo in (0, 60):
            small = nb.HipModel(hip_ctx, qg, 4, capture_graph=False, fuse_residual=fuse)
            ys = small.run(x[lo:lo + 4])
            assert np.array_equal(ys.view(np.uint32), y[lo:lo + 4].view(np.uint32))
            smalls.append((lo, small))
        for i in range(len(qg.nodes)):
            if not big.materialized(i):
                continue
            whole = big.tensor(i)
            for lo, small in smalls:
                a, b = whole[lo:lo + 4], small.tensor(i)
                assert np.array_equal(a, b), f"node {i} ({qg.nodes[i].name}), images {lo}..{lo + 3}: {(a != b).sum()} bytes differ"
    want = netref.run_integer(qg, x[:1])
    want = want[0] if isinstance(want, tuple) else want
    assert np.array_equal(y[:1].view(np.uint32), np.asarray(want).view(np.uint32))


def test_yolov5s_config4(hip_ctx):
    """YOLOv5s-style backbone + neck + head at a reduced input (128 x 128, batch 2): every u8 tensor and the
    three dequantised head outputs equal the oracle's; the same graph through a kmodel file gives the same bytes."""
    from nncase_amd import kmodel as km
    from nncase_amd import runtime as rt
    g = nb.yolov5s(seed=4, input_hw=128)
    rng = np.random.default_rng(6)
    qg = nb.quantize_graph(g, rng.random((4, 128, 128, 3), dtype=f32))
    ops = [n.op for n in qg.nodes]
    assert ops.count("conv") == 60 and ops.count("lut") == 57 and ops.count("concat") == 13 and ops.count("maxpool") == 3
    assert ops.count("resize") == 2 and ops.count("add") == 7 and ops.count("s2d") == 1
    assert len(qg.output_nodes) == 3
    x = rng.random((2, 128, 128, 3), dtype=f32)
    wants, outs = netref.run_integer(qg, x, keep_all=True)
    for capture, fuse in ((False, False), (False, True), (True, True)):
        model = nb.HipModel(hip_ctx, qg, 2, capture_graph=capture, fuse_residual=fuse)
        model.run(x)
        # fused: every conv takes its swish table into the epilogue (the detect convs aside), the seven bottleneck
        # adds go in as well; the input's quantisation is done by the pack of 2 x 2 pixel blocks in front of the stem
        # and 17 convs whose result only feeds a concat write their slice of the concat's tensor themselves (their
        # requantisation to the concat's quant params composed with their tables), which leaves 6 of the 13 concat
        # operators, with fewer inputs each
        # ; the three detect convs store the dequantised outputs themselves
        assert (len(model.fused_lut), len(model.fused_into), len(model.write_through), len(model.fused_quant), len(model.fused_dequant),
                len(model.fn)) == ((57, 7, 17, 1, 3, 147 - 64 - 7 - 1 - 3 - 11) if fuse else (0, 0, 0, 0, 0, 147))
        assert len(model.pairs) == (11 if fuse else 0)     # 1x1 convolutions that read a 1x1 convolution run as one launch with it
        for i, ref in enumerate(outs):
            if not model.materialized(i):
                continue
            got = model.tensor(i)
            assert np.array_equal(got, ref), f"node {i} ({qg.nodes[i].name}, {qg.nodes[i].op}): {(got != ref).sum()} of {ref.size} bytes differ"
        for got, want in zip(model.all_outputs(), wants):
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # the zero-padded 4th stem channel and the fold of 2 x 2 pixel blocks into channels change nothing: the stem conv, a
    # 3x3 window of stride 1 over 16 channels of the half-size image, equals the 6x6 stride-2 convolution over RGB
    stem = next(i for i, n in enumerate(qg.nodes) if n.op == "conv")
    n, src = qg.nodes[stem], qg.nodes[0]
    assert n.weights.shape[1:] == (16, 3, 3) and tuple(n.stride) == (1, 1) and tuple(map(tuple, n.padding)) == ((1, 1), (1, 1))
    w66 = np.empty((n.weights.shape[0], 3, 6, 6), np.uint8)
    for dy in range(2):
        for dx in range(2):
            w66[:, :, dy::2, dx::2] = n.weights[:, (dy * 2 + dx) * 4:(dy * 2 + dx) * 4 + 3]
    plain = O.qconv2d(outs[0], w66, n.bias, src.out_qp[0], src.out_qp[1], n.w_qp[0], n.w_qp[1], n.out_qp[0], n.out_qp[1],
                      (2, 2), ((2, 2), (2, 2)), (1, 1), 1, n.clamp, O.OUT_U8)
    assert np.array_equal(plain, outs[stem])
    # float model vs quantised model: the reference's acceptance bar
    fl = nb.float_forward(g, x)
    for want, j in zip(wants, g.outputs):
        assert O.cosine(want, fl[j]) > 0.98
    loaded = rt.LoadedKModel(hip_ctx, km.compile_quant_graph(qg, 2))
    assert len(loaded.fn) == 147 - 64 - 7 - 1 - 3 - 11   # the native loader folds the same tables, adds, concat slices, quantize, dequantizes, pairs
    ys = loaded.run(x)
    assert len(ys) == 3
    for y, want in zip(ys, wants):
        assert np.array_equal(y.transpose(0, 3, 1, 2).view(np.uint32), want.view(np.uint32))


def test_yolov5s_batch_consistency_at_larger_size(hip_ctx):
    """Size-independent property at a size the oracle does not follow: 320 x 320 at batch 8 equals the same
    images at batch 1, tensor by tensor."""
    g = nb.yolov5s(seed=4, input_hw=320)
    rng = np.random.default_rng(7)
    qg = nb.quantize_graph(g, rng.random((2, 320, 320, 3), dtype=f32))
    x = rng.random((8, 320, 320, 3), dtype=f32)
    big = nb.HipModel(hip_ctx, qg, 8, capture_graph=True)
    big.run(x)
    for img in (0, 7):
        one = nb.HipModel(hip_ctx, qg, 1, capture_graph=False)
        one.run(x[img:img + 1])
        for i in range(len(qg.nodes)):
            if not big.materialized(i):
                continue
            a, b = big.tensor(i)[img:img + 1], one.tensor(i)
            assert np.array_equal(a, b), f"node {i} ({qg.nodes[i].name}), image {img}: {(a != b).sum()} bytes differ"


def test_yolov5s_config4_at_640_batch_16(hip_ctx):
    """BASELINE config 4 at full size: 640 x 640, batch 16.  Image 0 of the batch equals the oracle on every u8
    tensor and on the three dequantised heads; images 0 and 15 of the batch-16 run equal their batch-1 runs
    tensor by tensor (the property that does not need the oracle at this size)."""
    g = nb.yolov5s(seed=4, input_hw=640)
    rng = np.random.default_rng(7)
    qg = nb.quantize_graph(g, rng.random((2, 640, 640, 3), dtype=f32), calib_batch=1)
    x = rng.random((16, 640, 640, 3), dtype=f32)
    big = nb.HipModel(hip_ctx, qg, 16, capture_graph=True)
    big.run(x)
    heads16 = big.all_outputs()
    wants, outs = netref.run_integer(qg, x[:1], keep_all=True)
    for i, ref in enumerate(outs):
        if big.materialized(i):
            got = big.tensor(i)[:1]
            assert np.array_equal(got, ref), f"node {i} ({qg.nodes[i].name}, {qg.nodes[i].op}): {(got != ref).sum()} of {ref.size} bytes differ"
    for got, want in zip(heads16, wants):
        assert np.array_equal(got[:1].view(np.uint32), want.view(np.uint32))
    one = nb.HipModel(hip_ctx, qg, 1, capture_graph=False)
    for img in (0, 15):
        one.run(x[img:img + 1])
        for i in range(len(qg.nodes)):
            if big.materialized(i):
                a, b = big.tensor(i)[img:img + 1], one.tensor(i)
                assert np.array_equal(a, b), f"node {i} ({qg.nodes[i].name}), image {img}: {(a != b).sum()} bytes differ"
        for a, b in zip(heads16, one.all_outputs()):
            assert np.array_equal(a[img:img + 1].view(np.uint32), b.view(np.uint32))


def test_profile_and_kernel_names(hip_ctx):
    g = nb.conv_block(seed=1)
    rng = np.random.default_rng(1)
    qg = nb.quantize_graph(g, rng.random((4, 56, 56, 64), dtype=f32))
    model = nb.HipModel(hip_ctx, qg, 2, capture_graph=False)
    names = [model.fn.op_kernel(i) for i in range(len(model.fn))]
    assert names[0] == "quantize" and names[2] == "dw3x3<S=1>" and len(names) == 4
    assert names[1].startswith("qconv_igemm<T=") and names[3].startswith("qconv_igemm+dequantize<T=")   # (the output's Dequantize
    assert all(n.endswith(",rows16>") for n in (names[1], names[3]))                                     # is the last conv's store)
    ms = model.fn.profile(3)
    assert len(ms) == 4 and all(0 < t < 50 for t in ms)
    fused = nb.HipModel(hip_ctx, qg, 2, capture_graph=False, fuse_blocks="all")
    assert [fused.fn.op_kernel(i) for i in range(len(fused.fn))] == ["quantize", "qblock<S=1,P=4>", "dequantize"]
    assert fused.op_members == [[0], [1, 2, 3], []]


@pytest.mark.parametrize("lanes,capture", [(2, True), (4, True), (2, False)])
def test_lanes_split_the_batch_bit_exact(hip_ctx, lanes, capture):
    """A function recorded as `lanes` independent chains over image ranges (replayed on concurrent streams
    when captured) writes the same bytes into every tensor as the single-chain function, replay after replay."""
    g = nb.mobilenet_v2(seed=2)
    rng = np.random.default_rng(3)
    qg = nb.quantize_graph(g, rng.random((32, 224, 224, 3), dtype=f32))
    x = np.random.default_rng(4).random((16, 224, 224, 3), dtype=f32)
    one = nb.HipModel(hip_ctx, qg, 16, capture_graph=False, fuse_blocks="all")
    y1 = one.run(x)
    many = nb.HipModel(hip_ctx, qg, 16, capture_graph=capture, lanes=lanes, fuse_blocks="all")
    assert len(many.fn) == lanes * len(one.fn) and len(many.op_names) == len(one.op_names)
    y = many.run(x)
    assert np.array_equal(y.view(np.uint32), y1.view(np.uint32))
    for i in range(len(qg.nodes)):
        if one.materialized(i):
            a, b = one.tensor(i), many.tensor(i)
            assert np.array_equal(a, b), f"node {i} ({qg.nodes[i].name}): {(a != b).sum()} bytes differ"
    x2 = np.random.default_rng(5).random((16, 224, 224, 3), dtype=f32)
    y2 = one.run(x2)
    for r in range(3):                      # replays with eager work and other inputs in between
        assert np.array_equal(many.run(x2).view(np.uint32), y2.view(np.uint32)), f"replay {r}"
        one.fn.invoke_one(1)
        hip_ctx.sync()
        assert np.array_equal(many.run(x).view(np.uint32), y1.view(np.uint32)), f"replay {r}"


def test_queue_pool_is_filled_once(hip_ctx):
    """The idle streams that spread later contexts over the hardware queues are created once per process; the call
    reports the number of hardware queues (HIP's default of 4 unless GPU_MAX_HW_QUEUES says otherwise)."""
    import os
    from nncase_amd import runtime as rt
    want = int(os.environ.get("GPU_MAX_HW_QUEUES", "4") or 4)
    assert rt.fill_queue_pool(0) == want and rt.fill_queue_pool(0) == want
    with pytest.raises(rt.HipError) as e:
        rt.fill_queue_pool(999)
    assert e.value.code == -19


def test_copies_in_flight_give_the_bytes_of_one_function(hip_ctx):
    """HipPipeline: steps enqueued in turn on copies of the function (own stream, own buffers) overlap on the device;
    every copy still holds the bytes a single function computes, whatever was in flight beside it."""
    g = nb.mobilenet_v2(seed=2)
    qg = nb.quantize_graph(g, np.random.default_rng(3).random((32, 224, 224, 3), dtype=f32))
    xs = [np.random.default_rng(40 + i).random((8, 224, 224, 3), dtype=f32) for i in range(3)]
    one = nb.HipModel(hip_ctx, qg, 8, capture_graph=False)
    want = [one.run(x).copy() for x in xs]
    pipe = nb.HipPipeline(0, qg, 8, depth=3, capture_graph=True)
    for m, x in zip(pipe.models, xs):         # a different batch on every copy
        m.set_input(x)
    for _ in range(4):                        # 12 steps back to back, 3 in flight
        used = [pipe.submit() for _ in range(3)]
    assert used == pipe.models
    pipe.sync()
    for m, y in zip(pipe.models, want):
        assert np.array_equal(m.output().view(np.uint32), y.view(np.uint32))
    with pytest.raises(ValueError):
        nb.HipPipeline(0, qg, 8, depth=0)
    # the idle streams that spread the copies over the hardware queues go with the pipeline; a later one fills the pool again
    queues = pipe.hw_queues
    pipe.close()
    assert rt.release_queue_pool(0) == 0                      # already released
    again = nb.HipPipeline(0, qg, 8, depth=2, capture_graph=False)
    assert again.hw_queues == queues
    again.models[0].set_input(xs[0])
    again.submit()
    again.sync()
    assert np.array_equal(again.models[0].output().view(np.uint32), want[0].view(np.uint32))
    again.close()


def test_lanes_yolov5s_outputs(hip_ctx):
    g = nb.yolov5s(seed=5, input_hw=160)
    rng = np.random.default_rng(6)
    qg = nb.quantize_graph(g, rng.random((8, 160, 160, 3), dtype=f32))
    x = rng.random((4, 160, 160, 3), dtype=f32)
    one = nb.HipModel(hip_ctx, qg, 4, capture_graph=False)
    one.run(x)
    two = nb.HipModel(hip_ctx, qg, 4, capture_graph=True, lanes=2)
    two.run(x)
    for a, b in zip(one.all_outputs(), two.all_outputs()):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_lanes_argument_checks(hip_ctx):
    g = nb.conv_block(seed=1)
    qg = nb.quantize_graph(g, np.random.default_rng(1).random((4, 56, 56, 64), dtype=f32))
    with pytest.raises(ValueError):
        nb.HipModel(hip_ctx, qg, 3, lanes=2)
    with pytest.raises(ValueError):
        nb.HipModel(hip_ctx, qg, 18, lanes=9)
    from nncase_amd.runtime import Function, HipError
    fn = Function(hip_ctx)
    with pytest.raises(HipError):
        fn.set_lane(8)
    with pytest.raises(HipError):
        fn.set_lane(-2)
    # what is recorded behind the join of the lanes runs after all of them, and has to be recorded last
    a, b, c = (hip_ctx.alloc(64) for _ in range(3))
    a.upload(np.arange(64, dtype=np.uint8))
    table = ((np.arange(256) + 3) % 256).astype(np.uint8)
    fn.set_lane(0)
    fn.add_lut_u8(a.view(0, 32), b.view(0, 32), 32, table)
    fn.set_lane(1)
    fn.add_lut_u8(a.view(32, 32), b.view(32, 32), 32, table)
    fn.set_lane(Function.LANE_JOINED)
    fn.add_lut_u8(b, c, 64, table)
    fn.set_lane(1)
    with pytest.raises(HipError):
        fn.add_lut_u8(a, b, 64, table)
    for capture in (False, True):
        if capture:
            fn.capture()
        c.fill(0)
        fn.invoke()
        hip_ctx.sync()
        assert np.array_equal(c.download((64,), np.uint8), (np.arange(64) + 6).astype(np.uint8))


def test_mobilenetv2_fused_blocks_match_separate_operators(hip_ctx):
    """All 16 expand -> depthwise -> project blocks as single fused operators: every tensor that still reaches
    HBM equals the one the operator-per-convolution function writes, and the oracle's logits for image 0."""
    g = nb.mobilenet_v2(seed=2)
    rng = np.random.default_rng(3)
    qg = nb.quantize_graph(g, rng.random((32, 224, 224, 3), dtype=f32))
    x = np.random.default_rng(4).random((8, 224, 224, 3), dtype=f32)
    plain = nb.HipModel(hip_ctx, qg, 8, capture_graph=False, fuse_blocks=False, fuse_pairs=False)
    y0 = plain.run(x)
    for capture, lanes in ((False, 1), (True, 1), (True, 2)):
        fused = nb.HipModel(hip_ctx, qg, 8, capture_graph=capture, lanes=lanes, fuse_blocks="all")
        assert len(fused.blocks) == 16 and len(fused.fn) == lanes * (len(plain.fn) - 32)
        y = fused.run(x)
        assert np.array_equal(y.view(np.uint32), y0.view(np.uint32))
        for i in range(len(qg.nodes)):
            if fused.materialized(i):
                a, b = plain.tensor(i), fused.tensor(i)
                assert np.array_equal(a, b), f"node {i} ({qg.nodes[i].name}): {(a != b).sum()} bytes differ"
        for e, (d, _, _) in fused.blocks.items():
            assert not fused.materialized(e) and not fused.materialized(d)
    want = netref.run_integer(qg, x[:1])
    want = want[0] if isinstance(want, tuple) else want
    assert np.array_equal(y0[:1].view(np.uint32), np.asarray(want).view(np.uint32))
