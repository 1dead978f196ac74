"""Builds the quantised graphs of the benchmark configurations on the host and binds them to
a resident `hip` function.

What the reference's compiler does for a "u8/u8" model and this module reproduces:
  * fold BatchNorm into the preceding conv: scale = gamma / sqrt(var + eps),
    bias = beta - gamma * mean / sqrt(var + eps)   (src/Nncase.Passes/Rules/Neutral/BatchNormToBinary.cs:23-50)
  * ReLU6 -> Clamp(0, 6) fused into the conv as fused_clamp, applied to the float value before
    the Quantize                                       (ReluToClamp.cs:39-48, FuseClampConv2D.cs:22-38)
  * PTQ: running finite min/max of every activation over the calibration set (NoClip), the
    calibrator's FixUpRange, GetQuantParam(UnsignedMode, 8 bits)
                                                       (Quantizer.cs:358-408, QuantUtility.cs:41-97)
  * per-tensor asymmetric u8 weights, int32 bias with quant param (0, sx * sw)
                                                       (QLinearConv.cs:73)
The float forward pass used for calibration runs on the host (numpy); it plays the role of the
reference's Evaluator during calibration and is not part of the timed path.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import quant
from . import runtime as rt
from .runtime import Context, Function, qp

f32 = np.float32
FULL_CLAMP = (-rt.FLT_MAX, rt.FLT_MAX)


# --------------------------------------------------------------------------------------------- float graph
@dataclass
class Node:
    op: str                      # "input" | "conv" | "add" | "gap"
    inputs: Tuple[int, ...] = ()
    name: str = ""
    # conv
    weights: Optional[np.ndarray] = None   # OIHW float32 (BN already folded)
    bias: Optional[np.ndarray] = None      # float32 [O]
    stride: Tuple[int, int] = (1, 1)
    padding: Tuple[Tuple[int, int], Tuple[int, int]] = ((0, 0), (0, 0))
    groups: int = 1
    clamp: Tuple[float, float] = FULL_CLAMP


@dataclass
class FloatGraph:
    nodes: List[Node] = field(default_factory=list)
    input_shape: Tuple[int, int, int] = (224, 224, 3)  # H, W, C (NHWC at the boundary)

    def add(self, node: Node) -> int:
        self.nodes.append(node)
        return len(self.nodes) - 1


def _kaiming(rng, shape):
    fan_in = shape[1] * shape[2] * shape[3]
    return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(f32)


def _conv_bn(rng, g: FloatGraph, src: int, cin: int, cout: int, k: int, stride: int, groups: int, relu6: bool, name: str) -> int:
    w = _kaiming(rng, (cout, cin // groups, k, k))
    gamma = rng.uniform(0.8, 1.2, cout).astype(f32)
    beta = (rng.standard_normal(cout) * 0.1).astype(f32)
    mean = (rng.standard_normal(cout) * 0.1).astype(f32)
    var = rng.uniform(0.8, 1.2, cout).astype(f32)
    scale = gamma / np.sqrt(var + f32(1e-5))
    w = (w * scale.reshape(-1, 1, 1, 1)).astype(f32)
    b = (beta - gamma * mean / np.sqrt(var + f32(1e-5))).astype(f32)
    p = (k - 1) // 2
    return g.add(Node("conv", (src,), name, w, b, (stride, stride), ((p, p), (p, p)), groups,
                      (0.0, 6.0) if relu6 else FULL_CLAMP))


def mobilenet_v2(seed: int = 2, num_classes: int = 1000, input_hw: int = 224) -> FloatGraph:
    """MobileNetV2, width 1.0, torchvision layer table, random Kaiming weights, BN folded."""
    rng = np.random.default_rng(seed)
    g = FloatGraph(input_shape=(input_hw, input_hw, 3))
    x = g.add(Node("input", name="input"))
    x = _conv_bn(rng, g, x, 3, 32, 3, 2, 1, True, "stem")
    cin = 32
    cfg = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]
    bi = 0
    for t, c, n, s in cfg:
        for i in range(n):
            stride = s if i == 0 else 1
            inp = x
            hidden = cin * t
            if t != 1:
                x = _conv_bn(rng, g, x, cin, hidden, 1, 1, 1, True, f"b{bi}.expand")
            x = _conv_bn(rng, g, x, hidden, hidden, 3, stride, hidden, True, f"b{bi}.dw")
            x = _conv_bn(rng, g, x, hidden, c, 1, 1, 1, False, f"b{bi}.project")
            if stride == 1 and cin == c:
                x = g.add(Node("add", (inp, x), f"b{bi}.add"))
            cin = c
            bi += 1
    x = _conv_bn(rng, g, x, cin, 1280, 1, 1, 1, True, "head")
    x = g.add(Node("gap", (x,), "pool"))
    w = (rng.standard_normal((num_classes, 1280, 1, 1)) * 0.01).astype(f32)
    g.add(Node("conv", (x,), "fc", w, np.zeros(num_classes, f32)))
    return g


def conv_block(seed: int = 1) -> FloatGraph:
    """1x1 64->144, 3x3 depthwise, 1x1 144->64 on 56x56, ReLU6 after each."""
    rng = np.random.default_rng(seed)
    g = FloatGraph(input_shape=(56, 56, 64))
    x = g.add(Node("input", name="input"))
    for name, cin, cout, k, groups in (("pw1", 64, 144, 1, 1), ("dw", 144, 144, 3, 144), ("pw2", 144, 64, 1, 1)):
        w = _kaiming(rng, (cout, cin // groups, k, k))
        b = (rng.standard_normal(cout) * 0.01).astype(f32)
        p = (k - 1) // 2
        x = g.add(Node("conv", (x,), name, w, b, (1, 1), ((p, p), (p, p)), groups, (0.0, 6.0)))
    return g


# --------------------------------------------------------------------------------------------- host float pass
def _conv_float(x: np.ndarray, n: Node) -> np.ndarray:
    """NCHW float conv via im2col + matmul (calibration only)."""
    b, c, h, w = x.shape
    oc, gic, kh, kw = n.weights.shape
    (ph0, ph1), (pw0, pw1) = n.padding
    sh, sw = n.stride
    xp = np.pad(x, ((0, 0), (0, 0), (ph0, ph1), (pw0, pw1)))
    oh = (h + ph0 + ph1 - kh) // sh + 1
    ow = (w + pw0 + pw1 - kw) // sw + 1
    if n.groups == c and gic == 1 and oc == c:  # depthwise
        out = np.zeros((b, c, oh, ow), f32)
        for ky in range(kh):
            for kx in range(kw):
                out += xp[:, :, ky:ky + (oh - 1) * sh + 1:sh, kx:kx + (ow - 1) * sw + 1:sw] * n.weights[:, 0, ky, kx].reshape(1, -1, 1, 1)
    else:
        assert n.groups == 1
        cols = np.empty((b, gic, kh, kw, oh, ow), f32)
        for ky in range(kh):
            for kx in range(kw):
                cols[:, :, ky, kx] = xp[:, :, ky:ky + (oh - 1) * sh + 1:sh, kx:kx + (ow - 1) * sw + 1:sw]
        out = np.einsum("ok,bkp->bop", n.weights.reshape(oc, -1), cols.reshape(b, gic * kh * kw, oh * ow), optimize=True)
        out = out.reshape(b, oc, oh, ow).astype(f32)
    out += n.bias.reshape(1, -1, 1, 1)
    return np.clip(out, n.clamp[0], n.clamp[1]).astype(f32)


def float_forward(g: FloatGraph, x_nhwc: np.ndarray) -> List[np.ndarray]:
    """All node outputs (NCHW float32) for a batch of NHWC float32 inputs."""
    outs: List[np.ndarray] = []
    for n in g.nodes:
        if n.op == "input":
            y = np.ascontiguousarray(np.asarray(x_nhwc, f32).transpose(0, 3, 1, 2))
        elif n.op == "conv":
            y = _conv_float(outs[n.inputs[0]], n)
        elif n.op == "add":
            y = outs[n.inputs[0]] + outs[n.inputs[1]]
        elif n.op == "gap":
            y = outs[n.inputs[0]].mean(axis=(2, 3), keepdims=True).astype(f32)
        else:
            raise ValueError(n.op)
        outs.append(y)
    return outs


# --------------------------------------------------------------------------------------------- quantised graph
@dataclass
class QNode:
    op: str
    inputs: Tuple[int, ...]
    name: str
    out_qp: Tuple[int, np.float32]          # (zero_point, scale) of this node's u8 output
    out_shape: Tuple[int, int, int]          # C, H, W per image
    weights: Optional[np.ndarray] = None     # OIHW uint8
    w_qp: Optional[Tuple[int, np.float32]] = None
    bias: Optional[np.ndarray] = None        # int32
    stride: Tuple[int, int] = (1, 1)
    padding: Tuple[Tuple[int, int], Tuple[int, int]] = ((0, 0), (0, 0))
    groups: int = 1
    clamp: Tuple[float, float] = FULL_CLAMP


@dataclass
class QuantGraph:
    """u8/u8 graph: float32 NHWC input -> Quantize -> u8 nodes -> Dequantize -> float32 output."""
    nodes: List[QNode]
    input_shape: Tuple[int, int, int]

    @property
    def macs_per_image(self) -> Dict[str, int]:
        dense = dw = 0
        for n in self.nodes:
            if n.op != "conv":
                continue
            oc, gic, kh, kw = n.weights.shape
            m = oc * n.out_shape[1] * n.out_shape[2] * gic * kh * kw
            if n.groups > 1 and gic == 1:
                dw += m
            else:
                dense += m
        return {"dense": dense, "depthwise": dw}


def quantize_graph(g: FloatGraph, calib_nhwc: np.ndarray, calib_batch: int = 8) -> QuantGraph:
    """Per-tensor PTQ with min/max (NoClip) calibration over `calib_nhwc`."""
    ranges: List[Optional[Tuple[np.float32, np.float32]]] = [None] * len(g.nodes)
    shapes: List[Tuple[int, int, int]] = [None] * len(g.nodes)
    for s in range(0, len(calib_nhwc), calib_batch):
        outs = float_forward(g, calib_nhwc[s:s + calib_batch])
        for i, y in enumerate(outs):
            r = quant.range_of(y)
            ranges[i] = r if ranges[i] is None else quant.union(ranges[i], r)
            shapes[i] = tuple(y.shape[1:])
    qnodes: List[QNode] = []
    for i, n in enumerate(g.nodes):
        zp, sc = quant.get_quant_param(quant.calib_fixup_range(ranges[i]), 8, quant.QuantMode.UnsignedMode)
        qn = QNode(n.op, n.inputs, n.name, (zp, sc), shapes[i])
        if n.op == "conv":
            wq, zw, sw = quant.quantize_weights(n.weights)
            sx = qnodes[n.inputs[0]].out_qp[1]
            bscale = f32(sx) * f32(sw)  # bias quant param is (0, sx * sw)
            qn.weights, qn.w_qp = wq, (zw, sw)
            qn.bias = np.clip(np.rint(n.bias / bscale), -2 ** 31, 2 ** 31 - 1).astype(np.int32)
            qn.stride, qn.padding, qn.groups, qn.clamp = n.stride, n.padding, n.groups, n.clamp
        qnodes.append(qn)
    return QuantGraph(qnodes, g.input_shape)


# --------------------------------------------------------------------------------------------- device binding
class HipModel:
    """A QuantGraph resident on the device: packed weights, one HBM buffer per tensor, and the
    operator list recorded in a `hip` function.  run() = upload input, invoke, download output."""

    def __init__(self, ctx: Context, qg: QuantGraph, batch: int, capture_graph: bool = True, fuse_residual: bool = True):
        self.ctx, self.qg, self.batch = ctx, qg, batch
        h, w, c = qg.input_shape
        self.in_count = batch * h * w * c
        self.input_f32 = ctx.alloc(self.in_count * 4)
        self.fn = Function(ctx)
        self.buffers: List[Optional[rt.DeviceBuffer]] = []
        self.weights: List[Optional[rt.Weights]] = []
        self.op_names: List[str] = []
        self.op_nodes: List[int] = []
        # A residual add whose second operand is a dense conv consumed by nothing else is folded into
        # that conv's epilogue (the conv's own u8 tensor is then never written).
        consumers = [0] * len(qg.nodes)
        for n in qg.nodes:
            for j in n.inputs:
                consumers[j] += 1
        self.fused_into: Dict[int, int] = {}   # conv node -> add node
        if fuse_residual:
            for i, n in enumerate(qg.nodes):
                if n.op == "add":
                    a, b = n.inputs
                    nb_ = qg.nodes[b]
                    dense = nb_.op == "conv" and not (nb_.groups > 1 and nb_.weights.shape[1] == 1) and nb_.weights.shape[1] * nb_.groups > 4
                    if dense and consumers[b] == 1 and b == i - 1 and a < b:
                        self.fused_into[b] = i
        for i, n in enumerate(qg.nodes):
            cc, hh, ww = n.out_shape
            fused_add = self.fused_into.get(i)
            if n.op == "add" and i in self.fused_into.values():
                self.buffers.append(self.buffers[i - 1])  # written by the fused conv
                self.weights.append(None)
                continue
            buf = ctx.alloc(batch * cc * hh * ww)
            self.buffers.append(buf)
            self.weights.append(None)
            if n.op == "input":
                self.fn.add_quantize(self.input_f32, rt.DT_F32, buf, rt.DT_U8, self.in_count, qp(*n.out_qp))
            elif n.op == "conv":
                src = qg.nodes[n.inputs[0]]
                wt = ctx.prepack_conv2d(n.weights, n.bias, qp(*n.w_qp), n.groups, expected_pixels=batch * hh * ww)
                self.weights[-1] = wt
                (ph0, ph1), (pw0, pw1) = n.padding
                args = rt.Conv2dArgs(batch, src.out_shape[1], src.out_shape[2], n.stride[0], n.stride[1], 1, 1, ph0, ph1, pw0,
                                     pw1, qp(*src.out_qp), qp(*n.out_qp), n.clamp[0], n.clamp[1], rt.DT_U8)
                if fused_add is not None:
                    add = qg.nodes[fused_add]
                    res_node = add.inputs[0]
                    args.residual_dev = self.buffers[res_node].ptr
                    args.residual_qp = qp(*qg.nodes[res_node].out_qp)
                    args.sum_qp = qp(*add.out_qp)
                    args.sum_clamp_min, args.sum_clamp_max = FULL_CLAMP
                    self.fn._keep.append(self.buffers[res_node])
                self.fn.add_qconv2d(self.buffers[n.inputs[0]], wt, buf, args)
            elif n.op == "add":
                a, b = (qg.nodes[j] for j in n.inputs)
                self.fn.add_qadd(self.buffers[n.inputs[0]], qp(*a.out_qp), self.buffers[n.inputs[1]], qp(*b.out_qp), buf,
                                 qp(*n.out_qp), batch * cc * hh * ww)
            elif n.op == "gap":
                src = qg.nodes[n.inputs[0]]
                self.fn.add_qglobal_avgpool(self.buffers[n.inputs[0]], buf, batch, src.out_shape[1], src.out_shape[2],
                                            src.out_shape[0], qp(*src.out_qp), qp(*n.out_qp))
            else:
                raise ValueError(n.op)
            self.op_names.append(f"{n.op}:{n.name}" + ("+add" if fused_add is not None else ""))
            self.op_nodes.append(i if fused_add is None else fused_add)
        last = qg.nodes[-1]
        self.out_shape = (batch,) + tuple(last.out_shape)
        self.out_count = int(np.prod(self.out_shape))
        self.output_f32 = ctx.alloc(self.out_count * 4)
        self.fn.add_dequantize(self.buffers[-1], rt.DT_U8, self.output_f32, rt.DT_F32, self.out_count, qp(*last.out_qp))
        self.op_names.append("dequantize:output")
        self.op_nodes.append(len(qg.nodes) - 1)
        if capture_graph:
            self.fn.capture()

    def set_input(self, x_nhwc: np.ndarray):
        x = np.ascontiguousarray(x_nhwc, f32)
        assert x.size == self.in_count, f"expected {self.in_count} input elements, got {x.size}"
        self.input_f32.upload(x)

    def invoke(self):
        self.fn.invoke()

    def output(self) -> np.ndarray:
        """Dequantised float32 output, NCHW-shaped [batch, C, H, W] (H = W = 1 for classifiers)."""
        c, h, w = self.qg.nodes[-1].out_shape
        y = self.output_f32.download((self.batch, h, w, c), f32)
        return np.ascontiguousarray(y.transpose(0, 3, 1, 2))

    def materialized(self, node: int) -> bool:
        """False for a conv whose output only exists inside a fused residual add."""
        return node not in self.fused_into

    def tensor(self, node: int) -> np.ndarray:
        """u8 output of a node as NCHW (for layer-by-layer parity checks)."""
        if not self.materialized(node):
            raise ValueError(f"node {node} is fused into node {self.fused_into[node]} and never written")
        c, h, w = self.qg.nodes[node].out_shape
        y = self.buffers[node].download((self.batch, h, w, c), np.uint8)
        return np.ascontiguousarray(y.transpose(0, 3, 1, 2))

    def run(self, x_nhwc: np.ndarray) -> np.ndarray:
        self.set_input(x_nhwc)
        self.invoke()
        self.ctx.sync()
        return self.output()
