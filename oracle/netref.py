"""Runs a quantised graph (nncase_amd.netbuilder.QuantGraph, used here as plain data) through
the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Byte-table, concat, resize, max-pool and channel-padding nodes are byte-exact in both runs (the CPU
target evaluates them between Dequantize and Quantize with the same fp32 formulas the tables hold).

run_integer(): node by node with the integer-exact operator definitions -- the values the
               HIP path must reproduce bit for bit.
run_float_chain(): what nncase's CPU target executes for the same model, every quantised conv
               as Dequantize -> float Conv2D(fused_clamp) -> Quantize with the loop-for-loop
               restatement of its kernels (src/Nncase.Importer/Onnx/QLinearConv.cs:61-75,
               src/Native/src/kernels/stackvm/reference/convolution.cpp:26-105).  This is the
               timed CPU baseline and the <= 1 LSB cross-check.
"""
from __future__ import annotations

from typing import List

import numpy as np

from . import oracle as O


def _input(qg, x_nhwc):
    x = np.ascontiguousarray(np.asarray(x_nhwc, np.float32).transpose(0, 3, 1, 2))
    zp, sc = qg.nodes[0].out_qp
    return O.quantize(x, sc, zp, O.U8)


def run_integer(qg, x_nhwc: np.ndarray, keep_all: bool = False):
    """Returns (float32 dequantised output NCHW, list of u8 node outputs NCHW if keep_all)."""
    outs: List[np.ndarray] = []
    for n in qg.nodes:
        if n.op == "input":
            y = _input(qg, x_nhwc)
        elif n.op == "conv":
            src = qg.nodes[n.inputs[0]]
            y = O.qconv2d(outs[n.inputs[0]], n.weights, n.bias, src.out_qp[0], src.out_qp[1], n.w_qp[0], n.w_qp[1],
                          n.out_qp[0], n.out_qp[1], n.stride, n.padding, (1, 1), n.groups, n.clamp, O.OUT_U8)
        elif n.op == "add":
            a, b = (qg.nodes[j] for j in n.inputs)
            y = O.qadd(outs[n.inputs[0]], outs[n.inputs[1]], a.out_qp[0], a.out_qp[1], b.out_qp[0], b.out_qp[1],
                       n.out_qp[0], n.out_qp[1])
        elif n.op == "gap":
            src = qg.nodes[n.inputs[0]]
            y = O.qglobal_avgpool(outs[n.inputs[0]], src.out_qp[0], src.out_qp[1], n.out_qp[0], n.out_qp[1])
            y = y.reshape(y.shape[0], y.shape[1], 1, 1)
        elif n.op == "lut":
            src = qg.nodes[n.inputs[0]]
            y = O.unary_lut(O.LUT_SWISH, src.out_qp[0], src.out_qp[1], n.out_qp[0], n.out_qp[1])[outs[n.inputs[0]]]
        elif n.op == "concat":
            y = O.qconcat([outs[j] for j in n.inputs], [qg.nodes[j].out_qp for j in n.inputs], n.out_qp)
        elif n.op == "resize":
            c, h, w = n.out_shape
            y = O.resize_nearest(outs[n.inputs[0]], h, w, n.resize_modes[0], n.resize_modes[1])
        elif n.op == "maxpool":
            src = qg.nodes[n.inputs[0]]
            k, st, p = n.pool
            y = O.qmaxpool(outs[n.inputs[0]], (k, k), (st, st), ((p, p), (p, p)), src.out_qp[0], src.out_qp[1], n.out_qp[0], n.out_qp[1])
        elif n.op == "padc":
            v = outs[n.inputs[0]]
            y = np.pad(v, ((0, 0), (0, n.out_shape[0] - v.shape[1]), (0, 0), (0, 0)))
        elif n.op == "s2d":       # 2 x 2 pixel blocks of <= 4 channels -> 16 channels: y[:, (dy * 2 + dx) * 4 + c, y', x'] = v[:, c, 2 y' + dy, 2 x' + dx]
            v = outs[n.inputs[0]]
            nb_, c_, h_, w_ = v.shape
            v4 = np.pad(v, ((0, 0), (0, 4 - c_), (0, 0), (0, 0)))
            y = np.ascontiguousarray(v4.reshape(nb_, 4, h_ // 2, 2, w_ // 2, 2).transpose(0, 3, 5, 1, 2, 4).reshape(nb_, 16, h_ // 2, w_ // 2))
        elif n.op == "fold2":     # pixel pairs along the width become channels: y[:, dx * C + c, :, x] = v[:, c, :, 2 x + dx]
            v = outs[n.inputs[0]]
            nb_, c_, h_, w_ = v.shape
            y = np.ascontiguousarray(v.reshape(nb_, c_, h_, w_ // 2, 2).transpose(0, 4, 1, 2, 3).reshape(nb_, 2 * c_, h_, w_ // 2))
        else:
            raise ValueError(n.op)
        outs.append(y)
    finals = [O.dequantize(outs[j], qg.nodes[j].out_qp[1], qg.nodes[j].out_qp[0]) for j in qg.output_nodes]
    final = finals[0] if len(finals) == 1 else finals
    return (final, outs) if keep_all else (final, None)


def run_float_chain(qg, x_nhwc: np.ndarray, keep_all: bool = False):
    """The CPU target's execution of the same graph (float kernels between DQ / Q)."""
    outs: List[np.ndarray] = []
    for n in qg.nodes:
        if n.op == "input":
            y = _input(qg, x_nhwc)
        elif n.op == "conv":
            src = qg.nodes[n.inputs[0]]
            y = O.qconv2d_float_chain(outs[n.inputs[0]], n.weights, n.bias, src.out_qp[0], src.out_qp[1], n.w_qp[0],
                                      n.w_qp[1], n.out_qp[0], n.out_qp[1], n.stride, n.padding, (1, 1), n.groups, n.clamp)
        elif n.op == "add":
            a, b = (qg.nodes[j] for j in n.inputs)
            fa = O.dequantize(outs[n.inputs[0]], a.out_qp[1], a.out_qp[0])
            fb = O.dequantize(outs[n.inputs[1]], b.out_qp[1], b.out_qp[0])
            y = O.quantize(fa + fb, n.out_qp[1], n.out_qp[0], O.U8)
        elif n.op == "gap":
            src = qg.nodes[n.inputs[0]]
            xf = O.dequantize(outs[n.inputs[0]], src.out_qp[1], src.out_qp[0])
            m = O.reduce_window2d_mean_f32(xf, xf.shape[2:], (1, 1))
            y = O.quantize(m, n.out_qp[1], n.out_qp[0], O.U8)
        elif n.op == "lut":
            src = qg.nodes[n.inputs[0]]
            y = O.unary_lut(O.LUT_SWISH, src.out_qp[0], src.out_qp[1], n.out_qp[0], n.out_qp[1])[outs[n.inputs[0]]]
        elif n.op == "concat":
            y = O.qconcat([outs[j] for j in n.inputs], [qg.nodes[j].out_qp for j in n.inputs], n.out_qp)
        elif n.op == "resize":
            c, h, w = n.out_shape
            y = O.resize_nearest(outs[n.inputs[0]], h, w, n.resize_modes[0], n.resize_modes[1])
        elif n.op == "maxpool":
            src = qg.nodes[n.inputs[0]]
            k, st, p = n.pool
            y = O.qmaxpool(outs[n.inputs[0]], (k, k), (st, st), ((p, p), (p, p)), src.out_qp[0], src.out_qp[1], n.out_qp[0], n.out_qp[1])
        elif n.op == "padc":
            v = outs[n.inputs[0]]
            y = np.pad(v, ((0, 0), (0, n.out_shape[0] - v.shape[1]), (0, 0), (0, 0)))
        elif n.op == "s2d":       # 2 x 2 pixel blocks of <= 4 channels -> 16 channels: y[:, (dy * 2 + dx) * 4 + c, y', x'] = v[:, c, 2 y' + dy, 2 x' + dx]
            v = outs[n.inputs[0]]
            nb_, c_, h_, w_ = v.shape
            v4 = np.pad(v, ((0, 0), (0, 4 - c_), (0, 0), (0, 0)))
            y = np.ascontiguousarray(v4.reshape(nb_, 4, h_ // 2, 2, w_ // 2, 2).transpose(0, 3, 5, 1, 2, 4).reshape(nb_, 16, h_ // 2, w_ // 2))
        elif n.op == "fold2":     # pixel pairs along the width become channels: y[:, dx * C + c, :, x] = v[:, c, :, 2 x + dx]
            v = outs[n.inputs[0]]
            nb_, c_, h_, w_ = v.shape
            y = np.ascontiguousarray(v.reshape(nb_, c_, h_, w_ // 2, 2).transpose(0, 4, 1, 2, 3).reshape(nb_, 2 * c_, h_, w_ // 2))
        else:
            raise ValueError(n.op)
        outs.append(y)
    finals = [O.dequantize(outs[j], qg.nodes[j].out_qp[1], qg.nodes[j].out_qp[0]) for j in qg.output_nodes]
    final = finals[0] if len(finals) == 1 else finals
    return (final, outs) if keep_all else (final, None)
