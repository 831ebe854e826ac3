"""Writes tests/golden/golden.npz: expected outputs of PyTorch's CPU quantized
ops (engine 'fbgemm') for the seeded cases in tests/cases.py.

PyTorch's CPU ops are the numerics the reference's own tests compare against
(torch_musa/testing/base_test_tool.py:814-825); they are a third-party
dependency of the reference, not part of it, and are installed here.  Nothing
from the reference tree is imported or executed.

Run from the repo root:   python tests/golden/make_golden.py
The fixture holds only outputs, scalars and CRCs of the rebuilt inputs.
"""
from __future__ import annotations

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import cases  # noqa: E402


def qdtype(signed):
    return torch.qint8 if signed else torch.quint8


def put_dq(g, k, dq):
    """Dequantized values must match exactly, so a CRC pins them; small arrays
    are also kept in full to make a mismatch readable."""
    g[k + "/dq_crc"] = np.uint32(cases.crc(dq))
    if dq.size <= 2048:
        g[k + "/dq"] = dq


def main():
    torch.backends.quantized.engine = "fbgemm"
    torch.set_num_threads(4)
    g = {}
    meta = {"torch": torch.__version__, "engine": torch.backends.quantized.engine}

    # ---- per-tensor quantize / dequantize --------------------------------
    for c in cases.quantize_per_tensor_cases():
        x = torch.from_numpy(c["x"])
        q = torch.quantize_per_tensor(x, c["scale"], c["zp"], qdtype(c["signed"]))
        k = "qpt/" + c["name"]
        g[k + "/x_crc"] = np.uint32(cases.crc(c["x"]))
        g[k + "/q"] = q.int_repr().numpy()
        put_dq(g, k, q.dequantize().numpy())

    # ---- dynamic qparams -------------------------------------------------
    pairs = cases.dynamic_qparams_cases()
    res = []
    for mn, mx in pairs:
        for rr in (False, True):
            x = torch.tensor([mn, mx], dtype=torch.float32)
            s, z = torch._choose_qparams_per_tensor(x, rr)
            res.append((float(mn), float(mx), float(rr), float(s), float(z)))
    g["dynq/pairs"] = np.array(res, dtype=np.float64)
    for c in cases.dynamic_tensor_cases():
        x = torch.from_numpy(c["x"])
        for rr in (False, True):
            q = torch.quantize_per_tensor_dynamic(x, torch.quint8, rr)
            k = f"dyn/{c['name']}/rr{int(rr)}"
            g[k + "/x_crc"] = np.uint32(cases.crc(c["x"]))
            g[k + "/scale"] = np.float64(q.q_scale())
            g[k + "/zp"] = np.int64(q.q_zero_point())
            g[k + "/q"] = q.int_repr().numpy()

    # ---- per-channel -----------------------------------------------------
    for c in cases.quantize_per_channel_cases():
        x = torch.from_numpy(c["x"])
        q = torch.quantize_per_channel(x, torch.from_numpy(c["scales"].astype(np.float64)),
                                       torch.from_numpy(c["zps"].astype(np.int64)),
                                       c["axis"], qdtype(c["signed"]))
        k = "qpc/" + c["name"]
        g[k + "/x_crc"] = np.uint32(cases.crc(c["x"]))
        g[k + "/q"] = q.int_repr().numpy()
        put_dq(g, k, q.dequantize().numpy())

    # ---- per-channel, float scales / float zero points --------------------
    for c in cases.quantize_per_channel_float_cases():
        x = torch.from_numpy(c["x"])
        q = torch.quantize_per_channel(x, torch.from_numpy(c["scales"]), torch.from_numpy(c["zps"]),
                                       c["axis"], qdtype(c["signed"]))
        assert q.qscheme() == torch.per_channel_affine_float_qparams
        k = "qpcf/" + c["name"]
        g[k + "/x_crc"] = np.uint32(cases.crc(c["x"]))
        g[k + "/q"] = q.int_repr().numpy()
        put_dq(g, k, q.dequantize().numpy())

    # ---- quantized::linear (integer-domain cases) ------------------------
    def make_w(wq, w_scales, axis_len):
        wt = torch.from_numpy(wq)
        if len(w_scales) == 1:
            return torch._make_per_tensor_quantized_tensor(wt, float(w_scales[0]), 0)
        return torch._make_per_channel_quantized_tensor(
            wt, torch.from_numpy(w_scales.astype(np.float64)),
            torch.zeros(axis_len, dtype=torch.int64), 0)

    for c in cases.linear_cases():
        xq = torch._make_per_tensor_quantized_tensor(torch.from_numpy(c["xq"]),
                                                     c["x_scale"], c["x_zp"])
        w = make_w(c["wq"], c["w_scales"], c["wq"].shape[0])
        b = None if c["bias"] is None else torch.from_numpy(c["bias"])
        packed = torch.ops.quantized.linear_prepack(w, b)
        op = torch.ops.quantized.linear_relu if c["relu"] else torch.ops.quantized.linear
        y = op(xq, packed, c["out_scale"], c["out_zp"])
        k = "lin/" + c["name"]
        g[k + "/xq_crc"] = np.uint32(cases.crc(c["xq"]))
        g[k + "/wq_crc"] = np.uint32(cases.crc(c["wq"]))
        g[k + "/out_scale"] = np.float64(c["out_scale"])
        g[k + "/y"] = y.int_repr().numpy()

    # ---- per-tensor weight + bias: rows picked where the two ways of adding the bias
    # disagree after requantisation (a few outputs in a million), with the CPU op's
    # answer.  v = float(raw) + fl(bias / atw) is what the op computes for per-channel
    # weights, v = fma(bias, fl(1 / atw), float(raw)) for per-tensor ones.  The inputs
    # are stored with the outputs: finding them takes a search over 64 Mi candidates.
    f32 = np.float32
    rng = np.random.default_rng(2718)
    n_, k_, zp_, x_zp_ = 1024, 16, 128, 121
    xq_all = rng.integers(0, 256, (65536, k_), dtype=np.uint8)
    wq_ = rng.integers(-127, 128, (n_, k_), dtype=np.int8)
    bias_ = (rng.standard_normal(n_) * 30).astype(f32)
    x_scale_, w_scale_, out_scale_ = f32(0.031), f32(0.0027), f32(0.6)
    raw_ = (xq_all.astype(np.float64) - x_zp_) @ wq_.astype(np.float64).T      # exact in double
    atw_ = f32(x_scale_ * w_scale_)
    mult_ = f32(atw_ / out_scale_)
    v_div = raw_.astype(f32) + (bias_ / atw_).astype(f32)[None, :]
    v_fma = (bias_.astype(np.float64)[None, :] * np.float64(f32(f32(1) / atw_)) + raw_).astype(f32)
    q_div = np.rint((v_div * mult_).astype(f32))
    q_fma = np.rint((v_fma * mult_).astype(f32))
    inside = (q_fma + zp_ > 0) & (q_fma + zp_ < 255)
    rows_ = np.unique(np.nonzero((q_div != q_fma) & inside)[0])[:16]
    assert rows_.size >= 6, rows_.size
    xq_ = np.ascontiguousarray(xq_all[rows_])
    wt_ = torch._make_per_tensor_quantized_tensor(torch.from_numpy(wq_), float(w_scale_), 0)
    xt_ = torch._make_per_tensor_quantized_tensor(torch.from_numpy(xq_), float(x_scale_), x_zp_)
    y_ = torch.ops.quantized.linear(xt_, torch.ops.quantized.linear_prepack(wt_, torch.from_numpy(bias_)),
                                    float(out_scale_), zp_)
    g["ptbias/xq"], g["ptbias/wq"], g["ptbias/bias"] = xq_, wq_, bias_
    g["ptbias/params"] = np.array([float(x_scale_), x_zp_, float(w_scale_), float(out_scale_), zp_], dtype=np.float64)
    g["ptbias/y"] = y_.int_repr().numpy()
    want_div = np.clip(q_div[rows_] + zp_, 0, 255).astype(np.uint8)
    meta["ptbias_outputs_where_the_division_form_is_wrong"] = int((want_div != g["ptbias/y"]).sum())
    assert meta["ptbias_outputs_where_the_division_form_is_wrong"] >= 6

    # ---- quantized::linear_dynamic (float in, float out) ------------------------
    for c in cases.linear_dynamic_cases():
        w = make_w(c["wq"], c["w_scales"], c["wq"].shape[0])
        b = None if c["bias"] is None else torch.from_numpy(c["bias"])
        packed = torch.ops.quantized.linear_prepack(w, b)
        op = torch.ops.quantized.linear_relu_dynamic if c["relu"] else torch.ops.quantized.linear_dynamic
        y = op(torch.from_numpy(c["x"]), packed, c["reduce_range"])
        k = "lindyn/" + c["name"]
        g[k + "/x_crc"] = np.uint32(cases.crc(c["x"]))
        g[k + "/wq_crc"] = np.uint32(cases.crc(c["wq"]))
        g[k + "/y"] = y.numpy()

    # ---- plain-tensor int8 ops: goldens from PyTorch's oneDNN CPU ops, the reference
    # the reference's own tests compare with (test_quantized_ops.py:745-951) -------
    TD = {"uint8": torch.uint8, "int8": torch.int8, "float32": torch.float32}
    for c in cases.plain_linear_cases():
        n = c["w"].shape[1]
        b = None if c["bias"] is None else torch.from_numpy(c["bias"])
        y = torch.ops.onednn.qlinear_pointwise.default(
            torch.from_numpy(c["x"]), c["x_scale"], c["x_zp"], torch.from_numpy(c["w"]).to_mkldnn(),
            torch.from_numpy(c["w_scale"]), torch.zeros(n, dtype=torch.int), b, c["out_scale"], c["out_zp"],
            TD[c["out_dtype"]], c["post"], [], "")
        k = "plainlin/" + c["name"]
        g[k + "/x_crc"] = np.uint32(cases.crc(c["x"]))
        g[k + "/w_crc"] = np.uint32(cases.crc(c["w"]))
        g[k + "/y"] = y.numpy()
    for c in cases.plain_conv_cases():
        oc = c["w"].shape[0]
        ws = torch.from_numpy(c["w_scale"])
        wz = torch.zeros(oc, dtype=torch.int)
        b = None if c["bias"] is None else torch.from_numpy(c["bias"])
        st, pd = [c["stride"]] * 2, [c["pad"]] * 2
        x = torch.from_numpy(c["x"]).contiguous(memory_format=torch.channels_last)
        pw = torch.ops.onednn.qconv_prepack(torch.from_numpy(c["w"]), ws, c["x_scale"], c["x_zp"], st, pd, [1, 1],
                                            c["groups"], None)
        if c["accum"] is None:
            y = torch.ops.onednn.qconv2d_pointwise.default(
                x, c["x_scale"], c["x_zp"], pw, ws, wz, b, st, pd, [1, 1], c["groups"], c["out_scale"], c["out_zp"],
                TD[c["out_dtype"]], "relu" if c["relu"] else "none", [], "")
        else:
            acc = torch.from_numpy(c["accum"].copy()).contiguous(memory_format=torch.channels_last)  # overwritten
            y = torch.ops.onednn.qconv2d_pointwise.binary(
                x, c["x_scale"], c["x_zp"], pw, ws, wz, acc, b, st, pd, [1, 1], c["groups"], c["out_scale"],
                c["out_zp"], TD[c["out_dtype"]], c["accum_scale"], c["accum_zp"], "sum", 1.0,
                "relu" if c["relu"] else "none", [], "")
        k = "plainconv/" + c["name"]
        g[k + "/x_crc"] = np.uint32(cases.crc(c["x"]))
        g[k + "/w_crc"] = np.uint32(cases.crc(c["w"]))
        g[k + "/y"] = y.contiguous().numpy()   # NCHW order

    # ---- C1 ---------------------------------------------------------------
    c1 = cases.c1_case()
    x = torch.from_numpy(c1["x"])
    xq = torch.quantize_per_tensor_dynamic(x, torch.quint8, False)
    wq = torch.quantize_per_channel(torch.from_numpy(c1["w"]),
                                    torch.from_numpy(c1["w_scales"]),
                                    torch.zeros(1024, dtype=torch.int64), 0, torch.qint8)
    packed = torch.ops.quantized.linear_prepack(wq, torch.from_numpy(c1["bias"]))
    y = torch.ops.quantized.linear(xq, packed, c1["out_scale"], c1["out_zp"])
    g["c1/x_crc"] = np.uint32(cases.crc(c1["x"]))
    g["c1/w_crc"] = np.uint32(cases.crc(c1["w"]))
    g["c1/x_scale"] = np.float64(xq.q_scale())
    g["c1/x_zp"] = np.int64(xq.q_zero_point())
    g["c1/xq_crc"] = np.uint32(cases.crc(xq.int_repr().numpy()))
    g["c1/wq_crc"] = np.uint32(cases.crc(wq.int_repr().numpy()))
    g["c1/y"] = y.int_repr().numpy()
    g["c1/y_dq_crc"] = np.uint32(cases.crc(y.dequantize().numpy()))
    # engines agree on C1 (recorded, so a later engine drift is visible)
    for eng in ("x86", "onednn"):
        if eng in torch.backends.quantized.supported_engines:
            torch.backends.quantized.engine = eng
            p2 = torch.ops.quantized.linear_prepack(wq, torch.from_numpy(c1["bias"]))
            y2 = torch.ops.quantized.linear(xq, p2, c1["out_scale"], c1["out_zp"])
            meta[f"c1_mismatch_{eng}"] = int((y2.int_repr() != y.int_repr()).sum())
    torch.backends.quantized.engine = "fbgemm"

    # ---- fused conv variants: the float pipeline of the reference's tests ----
    # quantize( act( conv(dq(x), dq(w)) + bias + dq(accum) ) )
    # (test_quantized_conv.py:159-227, :236-360 of the reference)
    for c in cases.conv_fused_cases():
        qd = torch.qint8 if c["signed"] else torch.quint8
        xq = torch._make_per_tensor_quantized_tensor(
            torch.from_numpy(c["xq"]).permute(0, 3, 1, 2).contiguous(), c["x_scale"], c["x_zp"])
        wt = torch.from_numpy(c["wq"]).permute(0, 3, 1, 2).contiguous()
        if len(c["w_scales"]) == 1:
            w = torch._make_per_tensor_quantized_tensor(wt, float(c["w_scales"][0]), 0)
        else:
            w = torch._make_per_channel_quantized_tensor(
                wt, torch.from_numpy(c["w_scales"]), torch.zeros(wt.shape[0], dtype=torch.int64), 0)
        b = None if c["bias"] is None else torch.from_numpy(c["bias"])
        f = torch.nn.functional.conv2d(xq.dequantize().double(), w.dequantize().double(),
                                       None if b is None else b.double(), c["stride"], c["padding"],
                                       c["dilation"], c["groups"])
        if c["accq"] is not None:
            aq = torch._make_per_tensor_quantized_tensor(
                torch.from_numpy(c["accq"]).permute(0, 3, 1, 2).contiguous(), c["acc_scale"], c["acc_zp"])
            f = f + aq.dequantize().double()
        if c["activation"] == "relu":
            f = torch.relu(f)
        elif c["activation"] == "silu":
            f = torch.nn.functional.silu(f)
        y = torch.quantize_per_tensor(f.float(), c["out_scale"], c["out_zp"], qd)
        k = "convf/" + c["name"]
        g[k + "/xq_crc"] = np.uint32(cases.crc(c["xq"]))
        g[k + "/wq_crc"] = np.uint32(cases.crc(c["wq"]))
        g[k + "/y"] = y.int_repr().permute(0, 2, 3, 1).contiguous().numpy()

    # ---- quantized::add / add_relu, relu ------------------------------------
    for c in cases.qadd_cases():
        qa = torch._make_per_tensor_quantized_tensor(torch.from_numpy(c["qa"]), c["a_scale"], c["a_zp"])
        qb = torch._make_per_tensor_quantized_tensor(torch.from_numpy(c["qb"]), c["b_scale"], c["b_zp"])
        op = torch.ops.quantized.add_relu if c["relu"] else torch.ops.quantized.add
        y = op(qa, qb, c["out_scale"], c["out_zp"])
        k = "qadd/" + c["name"]
        g[k + "/qa_crc"] = np.uint32(cases.crc(c["qa"]))
        g[k + "/qb_crc"] = np.uint32(cases.crc(c["qb"]))
        g[k + "/y"] = y.int_repr().numpy()
        g[k + "/relu_a"] = torch.relu(qa).int_repr().numpy()

    # ---- quantized::cat, quantized max pooling -------------------------------
    for c in cases.qcat_cases():
        qs = [torch._make_per_tensor_quantized_tensor(torch.from_numpy(q), s_, z_)
              for q, s_, z_ in zip(c["qs"], c["scales"], c["zps"])]
        y = torch.ops.quantized.cat(qs, c["axis"], c["out_scale"], c["out_zp"])
        k = "qcat/" + c["name"]
        g[k + "/q0_crc"] = np.uint32(cases.crc(c["qs"][0]))
        g[k + "/y"] = y.int_repr().numpy()
    for c in cases.qmaxpool_cases():
        xq = torch._make_per_tensor_quantized_tensor(
            torch.from_numpy(c["x"]).permute(0, 3, 1, 2).contiguous(), 0.1, -7 if c["signed"] else 33)
        y = torch.nn.functional.max_pool2d(xq, c["kernel"], c["stride"], c["padding"], c["dilation"],
                                           c["ceil_mode"])
        k = "qmaxpool/" + c["name"]
        g[k + "/x_crc"] = np.uint32(cases.crc(c["x"]))
        g[k + "/y"] = y.int_repr().permute(0, 2, 3, 1).contiguous().numpy()

    for c in cases.qavgpool_cases():
        xq = torch._make_per_tensor_quantized_tensor(
            torch.from_numpy(c["x"]).permute(0, 3, 1, 2).contiguous(memory_format=torch.channels_last),
            0.05, c["zp"])
        y = torch.nn.functional.adaptive_avg_pool2d(xq, c["out_hw"])
        assert y.q_scale() == xq.q_scale() and y.q_zero_point() == c["zp"]
        k = "qavgpool/" + c["name"]
        g[k + "/x_crc"] = np.uint32(cases.crc(c["x"]))
        g[k + "/y"] = y.int_repr().permute(0, 2, 3, 1).contiguous().numpy()

    # ---- gelu / sigmoid of quantized tensors ------------------------------------
    for c in cases.qunary_cases():
        xq = torch._make_per_tensor_quantized_tensor(torch.from_numpy(c["x"]), c["scale"], c["zp"])
        for kind, fn in (("gelu", lambda t: torch.nn.functional.gelu(t)),
                         ("gelu_tanh", lambda t: torch.nn.functional.gelu(t, approximate="tanh")),
                         ("sigmoid", torch.sigmoid)):
            y = fn(xq)
            k = "qunary/" + c["name"] + "/" + kind
            g[k + "/y"] = y.int_repr().numpy()
            g[k + "/qparams"] = np.array([y.q_scale(), y.q_zero_point()], dtype=np.float64)
        g["qunary/" + c["name"] + "/x_crc"] = np.uint32(cases.crc(c["x"]))

    # ---- quantized::conv2d -------------------------------------------------
    for c in cases.conv_cases():
        x_nchw = torch.from_numpy(c["xq"]).permute(0, 3, 1, 2)  # channels-last view
        xq = torch._make_per_tensor_quantized_tensor(x_nchw, c["x_scale"], c["x_zp"])
        w_oihw = torch.from_numpy(c["wq"]).permute(0, 3, 1, 2).contiguous()
        w = make_w(w_oihw.numpy(), c["w_scales"], w_oihw.shape[0])
        b = None if c["bias"] is None else torch.from_numpy(c["bias"])
        packed = torch.ops.quantized.conv2d_prepack(w, b, list(c["stride"]),
                                                    list(c["padding"]),
                                                    list(c["dilation"]), c["groups"])
        op = torch.ops.quantized.conv2d_relu if c["relu"] else torch.ops.quantized.conv2d
        y = op(xq, packed, c["out_scale"], c["out_zp"])
        k = "conv/" + c["name"]
        g[k + "/xq_crc"] = np.uint32(cases.crc(c["xq"]))
        g[k + "/wq_crc"] = np.uint32(cases.crc(c["wq"]))
        g[k + "/out_scale"] = np.float64(c["out_scale"])
        # NHWC bytes
        g[k + "/y"] = y.int_repr().permute(0, 2, 3, 1).contiguous().numpy()

    g["meta"] = np.array(repr(meta))
    path = os.path.join(HERE, "golden.npz")
    np.savez_compressed(path, **g)
    print("wrote", path, os.path.getsize(path), "bytes;", len(g), "arrays;", meta)


if __name__ == "__main__":
    main()
