"""Quantised ResNet-18 (int8 x int8 -> int32, per-output-channel requantisation) on the int8 matrix cores.

Topology = the fp32 graph of the reference's test/resnet18_ir_dump.cpp:191-452 with every convolution and
the FC layer replaced by its quantised form; the reference has no int8 operator, so the definition is
this build's (see csrc/qconv_c16_i8.hip):
  * activations: per-tensor symmetric scale s = max|x| / 127 taken from an fp32 calibration pass,
  * weights: per-output-channel symmetric scale s_w[o] = max|w[o]| / 127,
  * conv: acc + rint(b / (s_in*s_w[o])), requantised with mult[o] = s_in*s_w[o]/s_out, ReLU fused,
    the residual operand added as (float)res * (s_res/s_out) before rounding,
  * max pool keeps the scale; global average pool requantises with s_in/(H*W*s_out),
  * FC: fp32 logits = (acc + bias_q) * (s_in*s_w[j]).
This module only calibrates and quantises the constants (numpy, once per model).  The network itself is the Relay
graph of host/src/models.cc (BuildQResNet18) compiled by Compiler::Compile -- hostapi.CompiledQResNet18 -- whose
operator hooks choose the channel-blocked activation layout of the int8 matrix cores and pack the weights.
"""
import numpy as np

from . import hipabi as H

# (name, cin, cout, k, stride, pad) in constant order (weights, bias pairs)
def layer_table():
    layers = [("conv1", 3, 64, 7, 2, 3)]
    cin = 64
    for stage, ch in enumerate((64, 128, 256, 512)):
        for blk in range(2):
            first = blk == 0 and stage > 0
            s = 2 if first else 1
            layers.append(("l%d.%d.conv1" % (stage + 1, blk), cin, ch, 3, s, 1))
            layers.append(("l%d.%d.conv2" % (stage + 1, blk), ch, ch, 3, 1, 1))
            if first:
                layers.append(("l%d.%d.down" % (stage + 1, blk), cin, ch, 1, s, 0))
            cin = ch
    return layers


def quantize_weights(w):
    """Per-output-channel symmetric int8: returns (q int8, scale float32[O])."""
    o = w.shape[0]
    s = (np.abs(w).reshape(o, -1).max(axis=1) / np.float32(127.0)).astype(np.float32)
    s[s == 0] = np.float32(1.0)
    q = np.clip(np.rint(w / s.reshape((o,) + (1,) * (w.ndim - 1))), -127, 127).astype(np.int8)
    return q, s


def calibrate(x, consts):
    """fp32 pass on the GPU (hand-written kernels, one call per layer) recording max|activation| of every
    tensor that gets a scale.  x, consts: GPU tensors.  Returns {name: max_abs}."""
    amax = {"input": H.absmax(x)}
    y = H.conv2d(x, consts[0], consts[1], None, 2, 3, 1, True)
    amax["conv1"] = H.absmax(y)
    cur = H.pool2d(y, 3, 2, 1)
    k = 2
    for stage in range(4):
        for blk in range(2):
            first = blk == 0 and stage > 0
            s = 2 if first else 1
            name = "l%d.%d" % (stage + 1, blk)
            a = H.conv2d(cur, consts[k], consts[k + 1], None, s, 1, 1, True)
            amax[name + ".conv1"] = H.absmax(a)
            idn = cur
            if first:
                idn = H.conv2d(cur, consts[k + 4], consts[k + 5], None, s, 0, 1, False)
                amax[name + ".down"] = H.absmax(idn)
            cur = H.conv2d(a, consts[k + 2], consts[k + 3], idn, 1, 1, 1, True)
            amax[name + ".conv2"] = H.absmax(cur)
            k += 6 if first else 4
    g = H.global_avg_pool2d(cur)
    amax["gap"] = H.absmax(g)
    return amax


def prepare(consts_np, amax):
    """consts_np: the 42 fp32 constants (numpy, lowering order); amax from calibrate().
    Returns the quantised model: list of per-layer dicts + fc dict + scales (all numpy)."""
    f32 = np.float32
    scale = {k: (f32(v) / f32(127.0) if v > 0 else f32(1.0)) for k, v in amax.items()}
    layers = []
    k = 0
    table = layer_table()
    # scale of each layer's input / residual
    s_in = {}
    s_res = {}
    cur = "conv1"   # max pool keeps conv1's scale
    s_in["conv1"] = scale["input"]
    for stage in range(4):
        for blk in range(2):
            first = blk == 0 and stage > 0
            name = "l%d.%d" % (stage + 1, blk)
            s_in[name + ".conv1"] = scale[cur]
            s_in[name + ".conv2"] = scale[name + ".conv1"]
            if first:
                s_in[name + ".down"] = scale[cur]
                s_res[name + ".conv2"] = scale[name + ".down"]
            else:
                s_res[name + ".conv2"] = scale[cur]
            cur = name + ".conv2"
    # constants come in the order conv1, then per block conv1, conv2, [down]
    for (name, cin, cout, ksz, stride, pad) in table:
        w, b = consts_np[k], consts_np[k + 1]
        k += 2
        wq, sw = quantize_weights(w)
        si, so = s_in[name], scale[name]
        acc_scale = (si * sw).astype(f32)                      # one rounded fp32 multiply
        bias_q = np.rint(b.astype(np.float64) / acc_scale.astype(np.float64)).astype(np.int32)
        mult = (acc_scale / so).astype(f32)
        layers.append({"name": name, "cin": cin, "cout": cout, "k": ksz, "stride": stride, "pad": pad,
                       "wq": wq, "bias_q": bias_q, "mult": mult,
                       "res_mult": float(f32(s_res[name]) / so) if name in s_res else 0.0,
                       "relu": not name.endswith(".down")})
    fw, fb = consts_np[k], consts_np[k + 1]
    fq, fs = quantize_weights(fw)
    acc_scale = (scale["gap"] * fs).astype(f32)
    fc = {"wq": fq, "bias_q": np.rint(fb.astype(np.float64) / acc_scale.astype(np.float64)).astype(np.int32),
          "mult": acc_scale}
    return {"layers": layers, "fc": fc, "scale": scale, "input_scale": float(scale["input"]),
            "gap_scale_out": float(scale["gap"]), "last": cur}


def int_ops_per_image(hw=224):
    from .resnet18 import flops_per_image
    return flops_per_image(hw)
