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
Activations live in the channel-blocked c16 layout between layers; the input is fp32 NCHW, the output fp32.

Host-side preparation (numpy) happens once per model; the per-batch work is one launch plan.
"""
import os

import numpy as np

from . import hipabi as H
from .hipabi import Buf, CONV_BIAS, CONV_RELU, CONV_RESIDUAL
from .resnet18 import _Arena

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


class QuantizedResNet18:
    """Device-resident quantised model + launch plan.  run(x_f32, out_f32) enqueues one forward pass."""

    def __init__(self, model, batch, hw=224, device="cuda", shares=None):
        """shares: parts of the batch that run side by side as chains of the one plan (each the whole network on
        batch / shares images, on its own stream between the fork at the start of a run and the join at its end, so
        that the launches of one fill the compute units the other's leave idle).  None: two from 128 images on, else
        one (KXC_HIP_BATCH_LANES overrides) -- measured: batch 64 0.311 ms in one share, 0.308-0.317 in two, 0.413 in
        four (these launches are 7-15 us each; a fork and a join cost as much as the tails they would fill); batch
        128 0.461 ms in one share, 0.430 in two (298 against 277 k img/s).  The fp32 network gains 9 % at batch 64."""
        import torch
        self.batch, self.hw = batch, hw
        if shares is None:
            shares = int(os.environ.get("KXC_HIP_BATCH_LANES", "0")) or (2 if batch >= 128 else 1)
        if shares < 1 or shares > 8 or batch % shares != 0 or (batch // shares) % 4 != 0:
            shares = 1           # (a share of the fp32 logits and of the input must start on a 16-byte boundary)
        self.shares = shares
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
        self.consts = []          # packed args after the input: per layer w_packed, bias, mult; fc w, bias, mult
        # the 7x7/2 first layer runs on the 4-channel input layout when the width allows it
        self.first_c4 = hw % 4 == 0 and model["layers"][0]["k"] == 7 and model["layers"][0]["cin"] <= 4
        for i, L in enumerate(model["layers"]):
            pack = H.qconv2d_c4_pack_weights if (i == 0 and self.first_c4) else H.qconv2d_c16_pack_weights
            self.consts += [pack(dev(L["wq"])), dev(L["bias_q"]), dev(L["mult"])]
        self.consts += [dev(model["fc"]["wq"]), dev(model["fc"]["bias_q"]), dev(model["fc"]["mult"])]
        nargs = 1 + len(self.consts) + 1
        plan = H.Plan(nargs)
        arena = _Arena()
        arg = lambda i: Buf.arg(i)
        OUT = nargs - 1

        def new_act(n, c, h, w):
            nbytes = n * ((c + 15) // 16) * h * w * 16
            off, size = arena.alloc(nbytes)
            return {"buf": Buf.ws(off), "off": off, "size": size, "shape": (n, c, h, w)}

        def free_act(a):
            arena.release(a["off"], a["size"])

        by_name = {L["name"]: (i, L) for i, L in enumerate(model["layers"])}

        def conv(x, name, residual=None):
            i, L = by_name[name]
            n, c, h, w = x["shape"]
            flags = CONV_BIAS | (CONV_RELU if L["relu"] else 0) | (CONV_RESIDUAL if residual is not None else 0)
            d = H.qconv_desc(n, c, h, w, L["cout"], L["k"], L["k"], L["stride"], L["pad"], flags,
                             L["res_mult"] if residual is not None else 0.0)
            oh = (h + 2 * L["pad"] - L["k"]) // L["stride"] + 1
            ow = (w + 2 * L["pad"] - L["k"]) // L["stride"] + 1
            y = new_act(n, L["cout"], oh, ow)
            plan.add_qconv2d_c16(d, x["buf"], arg(1 + 3 * i), arg(2 + 3 * i), arg(3 + 3 * i),
                                 residual["buf"] if residual is not None else Buf.none(), y["buf"])
            return y

        def conv_pair(x, name, down_name):
            # a block's first 3x3/2 convolution and its 1x1/2 downsample in one launch (two outputs); the
            # downsample's weights are re-packed in the chunking of the 3x3 kernel
            i, L = by_name[name]
            j, D = by_name[down_name]
            n, c, h, w = x["shape"]
            d = H.qconv_desc(n, c, h, w, L["cout"], L["k"], L["k"], L["stride"], L["pad"], CONV_BIAS | CONV_RELU, 0.0)
            oh = (h + 2 * L["pad"] - L["k"]) // L["stride"] + 1
            ow = (w + 2 * L["pad"] - L["k"]) // L["stride"] + 1
            self.consts[3 * j] = H.qconv2d_c16_pair_pack_weights(dev(D["wq"]), L["k"])
            y = new_act(n, L["cout"], oh, ow)
            y2 = new_act(n, L["cout"], oh, ow)
            plan.add_qconv2d_c16_pair(d, x["buf"], arg(1 + 3 * i), arg(2 + 3 * i), arg(3 + 3 * i), Buf.none(), y["buf"],
                                      arg(1 + 3 * j), arg(2 + 3 * j), arg(3 + 3 * j), y2["buf"])
            return y, y2

        def can_pair(x, name, down_name):
            if os.environ.get("KXC_HIP_QPAIR", "1") == "0":
                return False
            _, L = by_name[name]
            _, D = by_name[down_name]
            n, c, h, w = x["shape"]
            return (D["k"] == 1 and D["pad"] == 0 and D["stride"] == L["stride"] and D["cout"] == L["cout"] and not D["relu"]
                    and H.qconv2d_c16_pair_supported(n, c, h, w, L["cout"], L["k"], L["stride"], L["pad"]))

        whole_batch = batch
        plan.set_select_lanes(shares)
        for share in range(shares):
            first_node = plan.num_nodes()
            self._emit_share(plan, arena, model, by_name, conv, conv_pair, can_pair, new_act, free_act, arg, OUT, share,
                             whole_batch // shares, hw)
            # a share's activations stay out of the regions the other shares use at the same time
            arena.free = []
            for node in range(first_node, plan.num_nodes()):
                if share > 0:
                    plan.set_chain(node, share)
        if shares > 1:
            plan.interleave_chains()          # a run feeds every share's stream at the same pace
        plan.finalize(arena.top)
        self.plan = plan
        self.workspace_bytes = arena.top
        self.launches = plan.symbols()

    def _emit_share(self, plan, arena, model, by_name, conv, conv_pair, can_pair, new_act, free_act, arg, OUT, share, batch, hw):
        in_arg = Buf.arg_offset(0, share * batch * 3 * hw * hw * 4) if self.shares > 1 else arg(0)
        out_arg = Buf.arg_offset(OUT, share * batch * 1000 * 4) if self.shares > 1 else arg(OUT)
        if self.first_c4:
            L0 = model["layers"][0]
            off, size = arena.alloc(batch * hw * hw * 4)
            xq = {"buf": Buf.ws(off), "off": off, "size": size}
            plan.add_quantize_c4(batch, 3, hw * hw, model["input_scale"], in_arg, xq["buf"])
            d = H.qconv_desc(batch, 3, hw, hw, L0["cout"], 7, 7, 2, 3, CONV_BIAS | CONV_RELU)
            oh = (hw + 6 - 7) // 2 + 1
            y = new_act(batch, L0["cout"], oh, oh)
            plan.add_qconv2d_c4(d, xq["buf"], arg(1), arg(2), arg(3), y["buf"])
        else:
            xq = new_act(batch, 3, hw, hw)
            plan.add_quantize_c16(batch, 3, hw * hw, model["input_scale"], in_arg, xq["buf"])
            y = conv(xq, "conv1")
        free_act(xq)
        n, c, h, w = y["shape"]
        pd = H.pool_desc((n, c, h, w), 3, 2, 1)
        _, _, ph, pw = H.pool_out_shape(pd)
        cur = new_act(n, c, ph, pw)
        plan.add_maxpool2d_c16_i8(pd, y["buf"], cur["buf"])
        free_act(y)
        for stage in range(4):
            for blk in range(2):
                first = blk == 0 and stage > 0
                name = "l%d.%d" % (stage + 1, blk)
                if first and can_pair(cur, name + ".conv1", name + ".down"):
                    a, idn = conv_pair(cur, name + ".conv1", name + ".down")
                else:
                    a = conv(cur, name + ".conv1")
                    idn = conv(cur, name + ".down") if first else cur
                out = conv(a, name + ".conv2", residual=idn)
                free_act(a)
                if first:
                    free_act(idn)
                free_act(cur)
                cur = out
        n, c, h, w = cur["shape"]
        s_last = model["scale"][model["last"]]
        gap_mult = float(np.float32(s_last) / (np.float32(h * w) * np.float32(model["gap_scale_out"])))
        self.gap_mult = gap_mult
        g = new_act(n, c, 1, 1)
        plan.add_global_avg_pool2d_c16_i8(n, c, h, w, gap_mult, cur["buf"], g["buf"])
        free_act(cur)
        nl = len(model["layers"])
        plan.add_qdense(n, 1000, c, g["buf"], arg(1 + 3 * nl), arg(2 + 3 * nl), arg(3 + 3 * nl), out_arg)

    def packed(self, x, out):
        return self.plan.packed([x] + self.consts + [out])

    def run(self, x, out, stream=None):
        self.plan.run([x] + self.consts + [out], stream)


def int_ops_per_image(hw=224):
    from .resnet18 import flops_per_image
    return flops_per_image(hw)
