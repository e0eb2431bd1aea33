"""Launch plan for the ResNet-18 graph of the reference's test/resnet18_ir_dump.cpp:191-452.

Packed arguments follow the lowered function's parameter order (src/relay/backend/lower.cc:530-565):
[input, const_0 .. const_41 (depth-first argument order), output].  The 49 Relay calls collapse to
23 launches: conv+bias+relu (9), conv+bias (3 downsamples), conv+bias+add+relu (8), max pool,
global average pool, gemm; nn_flatten of [N,512,1,1] is an alias and launches nothing.
Intermediates are slots of one workspace, reused as soon as their last reader has been enqueued.
"""
from .hipabi import (Plan, Buf, conv_desc, conv_out_shape, pool_desc, pool_out_shape,
                     CONV_BIAS, CONV_RESIDUAL, CONV_RELU)

_ALIGN = 256


class _Arena:
    """First-fit reuse of freed blocks; all offsets are multiples of 256 bytes."""

    def __init__(self):
        self.free = []      # (offset, size)
        self.top = 0

    def alloc(self, nbytes):
        size = (nbytes + _ALIGN - 1) // _ALIGN * _ALIGN
        for i, (off, sz) in enumerate(self.free):
            if sz >= size:
                if sz == size:
                    self.free.pop(i)
                else:
                    self.free[i] = (off + size, sz - size)
                return off, size
        off = self.top
        self.top += size
        return off, size

    def release(self, off, size):
        self.free.append((off, size))
        self.free.sort()
        merged = []
        for o, s in self.free:
            if merged and merged[-1][0] + merged[-1][1] == o:
                merged[-1] = (merged[-1][0], merged[-1][1] + s)
            else:
                merged.append((o, s))
        self.free = merged


def build_plan(batch, hw=224, fuse=True):
    """Returns (plan, info).  fuse=False keeps every Relay call a separate launch (conv, bias add is
    still inside the conv kernel; relu / add separate) -- used by tests to check the fusion."""
    plan = Plan(44)
    arena = _Arena()
    INPUT, OUTPUT = 0, 43
    const = lambda k: Buf.arg(1 + k)
    info = {"launches": [], "shapes": {}}

    def new_act(shape):
        n = 1
        for d in shape:
            n *= d
        off, size = arena.alloc(4 * n)
        return {"buf": Buf.ws(off), "off": off, "size": size, "shape": tuple(shape)}

    def free_act(a):
        if a is not None and "off" in a:
            arena.release(a["off"], a["size"])

    def conv(x, k, cin, cout, ksz, stride, pad, relu, residual=None):
        flags = CONV_BIAS | (CONV_RELU if relu else 0) | (CONV_RESIDUAL if residual is not None else 0)
        d = conv_desc(x["shape"], (cout, cin, ksz, ksz), stride, pad, 1, flags)
        y = new_act(conv_out_shape(d))
        plan.add_conv2d(d, x["buf"], const(k), const(k + 1), residual["buf"] if residual is not None else Buf.none(),
                        y["buf"])
        return y

    x = {"buf": Buf.arg(INPUT), "shape": (batch, 3, hw, hw)}
    k = 0
    if fuse:
        y = conv(x, k, 3, 64, 7, 2, 3, True)
    else:
        t = conv(x, k, 3, 64, 7, 2, 3, False)
        y = new_act(t["shape"])
        plan.add_relu(_numel(t["shape"]), t["buf"], y["buf"])
        free_act(t)
    k += 2
    pd = pool_desc(y["shape"], 3, 2, 1)
    mp = new_act(pool_out_shape(pd))
    plan.add_pool2d(pd, y["buf"], mp["buf"])
    free_act(y)
    info["shapes"]["maxpool"] = mp["shape"]

    cur, cin = mp, 64
    for stage, ch in enumerate((64, 128, 256, 512)):
        for blk in range(2):
            first = blk == 0 and stage > 0
            stride = 2 if first else 1
            if fuse:
                a = conv(cur, k, cin, ch, 3, stride, 1, True)
                idn = conv(cur, k + 4, cin, ch, 1, stride, 0, False) if first else cur
                out = conv(a, k + 2, ch, ch, 3, 1, 1, True, residual=idn)
                free_act(a)
            else:
                t = conv(cur, k, cin, ch, 3, stride, 1, False)
                a = new_act(t["shape"])
                plan.add_relu(_numel(t["shape"]), t["buf"], a["buf"])
                free_act(t)
                b = conv(a, k + 2, ch, ch, 3, 1, 1, False)
                free_act(a)
                idn = conv(cur, k + 4, cin, ch, 1, stride, 0, False) if first else cur
                s = new_act(b["shape"])
                plan.add_binary(0, b["shape"], idn["shape"], False, b["buf"], idn["buf"], s["buf"])
                free_act(b)
                out = new_act(s["shape"])
                plan.add_relu(_numel(s["shape"]), s["buf"], out["buf"])
                free_act(s)
            if first:
                free_act(idn)
            free_act(cur)
            cur, cin = out, ch
            k += 6 if first else 4
    n, c, h, w = cur["shape"]
    gap = new_act((n, c, 1, 1))
    plan.add_global_avg_pool2d(n, c, h, w, cur["buf"], gap["buf"])
    free_act(cur)
    # nn_flatten: [N,512,1,1] -> [N,512] is the same memory
    plan.add_gemm(n, 1000, c, 1.0, 1.0, 1, 1000, gap["buf"], const(k), const(k + 1), Buf.arg(OUTPUT))
    plan.finalize(arena.top)
    info["workspace_bytes"] = arena.top
    info["launches"] = plan.symbols()
    return plan, info


def _numel(shape):
    n = 1
    for d in shape:
        n *= d
    return n


# Multiply-accumulate count of one image (convolutions and the FC layer), for FLOP accounting.
def flops_per_image(hw=224):
    total = 0
    h = (hw + 6 - 7) // 2 + 1
    total += 2 * 64 * h * h * 3 * 49
    h = (h + 2 - 3) // 2 + 1
    cin = 64
    for stage, ch in enumerate((64, 128, 256, 512)):
        for blk in range(2):
            first = blk == 0 and stage > 0
            if first:
                h = (h + 2 - 3) // 2 + 1
                total += 2 * ch * h * h * cin * 1           # 1x1 downsample
            total += 2 * ch * h * h * (cin if blk == 0 else ch) * 9
            total += 2 * ch * h * h * ch * 9
        cin = ch
    total += 2 * 1000 * 512
    return total
