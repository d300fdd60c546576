"""The benchmark workloads as lists of ConvBias descriptors (shapes only; no model code).

config 2: the 53 ConvBias layers of ResNet-50 v1.5 at batch 64 (stem in NCHW4 with the input
          padded to 4 channels, everything after the max-pool in NCHW32);
config 1: the 1x1 NCHW32 sweep at N=64;
config 3: MobileNetV2 (t=6, width 1.0) inverted-residual blocks at batch 64, NCHW4;
config 4: large NCHW32 ConvBias + H_SWISH cases at batch 128 with relayouts on both sides.
Work accounting follows the reference's own TOPS print (dnn/test/cuda/conv_test_utils.cpp:193,405):
ops = 2*N*OC*OH*OW*(IC/group)*FH*FW; bytes = src + filter + 4*OC + (z ? dst : 0) + dst.
"""
from . import _abi


class Layer:
    def __init__(self, name, fmt, n, ic, ih, iw, oc, f, stride=1, pad=0, group=1, nonline="RELU", z=None,
                 src=None):
        self.name, self.fmt = name, fmt
        self.n, self.ic, self.ih, self.iw, self.oc, self.f = n, ic, ih, iw, oc, f
        self.stride, self.pad, self.group, self.nonline = stride, pad, group, nonline
        self.z = z        # name of the layer whose output is added, or "input:<name>"
        self.src = src    # name of the producing layer (None = the previous layer)
        self.oh = _abi.out_size(ih, f, 1, stride, pad)
        self.ow = _abi.out_size(iw, f, 1, stride, pad)

    @property
    def ops(self):
        return 2 * self.n * self.oc * self.oh * self.ow * (self.ic // self.group) * self.f * self.f

    @property
    def bytes(self):
        src = self.n * self.ic * self.ih * self.iw
        flt = self.oc * (self.ic // self.group) * self.f * self.f
        dst = self.n * self.oc * self.oh * self.ow
        return src + flt + 4 * self.oc + (dst if self.z else 0) + dst

    def desc(self, s_bias, s_z, s_dst):
        return _abi.make_conv_desc(self.fmt, self.n, self.ic, self.ih, self.iw, self.oc, self.f, group=self.group,
                                   pad=self.pad, stride=self.stride, nonline=self.nonline, has_z=self.z is not None,
                                   scale_bias=s_bias, scale_z=s_z, scale_dst=s_dst)


def resnet50(batch=64):
    """53 layers.  The max-pool between the stem and stage 1 is not a ConvBias: stage 1 reads a
    separate seeded tensor 'pool' of 64 channels at 56x56."""
    L = [Layer("stem", "NCHW4", batch, 4, 224, 224, 64, 7, stride=2, pad=3)]
    cin, h, prev = 64, 56, "input:pool"
    for si, (mid, out, blocks, stride) in enumerate([(64, 256, 3, 1), (128, 512, 4, 2), (256, 1024, 6, 2),
                                                      (512, 2048, 3, 2)]):
        for b in range(blocks):
            s = stride if b == 0 else 1
            p = "s%db%d" % (si + 1, b)
            L.append(Layer(p + "c1", "NCHW32", batch, cin, h, h, mid, 1, src=prev))
            L.append(Layer(p + "c2", "NCHW32", batch, mid, h, h, mid, 3, stride=s, pad=1))
            ho = h // s
            if b == 0:
                L.append(Layer(p + "ds", "NCHW32", batch, cin, h, h, out, 1, stride=s, nonline="IDENTITY", src=prev))
                L.append(Layer(p + "c3", "NCHW32", batch, mid, ho, ho, out, 1, z=p + "ds", src=p + "c2"))
            else:
                L.append(Layer(p + "c3", "NCHW32", batch, mid, ho, ho, out, 1, z=prev, src=p + "c2"))
            prev, cin, h = p + "c3", out, ho
    assert len(L) == 53
    return L


def pointwise_sweep(batch=64):
    shapes = [(256, 64, 56, False), (64, 256, 56, True), (512, 128, 28, False), (1024, 256, 14, False),
              (2048, 512, 7, False)]
    out = []
    for ic, oc, hw, z in shapes:
        for nl in ("IDENTITY", "RELU"):
            out.append(Layer("pw%d_%d_%d_%s" % (ic, oc, hw, nl), "NCHW32", batch, ic, hw, hw, oc, 1, nonline=nl,
                             z="input:z" if z else None))
    return out


def mobilenet_v2(batch=64):
    """Inverted-residual blocks (expand 1x1, depthwise 3x3, project 1x1) from 16 channels at 112x112."""
    L = []
    cin, h = 16, 112
    for c, n, s in [(24, 2, 2), (32, 3, 2), (64, 4, 2), (96, 3, 1), (160, 3, 2), (320, 1, 1)]:
        for i in range(n):
            stride = s if i == 0 else 1
            hid = cin * 6
            p = "c%d_%d" % (c, i)
            L.append(Layer(p + "_expand", "NCHW4", batch, cin, h, h, hid, 1))
            L.append(Layer(p + "_dw", "NCHW4", batch, hid, h, h, hid, 3, stride=stride, pad=1, group=hid))
            ho = h // stride
            res = stride == 1 and cin == c
            L.append(Layer(p + "_project", "NCHW4", batch, hid, ho, ho, c, 1, nonline="IDENTITY",
                           z="input:block" if res else None))
            cin, h = c, ho
    return L


def large_hswish(batch=128):
    return [
        Layer("l3x3s1_256", "NCHW32", batch, 256, 64, 64, 256, 3, pad=1, nonline="H_SWISH", z="input:z"),
        Layer("l3x3s2_512_1024", "NCHW32", batch, 512, 32, 32, 1024, 3, stride=2, pad=1, nonline="H_SWISH", z="input:z"),
        Layer("l5x5s1_128", "NCHW32", batch, 128, 80, 80, 128, 5, pad=2, nonline="H_SWISH", z="input:z"),
    ]


def config0():
    return Layer("cfg0", "NCHW4", 16, 64, 56, 56, 64, 3, pad=1, nonline="RELU")


def build_stack(layers, seed):
    """Allocates every tensor of a layer list on the GPU (seeded random weights and inputs, per-tensor scales drawn
    log-uniform in [1e-3, 5e-2], bias scale = source scale x filter scale, residuals and sources wired to the real
    producer outputs) and returns one dict per layer: layer, desc, src, flt, bias, z, dst."""
    import numpy as np
    import torch

    rng = np.random.RandomState(seed)

    def scale():
        return float(np.float32(np.exp(rng.uniform(np.log(1e-3), np.log(5e-2)))))

    def rand_i8(shape, lo=-128, hi=127):
        return torch.randint(lo, hi + 1, shape, dtype=torch.int8, device="cuda")

    outs, out_scale, inputs = {}, {}, {}
    plan = []
    prev = None
    for i, L in enumerate(layers):
        d0 = L.desc(1.0, 1.0, 1.0)
        src_s, flt_s, bias_s, dst_s = _abi.conv_shapes(d0)
        # source tensor
        sname = L.src if L.src is not None else prev
        if sname is None or sname.startswith("input:") or sname not in outs or tuple(outs[sname].shape) != tuple(src_s):
            key = "in:%s:%s" % (sname, src_s)
            if key not in inputs:
                inputs[key] = (rand_i8(src_s), scale())
            src, s_src = inputs[key]
        else:
            src, s_src = outs[sname], out_scale[sname]
        s_flt = scale()
        s_bias = float(np.float32(s_src) * np.float32(s_flt))
        s_dst = scale()
        flt = rand_i8(flt_s, -127, 127)
        bias = torch.randint(-1000, 1001, bias_s, dtype=torch.int32, device="cuda")
        z, s_z = None, 1.0
        if L.z is not None:
            if L.z in outs and tuple(outs[L.z].shape) == tuple(dst_s):
                z, s_z = outs[L.z], out_scale[L.z]
            else:
                key = "z:%s:%s" % (L.z, dst_s)
                if key not in inputs:
                    inputs[key] = (rand_i8(dst_s), scale())
                z, s_z = inputs[key]
        dst = torch.empty(dst_s, dtype=torch.int8, device="cuda")
        desc = L.desc(s_bias, s_z, s_dst)
        outs[L.name], out_scale[L.name] = dst, s_dst
        prev = L.name
        plan.append(dict(layer=L, desc=desc, src=src, flt=flt, bias=bias, z=z, dst=dst, s_src=s_src, s_z=s_z))
    return plan


def first_fit_offsets(tensors, granule=4096):
    """Offsets for tensors given as (bytes, index of the writing step, index of the last reading step[, index of a
    tensor whose range this one may take over]), in writing order: each goes to the lowest granule-aligned offset where
    it overlaps no tensor that is live at its writing step (written earlier and read at that step or later).  A tensor
    with a take-over candidate -- an earlier tensor of the same size whose last reading step is this tensor's writing
    step -- gets that tensor's range instead.  Returns (offsets, arena bytes)."""
    live, offsets, top = [], [], 0
    for k, spec in enumerate(tensors):
        size, i, last_read = spec[:3]
        over = spec[3] if len(spec) > 3 else None
        live = [r for r in live if r[2] >= i]
        size = (size + granule - 1) // granule * granule
        off = None
        if over is not None:
            for r in live:
                if r[3] == over and r[1] == size and r[2] == i:
                    off = r[0]
                    live.remove(r)
                    break
        if off is None:
            off = 0
            for o, sz, _, _ in sorted(live):
                if off + size <= o:
                    break
                off = max(off, o + sz)
        live.append((off, size, max(last_read, i), k))
        offsets.append(off)
        top = max(top, off + size)
    return offsets, top


def plan_memory(plan, residual_in_place=False):
    """Static activation-memory plan for a layer list of build_stack, as a graph runtime lays out the variables of a
    computing sequence before it runs (the reference: StaticMemAlloc, src/core/impl/graph/var_node_mem_mgr/
    static_mem_alloc.h:18-40, intervals = first write to last read): every layer output becomes a range of ONE arena
    that no LIVE tensor occupies -- live = written and still to be read, as a source or a residual, by this layer or a
    later one -- at the lowest address where it fits (address-ordered first fit, 4 KiB granules), instead of a buffer
    of its own.  Graph inputs (seeded tensors) keep theirs.  A layer never writes memory it reads as a source;
    `residual_in_place`: a layer whose residual is read for the last time by that very layer writes its output over it
    (every kernel reads the residual of an output element in the thread that writes the element, before the write).
    Rewires src / z / dst of the plan in place; returns the bytes of activation memory before and after."""
    import torch

    last, producer = {}, {}
    for i, p in enumerate(plan):
        for t in (p["src"], p["z"]):
            if t is not None:
                last[t.data_ptr()] = i
        producer[p["dst"].data_ptr()] = i
    specs = []
    for i, p in enumerate(plan):
        over = None
        z = p["z"]
        if residual_in_place and z is not None and z.data_ptr() in producer and last[z.data_ptr()] == i and \
                z.numel() == p["dst"].numel() and z.data_ptr() != p["src"].data_ptr():
            over = producer[z.data_ptr()]
        # an output nobody reads is dead after its own layer
        specs.append((p["dst"].numel(), i, last.get(p["dst"].data_ptr(), i), over))
    offsets, top = first_fit_offsets(specs)
    before = sum(p["dst"].numel() for p in plan)
    arena = torch.empty(top, dtype=plan[0]["dst"].dtype, device=plan[0]["dst"].device)
    remap = {}    # data_ptr of the original output -> its range of the arena
    for p, off in zip(plan, offsets):
        for k in ("src", "z"):
            t = p[k]
            if t is not None and t.data_ptr() in remap:
                p[k] = remap[t.data_ptr()].view(t.shape)
        old = p["dst"]
        remap[old.data_ptr()] = arena[off:off + old.numel()]
        p["dst"] = remap[old.data_ptr()].view(old.shape)
    return dict(one_buffer_per_layer=before, planned=top)


def snapshot_run(plan, calls, images):
    """Runs the launches of a plan once, in order, and copies the first `images` images of every layer's source and
    residual to the host right before its launch and of its output right after: with planned activation memory a
    buffer holds a tensor only until its last reader has run, and an output may replace the residual it was made from."""
    import torch

    snaps = []
    for p, c in zip(plan, calls):
        torch.cuda.synchronize()
        h_in = [None if t is None else t[:images].cpu().numpy() for t in (p["src"], p["z"])]
        c()
        torch.cuda.synchronize()
        snaps.append((h_in[0], h_in[1], p["dst"][:images].cpu().numpy()))
    return snaps


def run_calibrated(plan, seed, weight_preprocess=True):
    """Runs a plan of build_stack layer by layer with scales and biases re-drawn so that most outputs are LIVE values,
    strictly inside the int8 range, instead of the clamped bytes that per-tensor scales drawn at random give after a
    long reduction (there the typical |acc * s_bias / s_dst| is in the hundreds): a test on such a plan sees every
    accumulator.  In execution order, from the statistics of the layer's real input: the accumulator's spread is
    sigma = sqrt(K * mean(src^2) * mean(flt^2)); the bias is drawn in [1.3, 1.9] sigma (so that an activation keeps most
    values); the dst scale is drawn log-uniform in [1e-3, 5e-2] (with a residual: 2 to 3 times the residual's
    scale); the filter scale is what puts sigma at 25 output steps.  Same tensors, shapes and algorithm choice as the
    uncalibrated plan.  Returns the fraction of live outputs per layer."""
    import numpy as np
    import torch

    from . import ops
    rng = np.random.RandomState(seed)
    scale_of = {}
    live = []
    for p in plan:
        L = p["layer"]
        s_src = scale_of.get(id(p["src"]), p["s_src"])
        s_z = scale_of.get(id(p["z"]), p["s_z"]) if p["z"] is not None else 1.0
        k = (L.ic // L.group) * L.f * L.f
        src2 = float((p["src"].float() ** 2).mean())
        flt2 = float((p["flt"].float() ** 2).mean())
        sigma = max(1.0, (k * src2 * flt2) ** 0.5)
        p["bias"].copy_(torch.from_numpy(rng.uniform(1.3 * sigma, 1.9 * sigma, tuple(p["bias"].shape)).astype(np.int32)))
        if p["z"] is not None:
            s_dst = float(np.float32(s_z * rng.uniform(2.0, 3.0)))
        else:
            s_dst = float(np.float32(np.exp(rng.uniform(np.log(1e-3), np.log(5e-2)))))
        s_flt = np.float32(25.0 * s_dst / (sigma * s_src))
        s_bias = float(np.float32(s_src) * s_flt)
        p["desc"] = L.desc(s_bias, s_z, s_dst)
        scale_of[id(p["dst"])] = s_dst
        choose_algorithms([p], weight_preprocess)
        bind_plan([p])[0]()
        lo = 0 if L.nonline == "RELU" else -128
        d = p["dst"]
        live.append(float(((d > lo) & (d < 127)).float().mean()))
    torch.cuda.synchronize()
    return live


def choose_algorithms(plan, weight_preprocess=True, tiles=None):
    """Algorithm choice for every layer of a plan, as an inference graph does it once at load time: the heuristic
    (for a caller that pre-processes weights when `weight_preprocess`), then exec_preprocess of the filter where the
    chosen algorithm has a pre-processed form.  Fills p["algo"] and p["pre"] (None: exec takes the filter).
    `tiles` = {layer name: tile name}: those layers run the named tile of the MFMA algorithm instead (measurements)."""
    from . import lib, ops
    names = lib.tile_names() if tiles else []
    for p in plan:
        req = _abi.ALGO_HEURISTIC_PREPROCESS if weight_preprocess else _abi.ALGO_HEURISTIC
        p["algo"], _ = ops.conv_bias_query(p["desc"], req)
        if tiles and p["layer"].name in tiles:
            p["algo"], _ = ops.conv_bias_query(p["desc"], 1)
            p["algo"].tile_cfg = names.index(tiles[p["layer"].name])
        p["pre"] = ops.conv_bias_preprocess(p["desc"], p["flt"], p["algo"]) if weight_preprocess else None
    return plan


def bind_plan(plan, stream=None):
    """One pre-marshalled launch per layer (exec, or exec with the PreprocessedFilter)."""
    from . import ops
    return [ops.conv_bias_bind(p["desc"], p["src"], p["flt"], p["bias"], p["z"], p["dst"], p["algo"], stream=stream,
                               preprocessed=p.get("pre")) for p in plan]
