"""Parity on the benchmark's own plans: the exact layer lists, tensors, drawn scales and algorithm choices that
bench.py times (megengine_amd.workloads), at their full sizes.

Every layer runs through the heuristic exactly as in the bench; its output is
  * checked at >= 20 000 seeded random positions against the CPU checker evaluated on the layer's real input (the
    previous layer's GPU output, so an error cannot hide behind a matching downstream error), and
  * compared element for element with the generic one-thread-per-output kernel (itself pinned to the checker on
    small shapes, and which never uses the one-FMA requantisation form).
The shape lists are the reference's own benchmark shapes (dnn/test/cuda/conv_bias_int8.cpp:1127-1153,
dnn/test/cuda/conv_test_utils.cpp:23-55)."""
import numpy as np
import pytest
import torch

from megengine_amd import _abi, lib, ops, workloads
from tests import util
from tests.gpu_util import say

pytestmark = pytest.mark.gpu

DIRECT, IGEMM, DW, C4 = 0, 1, 2, 3
NPOINTS = 20000


def host(t):
    return None if t is None else t.cpu().numpy()


def run_plan(plan):
    """exactly what bench.py launches: the heuristic for pre-processing callers, filters pre-processed where the chosen
    algorithm has such a form"""
    workloads.choose_algorithms(plan)
    for call in workloads.bind_plan(plan):
        call()
    torch.cuda.synchronize()


def check_layer(oracle, p, seed):
    l, d = p["layer"], p["desc"]
    say("layer", l.name, "ic", l.ic, "oc", l.oc, "hw", l.ih, "f", l.f, "s", l.stride, "g", l.group, "z", l.z is not None,
        "algo", lib.algo_names()[p["algo"].id], lib.tile_names()[p["algo"].tile_cfg] if p["algo"].id == IGEMM else "",
        "pre-processed filter" if p.get("pre") is not None else "")
    got = p["dst"]
    idx = (util.splitmix64(seed, NPOINTS) % np.uint64(got.numel())).astype(np.int64)
    want = oracle.conv_bias_points(d, host(p["src"]), host(p["flt"]), host(p["bias"]), host(p["z"]), idx)
    g = got.reshape(-1)[torch.from_numpy(idx).cuda()].cpu().numpy()
    bad = np.nonzero(g != want)[0]
    assert len(bad) == 0, "%s: %d / %d sampled outputs differ, first idx %d got %d want %d" % (
        l.name, len(bad), NPOINTS, idx[bad[0]], g[bad[0]], want[bad[0]])
    ref = ops.conv_bias_exec(d, p["src"], p["flt"], p["bias"], p["z"], algo=DIRECT)
    torch.cuda.synchronize()
    assert torch.equal(got, ref), "%s differs from the generic kernel" % l.name


# ---------------------------------------------------------------------------------------------
# config 2: the 53-layer ResNet-50 stack at batch 64 with the bench's seed
# ---------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def resnet_plan():
    torch.manual_seed(1234)
    plan = workloads.build_stack(workloads.resnet50(64), 7)
    run_plan(plan)
    yield plan
    del plan
    torch.cuda.empty_cache()


@pytest.mark.parametrize("part", range(6))
def test_config2_resnet50_stack(oracle, resnet_plan, part):
    plan = resnet_plan
    assert len(plan) == 53
    for i in range(part, len(plan), 6):
        check_layer(oracle, plan[i], seed=1000 + i)


@pytest.fixture(scope="module")
def resnet_live_plan():
    """The same 53 layers, tensors and algorithm choices with scales and biases calibrated layer by layer so that the
    compared bytes are live values: with the bench's scale recipe most outputs of a long reduction sit at a clamp (0 or
    127), where a wrong accumulator in a minority of lanes would hide."""
    torch.manual_seed(1234)
    plan = workloads.build_stack(workloads.resnet50(64), 7)
    live = workloads.run_calibrated(plan, 77)
    yield plan, live
    del plan
    torch.cuda.empty_cache()


@pytest.mark.parametrize("part", range(6))
def test_config2_resnet50_stack_on_live_values(oracle, resnet_live_plan, part):
    plan, live = resnet_live_plan
    assert len(plan) == 53
    for i in range(part, len(plan), 6):
        say("live outputs", plan[i]["layer"].name, "%.3f" % live[i])
        assert live[i] >= 0.75, (plan[i]["layer"].name, live[i])
        check_layer(oracle, plan[i], seed=5000 + i)


@pytest.mark.parametrize("in_place", [False, True])
def test_static_memory_plan_changes_no_output(in_place):
    """The benchmark lays the activations of the stack out by liveness (workloads.plan_memory).  The planned stack
    must produce, layer by layer, the bytes of the stack with one buffer per output; no layer may write a buffer it
    reads -- except, with `in_place`, the residual that it reads last, which its output replaces -- and a buffer may
    only be reused after its last reader."""
    def build():
        torch.manual_seed(77)
        return workloads.choose_algorithms(workloads.build_stack(workloads.resnet50(4), 7))
    ref = build()
    for c in workloads.bind_plan(ref):
        c()
    torch.cuda.synchronize()
    plan = build()
    mem = workloads.plan_memory(plan, residual_in_place=in_place)
    assert mem["planned"] < (0.25 if in_place else 0.35) * mem["one_buffer_per_layer"]
    over = 0
    for p in plan:
        w = p["dst"].data_ptr()
        assert w != p["src"].data_ptr(), p["layer"].name
        if p["z"] is not None and w == p["z"].data_ptr():
            over += 1
    assert over == (16 if in_place else 0)
    snaps = workloads.snapshot_run(plan, workloads.bind_plan(plan), 4)
    for p, r, (h_src, h_z, h_dst) in zip(plan, ref, snaps):
        assert np.array_equal(h_src, r["src"].cpu().numpy()), "source of " + p["layer"].name
        assert r["z"] is None or np.array_equal(h_z, r["z"].cpu().numpy()), "residual of " + p["layer"].name
        assert np.array_equal(h_dst, r["dst"].cpu().numpy()), "output of " + p["layer"].name
    # and a second step over the same buffers (what a replayed graph does) ends on the same bytes
    snaps2 = workloads.snapshot_run(plan, workloads.bind_plan(plan), 4)
    assert all(np.array_equal(a[2], b[2]) for a, b in zip(snaps, snaps2))


def test_config2_uses_preprocessed_filters(resnet_plan):
    n = sum(p.get("pre") is not None for p in resnet_plan)
    say(n, "of 53 layers run with a pre-processed filter")
    assert n >= 20


def test_config2_requantisation_forms(resnet_plan):
    """The drawn scales send most layers without a residual through the one-FMA (linear) form -- the bench's timed
    kernels -- and the rest through the multi-step form: both are what test_config2_resnet50_stack compared."""
    import ctypes as C
    lin = other = 0
    for p in resnet_plan:
        d = p["desc"]
        if d.has_z:
            continue
        c, dd = C.c_float(), C.c_float()
        ok = lib.lib().mi355_epilogue_linear_form(C.c_float(d.scale_bias), C.c_float(d.scale_dst), d.nonline, C.byref(c),
                                                 C.byref(dd))
        lin += ok == 1
        other += ok != 1
    say("linear form on", lin, "layers, multi-step form on", other, "layers without residual; 16 layers have a residual")
    assert lin + other == 37
    assert lin >= 28 and other >= 1


# ---------------------------------------------------------------------------------------------
# config 1: the pointwise sweep, all five shapes x IDENTITY / RELU, residual on the expanding ones
# ---------------------------------------------------------------------------------------------

def test_config1_pointwise_sweep(oracle):
    torch.manual_seed(99)
    layers = workloads.pointwise_sweep()
    assert len(layers) == 10
    for i, l in enumerate(layers):
        plan = workloads.build_stack([l], 20 + i)
        # the scales the configuration names
        d = l.desc(2e-4, 0.05, 0.05)
        plan[0]["desc"] = d
        run_plan(plan)
        assert plan[0]["algo"].id == IGEMM
        check_layer(oracle, plan[0], seed=2000 + i)
        del plan
    torch.cuda.empty_cache()


# ---------------------------------------------------------------------------------------------
# config 0: the reference's CPU-runnable case, whole tensor against the checker
# ---------------------------------------------------------------------------------------------

def test_config0_whole_tensor(oracle):
    l = workloads.config0()
    d = l.desc(2e-4, 1.0, 0.05)
    src, flt, bias, z = util.make_tensors(d, seed=42, bias_range=(-1000, 1000))
    want = oracle.conv_bias(d, src, flt, bias, None)
    got = ops.conv_bias_exec(d, torch.from_numpy(src).cuda(), torch.from_numpy(flt).cuda(), torch.from_numpy(bias).cuda())
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)


# ---------------------------------------------------------------------------------------------
# config 3: all 48 MobileNetV2 layers at batch 64
# ---------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def mobilenet_plan():
    torch.manual_seed(4321)
    plan = workloads.build_stack(workloads.mobilenet_v2(), 3)
    run_plan(plan)
    yield plan
    del plan
    torch.cuda.empty_cache()


@pytest.fixture(scope="module")
def mobilenet_live_plan():
    torch.manual_seed(4321)
    plan = workloads.build_stack(workloads.mobilenet_v2(), 3)
    live = workloads.run_calibrated(plan, 33)
    yield plan, live
    del plan
    torch.cuda.empty_cache()


@pytest.mark.parametrize("part", range(4))
def test_config3_mobilenetv2_on_live_values(oracle, mobilenet_live_plan, part):
    """Calibrated scales: the depthwise kernel, the 4-packed pointwise tiles and the streaming kernel at full size on
    values inside the int8 range."""
    plan, live = mobilenet_live_plan
    for i in range(part, len(plan), 4):
        p = plan[i]
        say("live outputs", p["layer"].name, "%.3f" % live[i])
        assert live[i] >= 0.75, (p["layer"].name, live[i])
        assert p["algo"].id == (DW if p["layer"].group > 1 else IGEMM)
        check_layer(oracle, p, seed=6000 + i)


@pytest.mark.parametrize("part", range(4))
def test_config3_mobilenetv2(oracle, mobilenet_plan, part):
    plan = mobilenet_plan
    assert len(plan) == 48
    for i in range(part, len(plan), 4):
        p = plan[i]
        assert p["algo"].id == (DW if p["layer"].group > 1 else IGEMM)
        check_layer(oracle, p, seed=3000 + i)


# ---------------------------------------------------------------------------------------------
# config 4: the three large cases at batch 128 as the timed chain
#     NCHW -> NCHW32 relayout, ConvBias (+ bias, z, H_SWISH), NCHW32 -> NCHW relayout
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("case", range(3))
def test_config4_chain_at_batch_128(oracle, case):
    l = workloads.large_hswish()[case]
    assert l.n == 128
    d = l.desc(float(np.float32(0.02) * np.float32(0.01)), 0.05, 0.05)
    say("config 4 chain", l.name)
    g = torch.Generator(device="cuda")
    g.manual_seed(400 + case)
    x_nchw = torch.randint(-128, 128, (l.n, l.ic, l.ih, l.iw), dtype=torch.int8, device="cuda", generator=g)
    ss, fs, bs, ds = _abi.conv_shapes(d)
    flt = torch.randint(-127, 128, fs, dtype=torch.int8, device="cuda", generator=g)
    bias = torch.randint(-1000, 1001, bs, dtype=torch.int32, device="cuda", generator=g)
    z = torch.randint(-128, 128, ds, dtype=torch.int8, device="cuda", generator=g)
    src32 = ops.relayout_exec(ops.relayout_desc(_abi.RL_NCHW_NCHW32, tuple(x_nchw.shape)), x_nchw)
    # what the bench launches: the heuristic for a caller that pre-processes weights (the 8-wave second-generation tiles,
    # which read the residual in the epilogue), exec with the PreprocessedFilter
    algo, _ = ops.conv_bias_query(d, _abi.ALGO_HEURISTIC_PREPROCESS)
    assert algo.id == IGEMM
    tile = lib.tile_names()[algo.tile_cfg]
    say("tile", tile)
    assert tile in ("v2_256x256x64r3w8", "v2_128x256x64r3w8")
    pre = ops.conv_bias_preprocess(d, flt, algo)
    assert pre is not None
    dst32 = ops.conv_bias_exec_preprocessed(d, src32, pre, bias, z, algo=algo)
    # ... and the choice of a caller that hands over the filter as it is
    plain_algo, _ = ops.conv_bias_query(d)
    assert plain_algo.id == IGEMM
    dst_plain = ops.conv_bias_exec(d, src32, flt, bias, z, algo=plain_algo)
    y_nchw = ops.relayout_exec(ops.relayout_desc(_abi.RL_NCHW32_NCHW, tuple(dst32.shape)), dst32)
    torch.cuda.synchronize()
    assert tuple(y_nchw.shape) == (l.n, l.oc, l.oh, l.ow)

    # the chain composed on the host: closed-form permutation of the input, the checker at sampled positions of the
    # final NCHW tensor
    idx = (util.splitmix64(4000 + case, NPOINTS) % np.uint64(y_nchw.numel())).astype(np.int64)
    n_, r = np.divmod(idx, l.oc * l.oh * l.ow)
    c_, r = np.divmod(r, l.oh * l.ow)
    h_, w_ = np.divmod(r, l.ow)
    idx32 = (((n_ * (l.oc // 32) + c_ // 32) * l.oh + h_) * l.ow + w_) * 32 + c_ % 32
    src_host = util.nchw_to_packed(x_nchw.cpu().numpy(), 32)
    want = oracle.conv_bias_points(d, src_host, host(flt), host(bias), host(z), idx32)
    got = y_nchw.reshape(-1)[torch.from_numpy(idx).cuda()].cpu().numpy()
    bad = np.nonzero(got != want)[0]
    assert len(bad) == 0, "%d / %d sampled outputs of the chain differ" % (len(bad), NPOINTS)
    # the relayouts are permutations: whole tensors against torch
    assert torch.equal(src32, x_nchw.view(l.n, l.ic // 32, 32, l.ih, l.iw).permute(0, 1, 3, 4, 2).contiguous())
    assert torch.equal(y_nchw, dst32.permute(0, 1, 4, 2, 3).reshape(l.n, l.oc, l.oh, l.ow))
    # every element of the convolution against the generic kernel
    ref = ops.conv_bias_exec(d, src32, flt, bias, z, algo=DIRECT)
    torch.cuda.synchronize()
    assert torch.equal(dst32, ref)
    assert torch.equal(dst_plain, ref)
    # the patch-staged tiles at full size (stride-1 cases; every usable one, with the pre-processed filter)
    names = lib.tile_names()
    staged = [t for t, nm in enumerate(names) if nm.startswith("v3_") and lib.tile_usable(d, t)]
    assert (len(staged) >= 2) == (l.stride == 1), (l.name, [names[t] for t in staged])
    for t in staged:
        say("patch-staged tile", names[t])
        a3, _ = ops.conv_bias_query(d, IGEMM)
        a3.tile_cfg = t
        pre3 = ops.conv_bias_preprocess(d, flt, a3)
        out3 = ops.conv_bias_exec_preprocessed(d, src32, pre3, bias, z, algo=a3)
        torch.cuda.synchronize()
        assert torch.equal(out3, ref), names[t]
        del out3, pre3
    del x_nchw, src32, dst32, dst_plain, y_nchw, ref, z
    torch.cuda.empty_cache()
