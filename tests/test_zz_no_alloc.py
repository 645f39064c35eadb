"""The block entry point that allocates nothing (sd3_dit_block_static: intermediates in a fixed per-device array) against
sd3_dit_block, through the C ABI: identical bits, on two calls in a row with the second one smaller, in both precisions;
blocks that do not fit the array and bf16 calls without prepared weight copies are refused with status codes."""
import numpy as np
import pytest

from gpu_util import M, dev, dev_params, host
from sd3_c_amd import lib as L
from sd3_c_amd.params import block_param_shapes, synthetic_params_numpy

pytestmark = pytest.mark.gpu


def _case(B, Tc, Tx, C, NH, seed, dual=True, discard=False):
    rng = np.random.Generator(np.random.Philox(seed))
    return dict(B=B, Tc=Tc, Tx=Tx, C=C, NH=NH, dual=dual, discard=discard, y=rng.standard_normal((B, C), dtype=np.float32),
                c=rng.standard_normal((B, Tc, C), dtype=np.float32), x=rng.standard_normal((B, Tx, C), dtype=np.float32))


def _run(ctx, k, precision, static):
    y, c, x = dev(k["y"]), dev(k["c"]), dev(k["x"])
    fn = ctx.block_static if static else ctx.block
    fn(y, c, x, k["B"], k["Tc"], k["Tx"], k["C"], k["NH"], 4, k["dual"], True, k["discard"], precision=precision)
    return host(c), host(x)


@pytest.mark.parametrize("precision", ["fp32", "bf16"])
def test_static_block_equals_block_on_two_calls_the_second_smaller(precision):
    C, NH = 128, 2
    params = dev_params(synthetic_params_numpy(block_param_shapes(C, 4, True, True, False, C // NH), 77, 0.1, 0.1))
    ctx = M.Context()
    try:
        ctx.bind(params)
        big, small = _case(2, 9, 300, C, NH, 5), _case(1, 4, 37, C, NH, 6)
        want = [_run(ctx, k, precision, static=False) for k in (big, small)]  # (also builds the bf16 weight copies)
        got = [_run(ctx, k, precision, static=True) for k in (big, small)]    # two calls in a row on the shared array
        for (cw, xw), (cg, xg), k in zip(want, got, (big, small)):
            assert np.array_equal(cg, cw) and np.array_equal(xg, xw)
            assert not np.array_equal(xg, k["x"])
    finally:
        ctx.close()


def test_static_block_refuses_what_does_not_fit_and_unprepared_bf16_weights():
    C, NH = 128, 2
    ctx = M.Context()
    try:
        ctx.bind(dev_params(synthetic_params_numpy(block_param_shapes(C, 4, True, True, False, C // NH), 78, 0.1, 0.1)))
        k = _case(1, 4, 37, C, NH, 7)
        with pytest.raises(L.Sd3Error) as e:
            _run(ctx, k, "bf16", static=True)  # no bf16 copies yet and nothing may be allocated
        assert e.value.status == 2
        huge = _case(2, 154, 4096, 1536, 24, 8)  # ~0.9 GB of fp32 intermediates
        with pytest.raises(L.Sd3Error) as e:
            _run(ctx, huge, "fp32", static=True)
        assert e.value.status == 3 and "fixed scratch" in str(e.value)
    finally:
        ctx.close()


@pytest.mark.parametrize("precision", ["fp32", "bf16"])
def test_static_block_leaves_device_memory_alone_with_profiling_on_and_under_graph_capture(precision):
    """What "allocates nothing" means, observed: the device's free memory (hipMemGetInfo) is the same before and after a call, also
    while the library's per-kernel profiling is switched on (which otherwise creates events), and the call can be captured into a HIP
    graph -- where an allocation would fail -- whose replays give the bits of sd3_dit_block."""
    import torch
    C, NH = 128, 2
    params = dev_params(synthetic_params_numpy(block_param_shapes(C, 4, True, True, False, C // NH), 79, 0.1, 0.1))
    ctx = M.Context()
    try:
        ctx.bind(params)
        k = _case(2, 9, 300, C, NH, 9)
        args = (k["B"], k["Tc"], k["Tx"], k["C"], k["NH"], 4, k["dual"], True, k["discard"])
        cw, xw = _run(ctx, k, precision, static=False)   # (also builds the bf16 weight copies)
        y, c, x = dev(k["y"]), dev(k["c"]), dev(k["x"])
        c0, x0 = c.clone(), x.clone()
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        ctx.profile_begin()
        ctx.block_static(y, c, x, *args, precision=precision)
        prof = ctx.profile_end()                          # (waits for the stream)
        assert torch.cuda.mem_get_info()[0] == free_before
        assert all(n == 0 for _, _, n in prof.values())   # no event was created or recorded for this call
        assert np.array_equal(host(c), cw) and np.array_equal(host(x), xw)
        graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
        c.copy_(c0); x.copy_(x0)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            ctx.block_static(y, c, x, *args, precision=precision)
        for _ in range(3):                                # every replay, with eager work and synchronisations in between
            c.copy_(c0); x.copy_(x0)
            torch.cuda.synchronize()
            graph.replay()
            assert np.array_equal(host(c), cw) and np.array_equal(host(x), xw)
    finally:
        ctx.close()
