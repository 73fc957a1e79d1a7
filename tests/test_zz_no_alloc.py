"""espdl_hip_mbconv_s8_staged: the inverted-residual block as separate stages with the intermediate
activations in the library's own device array, for callers that cannot allocate.  Its output is compared,
bit for bit, with the existing single-launch entry point espdl_hip_mbconv_s8 (and with the oracle) on
two calls in a row, the second with a smaller input, so that whatever the first call left in the shared
array must not reach the second call's result.  The calls between `hipDeviceSynchronize`s allocate
nothing: outputs are created beforehand."""
import numpy as np
import pytest

from cases import rng_int8, typical_shift
from gpu_util import announce, espdl, to_dev, to_host

pytestmark = pytest.mark.gpu


def _block(rng, n, h, w, cin, ce, cout, with_expand=True):
    def stage(oc, kk, fshape):
        f = rng_int8(rng, fshape)
        b = rng.integers(-4096, 4097, size=oc).astype(np.int32)
        s = (typical_shift(kk) + rng.integers(-2, 3, size=oc)).astype(np.int32)
        return f, b, s
    x = rng_int8(rng, (n, h, w, cin))
    expand = stage(ce, cin, (ce, 1, 1, cin)) if with_expand else None
    e = ce if with_expand else cin
    dw = stage(e, 9, (3, 3, e))
    proj = stage(cout, e, (cout, 1, 1, e))
    return x, expand, dw, proj


def _oracle_block(oracle, x, expand, dw, proj, stride, pads, res):
    cur = x
    if expand is not None:
        cur = oracle.conv2d_s8(cur, expand[0], expand[1], expand[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.RELU)
    cur = oracle.depthwise_s8(cur, dw[0], dw[1], dw[2], (3, 3), stride, (1, 1), pads, oracle.RELU)
    cur = oracle.conv2d_s8(cur, proj[0], proj[1], proj[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR)
    return oracle.add_s8(cur, res) if res is not None else cur


def test_staged_block_matches_the_single_launch_entry_point_twice_in_a_row(oracle):
    import torch
    m = espdl()
    rng = np.random.default_rng(0x57A6ED)
    dev = lambda t: None if t is None else tuple(to_dev(a) for a in t)  # noqa: E731
    # first call: 6 images 28x28, 32 -> 192 -> 32 with residual (3.7 MB of intermediates);
    # second call: 2 images 14x14, 64 -> 256 -> 64, stride 2, no residual (a smaller input, other extents)
    calls = [((6, 28, 28, 32), 192, 32, (1, 1), (1, 1, 1, 1), True),
             ((2, 14, 14, 64), 256, 64, (2, 2), (0, 1, 0, 1), False)]
    prepared = []
    for (n, h, w, cin), ce, cout, stride, pads, with_res in calls:
        x, expand, dw, proj = _block(rng, n, h, w, cin, ce, cout)
        oh = (h + pads[0] + pads[1] - 3) // stride[0] + 1
        ow = (w + pads[2] + pads[3] - 3) // stride[1] + 1
        res = rng_int8(rng, (n, oh, ow, cout)) if with_res else None
        want = _oracle_block(oracle, x, expand, dw, proj, stride, pads, res)
        args = (to_dev(x), dev(expand), dev(dw), dev(proj), (3, 3), stride, (1, 1), pads, (True, True, False))
        out_staged = torch.empty(want.shape, dtype=torch.int8, device="cuda")
        out_fused = torch.empty(want.shape, dtype=torch.int8, device="cuda")
        prepared.append((args, to_dev(res), out_staged, out_fused, want))
    torch.cuda.synchronize()
    for i, (args, res, out_staged, out_fused, want) in enumerate(prepared):
        announce("mbconv_s8_staged call %d %s" % (i, tuple(args[0].shape)))
        m.mbconv_s8(*args, residual=res, out=out_fused)
        m.mbconv_s8(*args, residual=res, out=out_staged, staged=True)
    for i, (args, res, out_staged, out_fused, want) in enumerate(prepared):
        np.testing.assert_array_equal(to_host(out_staged), to_host(out_fused), err_msg="call %d vs espdl_hip_mbconv_s8" % i)
        np.testing.assert_array_equal(to_host(out_staged), want, err_msg="call %d vs oracle" % i)


def test_staged_block_without_expand_and_the_size_limit(oracle):
    import torch
    m = espdl()
    rng = np.random.default_rng(0x57A6EE)
    dev = lambda t: None if t is None else tuple(to_dev(a) for a in t)  # noqa: E731
    x, _, dw, proj = _block(rng, 3, 20, 20, 48, None, 24, with_expand=False)
    want = _oracle_block(oracle, x, None, dw, proj, (1, 1), (1, 1, 1, 1), None)
    out = torch.empty(want.shape, dtype=torch.int8, device="cuda")
    announce("mbconv_s8_staged without expand")
    m.mbconv_s8(to_dev(x), None, dev(dw), dev(proj), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), (True, True, False), out=out,
                staged=True)
    np.testing.assert_array_equal(to_host(out), want)
    fused = m.mbconv_s8(to_dev(x), None, dev(dw), dev(proj), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), (True, True, False))
    np.testing.assert_array_equal(to_host(out), to_host(fused))
    # beyond the array: 80 images of 56x56x144 need 2 x 36 MB of intermediates, more than the 64 MiB it holds
    big = torch.zeros((80, 56, 56, 24), dtype=torch.int8, device="cuda")
    xb, expand, dwb, projb = _block(rng, 1, 56, 56, 24, 144, 24)
    announce("mbconv_s8_staged over the limit (host-side refusal, no launch)")
    with pytest.raises(m.capi.EspdlHipError) as err:
        m.mbconv_s8(big, dev(expand), dev(dwb), dev(projb), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), (True, True, False),
                    out=torch.empty((80, 56, 56, 24), dtype=torch.int8, device="cuda"), staged=True)
    assert "ESPDL_HIP_MBCONV_STAGED_MAX_BYTES" in str(err.value)


def test_staged_block_allocates_nothing_and_replays_under_a_captured_graph(oracle):
    """Free device memory is the same before and after staged calls, and the entry point can be recorded into a
    HIP graph once it has been called (or initialised) outside capture: three replays with new inputs in
    between, each compared with the eager result of the single-launch entry point."""
    import torch
    m = espdl()
    rng = np.random.default_rng(0x57A6EF)
    dev = lambda t: None if t is None else tuple(to_dev(a) for a in t)  # noqa: E731
    n, h, w, cin, ce, cout = 4, 28, 28, 32, 192, 32
    x, expand, dw, proj = _block(rng, n, h, w, cin, ce, cout)
    assert m.lib().espdl_hip_mbconv_s8_staged_init() == 0
    geom = ((3, 3), (1, 1), (1, 1), (1, 1, 1, 1), (True, True, False))
    xd, ed, dd, pd = to_dev(x), dev(expand), dev(dw), dev(proj)
    res = to_dev(rng_int8(rng, (n, h, w, cout)))
    out = torch.empty((n, h, w, cout), dtype=torch.int8, device="cuda")
    announce("mbconv_s8_staged warm call, then free-memory check")
    m.mbconv_s8(xd, ed, dd, pd, *geom, residual=res, out=out, staged=True)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        m.mbconv_s8(xd, ed, dd, pd, *geom, residual=res, out=out, staged=True)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    # capture on a side stream, replay with new inputs
    announce("mbconv_s8_staged under a captured graph")
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        m.mbconv_s8(xd, ed, dd, pd, *geom, residual=res, out=out, staged=True, stream=side.cuda_stream)
    for rep in range(3):
        x2 = rng_int8(rng, (n, h, w, cin))
        xd.copy_(torch.from_numpy(x2))
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = m.mbconv_s8(xd, ed, dd, pd, *geom, residual=res)
        np.testing.assert_array_equal(to_host(out), to_host(eager), err_msg="replay %d" % rep)
        want = _oracle_block(oracle, x2, expand, dw, proj, (1, 1), (1, 1, 1, 1), to_host(res))
        np.testing.assert_array_equal(to_host(out), want, err_msg="replay %d vs oracle" % rep)
