"""ccn_lamb_f32_static, the LAMB step that allocates nothing: its scratch (tile sums, norms, scales, index tables) is a
static device array inside the library, shared by every call on the GPU.

Checked against ccn_lamb_f32, the existing entry point whose plan owns that scratch: bit for bit against a plan that
takes the same two-pass kernels, and at the fp32 bar of the benchmark (1e-6 relative; m and v bit for bit) against a
plan as ccn_lamb_plan_create makes it by default.  Two calls in a row, the second on a smaller input, so that what
the first call left in the shared array must not leak into the second.
"""
import numpy as np
import pytest
import torch

import oracle as orc
from util import grads_f32, rel_err, weights_f32

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
FP32_TOL = 1e-6
HYPER = (1e-3, 0.9, 0.999, 1e-6, 0.01)
TWO_PASS = {1: 1}      # ccn_lamb_plan_tune(CCN_LAMB_KNOB_TWO_PASS, 1): every segment through the two-pass kernels


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def run_plan(ccn, g, w0, seg_len, steps, mode, knobs=None):
    N = w0.size
    gd = [dev(x) for x in g]
    wd, md, vd = dev(w0), torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    plan = ccn.LambPlan(list(range(0, N + 1, seg_len)), knobs=knobs or {})
    for t in range(1, steps + 1):
        plan.step(gd, wd, md, vd, *HYPER, t, mode)
    norms = plan.norms()
    plan.close()
    return host(wd), host(md), host(vd), norms


def run_static(ccn, g, w0, seg_len, steps, mode, with_norms=True):
    N = w0.size
    gd = [dev(x) for x in g]
    wd, md, vd = dev(w0), torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    nd = torch.zeros(2 * (N // seg_len), dtype=torch.float64, device=DEV) if with_norms else None
    for t in range(1, steps + 1):
        ccn.lamb_f32_static(gd, wd, md, vd, N, seg_len, *HYPER, t, mode, nd)
    return host(wd), host(md), host(vd), (host(nd).reshape(-1, 2) if with_norms else None)


# (P, segments, segment length): the second call of each pair is the smaller one.  The third pair has segments of
# more than 4096 tiles, whose tile sums go through groups, followed by a call that does not.
CASES = [
    ((8, 16, 1 << 16), (3, 5, 2048)),
    ((4, 37, 3072), (9, 1, 1024)),
    ((2, 2, 5 * 1024 * 1024), (2, 3, 4096)),
]


@pytest.mark.parametrize("first,second", CASES)
@pytest.mark.parametrize("mode", [0, 1])
def test_static_scratch_lamb_matches_the_plan_entry_point(ccn, first, second, mode):
    for case_no, (P, nseg, seg_len) in enumerate((first, second)):
        N = nseg * seg_len
        g = grads_f32(90 + case_no, P, N, 1e-3)
        w0 = weights_f32(90 + case_no, N, 0.05)
        got = run_static(ccn, g, w0, seg_len, 2, mode)
        # the same kernels through a plan: bit for bit, the norms included
        want = run_plan(ccn, g, w0, seg_len, 2, mode, TWO_PASS)
        for name, a, b in zip("wmv", got[:3], want[:3]):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (case_no, name, rel_err(a, b))
        assert np.array_equal(got[3], want[3]), (case_no, "norms")
        # the entry point as it is by default (segments that fit stay on chip: other summation order for the norms)
        dflt = run_plan(ccn, g, w0, seg_len, 2, mode)
        assert np.array_equal(got[1].view(np.uint32), dflt[1].view(np.uint32)), (case_no, "m")
        assert np.array_equal(got[2].view(np.uint32), dflt[2].view(np.uint32)), (case_no, "v")
        scale = float(np.max(np.abs(dflt[0])))
        assert np.max(np.abs(got[0].astype(np.float64) - dflt[0])) <= FP32_TOL * scale, (case_no, "w")
        assert rel_err(got[3], dflt[3]) < 1e-12, (case_no, "norms against the default plan")


@pytest.mark.parametrize("mode", [0, 1])
def test_static_scratch_lamb_against_the_oracle(ccn, mode):
    """Directly against the CPU oracle (not only against the plan entry point): two calls in a row, the second on a smaller
    input; m and v bit for bit, w to 1e-6, the norms to 1e-9 (float64 sums in another order)."""
    for case_no, (P, nseg, seg_len) in enumerate(((5, 12, 1 << 14), (3, 2, 3072))):
        N = nseg * seg_len
        g = grads_f32(93 + case_no, P, N, 1e-3)
        w0 = weights_f32(93 + case_no, N, 0.05)
        got = run_static(ccn, g, w0, seg_len, 2, mode)
        w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
        segs = list(range(0, N + 1, seg_len))
        for t in (1, 2):
            norms = orc.lamb_f32(g, w, m, v, segs, *HYPER, t, mode)
        assert np.array_equal(got[1].view(np.uint32), m.view(np.uint32)), (case_no, "m")
        assert np.array_equal(got[2].view(np.uint32), v.view(np.uint32)), (case_no, "v")
        assert np.max(np.abs(got[0].astype(np.float64) - w)) <= FP32_TOL * float(np.max(np.abs(w))), (case_no, "w")
        assert rel_err(got[3], np.asarray(norms).reshape(-1, 2)) < 1e-9, (case_no, "norms")


def test_static_scratch_lamb_calls_on_two_streams_in_order(ccn):
    """All calls on a GPU share the one static array, so calls on different streams must be ordered by the caller: a call
    on stream A, an event, stream B waits for it, a call on stream B on other buffers, and back.  Each result equals the
    same call made alone."""
    shapes = [(4, 8, 8192), (2, 3, 2048)]
    data = []
    for k, (P, nseg, seg_len) in enumerate(shapes):
        N = nseg * seg_len
        g, w0 = grads_f32(98 + k, P, N, 1e-3), weights_f32(98 + k, N, 0.05)
        data.append((g, w0, N, seg_len, run_static(ccn, g, w0, seg_len, 2, 0, with_norms=False)))
    a, b = ccn.Stream(), ccn.Stream()
    ev = [ccn.Event() for _ in range(4)]
    state = []
    for (g, w0, N, seg_len, _want) in data:
        state.append(([dev(x) for x in g], dev(w0), torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)))
    torch.cuda.synchronize()
    k = 0
    for t in (1, 2):
        for which, stream, other in ((0, a, b), (1, b, a)):
            gd, wd, md, vd = state[which]
            _g, _w0, N, seg_len, _want = data[which]
            ccn.lamb_f32_static(gd, wd, md, vd, N, seg_len, *HYPER, t, 0, None, stream.h)
            ev[k].record(stream)
            other.wait_event(ev[k])          # the next call, on the other stream, starts after this one has finished
            k += 1
    a.sync()
    b.sync()
    for which, (gd, wd, md, vd) in enumerate(state):
        want = data[which][4]
        for name, t_, w_ in zip("wmv", (wd, md, vd), want[:3]):
            assert np.array_equal(host(t_).view(np.uint32), w_.view(np.uint32)), (which, name)
    for e in ev:
        e.close()
    a.close()
    b.close()


def test_static_scratch_lamb_without_a_norms_array_and_unaligned(ccn):
    """norms = NULL keeps the norms in the static array; buffers 4 bytes off a 16-byte boundary take the scalar path."""
    P, nseg, seg_len = 3, 4, 2048
    N = nseg * seg_len
    g = grads_f32(95, P, N, 1e-3)
    w0 = weights_f32(95, N, 0.05)
    gd = [dev(np.concatenate([[np.float32(0)], x]))[1:] for x in g]
    wd = dev(np.concatenate([[np.float32(0)], w0]))[1:]
    md, vd = torch.zeros(N + 1, device=DEV)[1:], torch.zeros(N + 1, device=DEV)[1:]
    ccn.lamb_f32_static(gd, wd, md, vd, N, seg_len, *HYPER, 1, 0, None)
    want = run_plan(ccn, g, w0, seg_len, 1, 0, TWO_PASS)
    for name, a, b in zip("wmv", (host(wd), host(md), host(vd)), want[:3]):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), name


def test_static_scratch_lamb_rejects_what_it_cannot_hold(ccn):
    g = [torch.zeros(4096, device=DEV)]
    w, m, v = (torch.zeros(4096, device=DEV) for _ in range(3))
    call = lambda n, seg: ccn.lamb_f32_static(g, w, m, v, n, seg, *HYPER, 1, 0, None)
    for n, seg, code in [((1 << 28) + 1024, 1024, ccn.CCN_ERANGE),       # more elements than the array has tiles for
                         (4097 * 1024, 1024, ccn.CCN_ERANGE),            # more segments than it has norms for
                         (4096, 1000, ccn.CCN_EINVAL),                   # segments must be whole tiles
                         (4096 + 1024, 2048, ccn.CCN_EINVAL),            # and divide N
                         (0, 1024, ccn.CCN_EINVAL)]:
        with pytest.raises(ccn.CoconetError) as e:
            call(n, seg)
        assert e.value.code == code, (n, seg)
    torch.cuda.synchronize()
    assert float(w.abs().max()) == 0.0      # a rejected call launches nothing


def test_static_scratch_lamb_can_be_recorded_and_replayed(ccn):
    """The callers it is for: a recording of the call (ccn_graph_begin/end) replays to the same bits as eager calls.
    Every replay is checked, with eager work and synchronisations between the replays."""
    P, nseg, seg_len = 4, 6, 4096
    N = nseg * seg_len
    g = grads_f32(97, P, N, 1e-3)
    w0 = weights_f32(97, N, 0.05)
    gd = [dev(x) for x in g]
    wd, md, vd = dev(w0), torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    stream = ccn.Stream()
    torch.cuda.synchronize()
    with ccn.Graph(stream) as graph:
        ccn.lamb_f32_static(gd, wd, md, vd, N, seg_len, *HYPER, 1, 0, None, stream.h)
    we, me, ve = dev(w0), torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    for replay in range(3):
        graph.launch()
        stream.sync()
        # an eager call on other buffers between the replays leaves its own sums in the shared array
        other = [dev(x[:2048] * np.float32(3.0)) for x in g]
        ow, om, ov = dev(w0[:2048]), torch.zeros(2048, device=DEV), torch.zeros(2048, device=DEV)
        ccn.lamb_f32_static(other, ow, om, ov, 2048, 1024, *HYPER, 1, 0, None)
        torch.cuda.synchronize()
        ccn.lamb_f32_static(gd, we, me, ve, N, seg_len, *HYPER, 1, 0, None)      # the recording keeps step = 1
        for name, a, b in zip("wmv", (host(wd), host(md), host(vd)), (host(we), host(me), host(ve))):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (replay, name)
    graph.close()
    stream.close()
