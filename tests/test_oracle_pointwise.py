"""The numpy restatement of the per-channel Operations (oracle/pointwise_oracle.py) held against closed forms and against
the reference's CPU backend running the same chains (tests/cases/pointwise_chains.h compiled against the reference's
headers: oracle/_ref).  No GPU."""
import numpy as np
import pytest

import oracle_lib as ol
import pointwise_cases as pc

po = ol.pointwise_oracle()
ALL = sorted(po.CASES)


def test_closed_forms():
    f = np.array([[[-2.5, 0.0, 3.0], [-0.0, np.nan, -np.inf]]], np.float32)
    a = po.run(0, f)
    assert a[0, 0].tolist() == [2.5, 0.0, 3.0] and np.signbit(a[0, 1, 0]) and np.isnan(a[0, 1, 1]) and a[0, 1, 2] == np.inf
    assert po.run(1, np.array([[-7, 7, -2**31]], np.int32)).tolist() == [[7, 7, -2**31]]          # the most negative int stays
    assert po.run(2, np.array([[[-128, -1, 5]]], np.int8)).tolist() == [[[-128, 1, 5]]]
    assert po.run(4, np.array([[[255, 16, 0]]], np.uint8)).tolist() == [[[65025, 256, 0]]]          # done in int, not in uchar
    assert po.run(5, np.array([[[16.0, 2.25, 0.0]]], np.float32)).tolist() == [[[4.0, 1.5, 0.0]]]
    assert po.run(6, np.array([[[144, 81, 1]]], np.uint8)).tolist() == [[[12.0, 9.0, 1.0]]]
    assert abs(float(po.run(7, np.array([[np.e ** 3]], np.float32))[0, 0]) - 3.0) < 1e-6
    assert po.run(8, np.array([[[0.0, 0.0, 0.0]]], np.float32)).tolist() == [[[1.0, 1.0, 1.0]]]
    assert po.run(9, np.array([[[1.0, 1.0, 1.0]]], np.float32), c=(0.25, -3.5, 100.0, 0)).tolist() == [[[0.75, 4.5, 99.0]]]
    assert po.run(10, np.array([[-80, 3]], np.int32), c=(-77, 0, 0, 0)).tolist() == [[3, 80]]
    nan = np.float32(np.nan)
    mx = po.run(11, np.array([[[nan, -2.0, 2.0]]], np.float32), c=(0.0, -1.5, 2.5, 0))
    assert np.isnan(mx[0, 0, 0]) and mx[0, 0, 1:].tolist() == [-1.5, 2.5]                           # (a < b) ? b : a keeps a NaN input
    mn = po.run(12, np.array([[[nan, -2.0, 2.0]]], np.float32), c=(0.0, -1.5, 2.5, 0))
    assert np.isnan(mn[0, 0, 0]) and mn[0, 0, 1:].tolist() == [-2.0, 2.0]
    assert po.run(13, np.array([[7, 200]], np.uint8), c=(100, 0, 0, 0)).tolist() == [[100, 200]]
    assert po.run(15, np.array([[0x12345678]], np.uint32), c=(0x00ffff00, 0, 0, 0)).tolist() == [[0x00345600]]
    assert po.run(16, np.array([[[0x10, 2, 255]]], np.int32), c=(0x0f0f, 1, -256, 0)).tolist() == [[[0x0f1f, 3, -1]]]
    assert po.run(17, np.array([[0xffffffff]], np.uint32), c=(0x7fffff80, 0, 0, 0)).tolist() == [[0x8000007f]]
    assert po.run(18, np.array([[0, 0xffffffff, 0x0000ffff]], np.uint32)).tolist() == [[0xffffffff, 0, 0xffff0000]]
    assert po.run(19, np.array([[1, 0x08000001]], np.uint32), c=(5, 0, 0, 0)).tolist() == [[32, 0x20]]  # bits shifted out are gone
    assert po.run(20, np.array([[-64, 64]], np.int32), c=(3, 0, 0, 0)).tolist() == [[-8, 8]]             # arithmetic shift
    v = np.array([[[1.0, 2.0, 3.0]]], np.float32)
    assert po.run(21, v).tolist() == v.tolist()                                                       # identity matrix
    assert po.run(21, v, m=(0, 0, 1, 0, 1, 0, 1, 0, 0)).tolist() == [[[3.0, 2.0, 1.0]]]
    assert po.run(23, np.array([[[-32768, -5]]], np.int16)).tolist() == [[[-32768, 5]]]


def test_constants_of_the_chain_text_convert_like_c_casts():
    # 0x7fffff80 is the largest float below 2**31 (a float constant converted to uint by the chain text): exact
    assert float(np.float32(0x7fffff80)) == 0x7fffff80 and float(np.float32(0x00ffff00)) == 0x00ffff00


@pytest.mark.skipif(not ol.have_ref(), reason="oracle/_ref not built")
@pytest.mark.parametrize("which", ALL)
def test_oracle_equals_the_reference_backend(which):
    for seed, (h, w) in enumerate(((5, 9), (16, 33))):
        src = pc.inputs(which, po.CASES, h, w, seed)
        want = ol.ref_pointwise(which, src, pc.constants(which), pc.MATRIX)
        got = po.run(which, src, pc.constants(which), pc.MATRIX)
        assert got.dtype == want.dtype and pc.same(which, got, want, po.INEXACT), (which, seed)


@pytest.mark.parametrize("which", ALL)
def test_oracle_equals_the_committed_reference_vectors(which):
    # tests/golden/pointwise_reference_vectors.npz: outputs of the reference's CPU backend (make_pointwise_golden.py)
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "pointwise_reference_vectors.npz"))
    src = pc.inputs(which, po.CASES, 5, 9, 0)
    assert src.tobytes() == g[f"in_{which}"].tobytes(), "the seeded inputs changed: regenerate the fixture"
    assert pc.same(which, po.run(which, src, pc.constants(which), pc.MATRIX), g[f"out_{which}"], po.INEXACT)


def _split_input(which, h, w, seed):
    in_dtype, cn, _ = ol.SPLIT_WRITE_CASES[which]
    rng = np.random.default_rng(500 + 10 * which + seed)
    if in_dtype == np.uint8:
        return rng.integers(0, 256, (h, w, cn), dtype=np.uint8)
    return rng.uniform(-100, 100, (h, w, cn)).astype(np.float32)


def test_split_write_closed_form():
    src = np.arange(2 * 3 * 3, dtype=np.uint8).reshape(2, 3, 3)
    planes = ol.oracle_split_write(0, src)
    assert [p.tolist() for p in planes] == [[[0, 3, 6], [9, 12, 15]], [[1, 4, 7], [10, 13, 16]], [[2, 5, 8], [11, 14, 17]]]


@pytest.mark.skipif(not ol.have_ref(), reason="oracle/_ref not built")
@pytest.mark.parametrize("which", sorted(ol.SPLIT_WRITE_CASES))
def test_split_write_equals_the_reference_backend(which):
    # every output image with a pitch of its own
    for seed, (h, w) in enumerate(((24, 40), (37, 53))):
        src = _split_input(which, h, w, seed)
        dst = (29, 17) if which == 3 else None
        c = (0.5, -2.0, 3.25, 0)
        want = ol.ref_split_write(which, src, dst, c, pad=(0, 3, 1, 2))
        got = ol.oracle_split_write(which, src, dst, c)
        assert len(got) == len(want)
        for g, r in zip(got, want):
            assert g.dtype == r.dtype and g.tobytes() == r.tobytes(), (which, seed)


def test_two_image_closed_forms():
    a = np.array([[[1.0, 2.0, 3.0]]], np.float32)
    b = np.array([[[0.5, -2.0, 4.0]]], np.float32)
    assert po.run_dual(0, a, b).tolist() == [[[1.5, 0.0, 7.0]]] and po.run_dual(4, a, b).tolist() == [[[0.5, 4.0, -1.0]]]
    assert po.run_dual(3, a, b).tolist() == [[[2.0, -1.0, 0.75]]] and po.run_dual(6, a, b).tolist() == [[[1.0, 2.0, 4.0]]]
    u = np.array([[[0, 255, 7]]], np.uint8)
    v = np.array([[[255, 0, 9]]], np.uint8)
    assert po.run_dual(1, u, v).tolist() == [[[255, 255, 2]]]                    # the difference is taken in int
    assert po.run_dual(8, u, v).tolist() == [[[128, 128, 8]]]                    # 127.5 rounds to the even 128, 8.0 stays
    x = np.array([[0xff00ff00, 0x0f0f0f0f]], np.uint32)
    y = np.array([[0x0ff00ff0, 0xffffffff]], np.uint32)
    assert po.run_dual(5, x, y).tolist() == [[0xf0f0f0f0, 0xf0f0f0f0]] and po.run_dual(9, x, y).tolist() == [[0x0f000f00, 0x0f0f0f0f]]
    assert po.run_dual(7, np.array([[5, -9]], np.int32), np.array([[-5, 9]], np.int32)).tolist() == [[-5, -9]]


@pytest.mark.skipif(not ol.have_ref(), reason="oracle/_ref not built")
@pytest.mark.parametrize("which", sorted(po.DUAL_CASES))
def test_two_image_chains_equal_the_reference_backend(which):
    for seed, (h, w) in enumerate(((6, 11), (19, 34))):
        a, b = pc.dual_inputs(which, po.DUAL_CASES, h, w, seed)
        want = ol.ref_dual(which, a, b, pad=(0, 8))
        got = po.run_dual(which, a, b)
        assert got.dtype == want.dtype and got.tobytes() == want.tobytes(), (which, seed)


def test_two_image_and_split_chains_equal_the_committed_reference_vectors():
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "pointwise_reference_vectors.npz"))
    for which in sorted(po.DUAL_CASES):
        a, b = pc.dual_inputs(which, po.DUAL_CASES, 6, 11, 0)
        assert a.tobytes() == g[f"dual_a_{which}"].tobytes() and b.tobytes() == g[f"dual_b_{which}"].tobytes()
        assert po.run_dual(which, a, b).tobytes() == g[f"dual_out_{which}"].tobytes(), which
    for which in sorted(ol.SPLIT_WRITE_CASES):
        src = _split_input(which, 24, 40, 0)
        assert src.tobytes() == g[f"split_in_{which}"].tobytes()
        planes = ol.oracle_split_write(which, src, (29, 17) if which == 3 else None, (0.5, -2.0, 3.25, 0))
        for k, plane in enumerate(planes):
            assert plane.tobytes() == g[f"split_out_{which}_{k}"].tobytes(), (which, k)


@pytest.mark.skipif(not ol.have_ref(), reason="oracle/_ref not built")
def test_oracle_equals_the_reference_backend_on_the_sweep_of_random_sizes():
    # the 800 cases tests/test_gpu_pointwise.py runs on the GPU (pointwise_cases.sweep_case)
    for i in range(800):
        two, which, w, h, pads = pc.sweep_case(i, po.CASES, po.DUAL_CASES)
        if not two:
            src = pc.inputs(which, po.CASES, h, w, i)
            want = ol.ref_pointwise(which, src, pc.constants(which), pc.MATRIX)
            assert pc.same(which, po.run(which, src, pc.constants(which), pc.MATRIX), want, po.INEXACT), (i, which, w, h)
        else:
            a, b = pc.dual_inputs(which, po.DUAL_CASES, h, w, i)
            want = ol.ref_dual(which, a, b, pad=tuple(pads))
            got = po.run_dual(which, a, b)
            same = got.tobytes() == want.tobytes() or np.array_equal(np.isnan(got), np.isnan(want)) and \
                np.array_equal(got[~np.isnan(got)].view(np.uint8), want[~np.isnan(want)].view(np.uint8))
            assert got.dtype == want.dtype and same, (i, which, w, h)
