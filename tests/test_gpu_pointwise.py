"""GPU parity of the per-channel Operations of math.h / logical.h / bitwise.h / algebraic.h (Abs, Sqr, Sqrt, Ln, Exp, AbsDiff,
Max, Min, BwAnd, BwOr, BwXor, BwNot, ShiftLeft, ShiftRight, MxVFloat3) in a chain Read -> Operation -> Write: the chain
texts of tests/cases/pointwise_chains.h through the C++ host API and the C ABI, compiled at run time, against the numpy
restatement (oracle/pointwise_oracle.py, itself pinned by the reference's CPU backend).  Bit-exact, except Ln and Exp:
the platform's logf / expf, 1e-5 relative."""
import numpy as np
import pytest

import fkl_cases as cases
import oracle_lib as ol
import pointwise_cases as pc

po = ol.pointwise_oracle()
ALL = sorted(po.CASES)


def run_on_gpu(device, which, src, pad_in=0, pad_out=0):
    import torch
    in_dtype, cn, out_dtype = po.CASES[which]
    h, w = src.shape[:2]
    in_row = w * cn * np.dtype(in_dtype).itemsize
    out_row = w * cn * np.dtype(out_dtype).itemsize
    host_in = np.zeros((h, in_row + pad_in), np.uint8)
    host_in[:, :in_row] = np.ascontiguousarray(src).view(np.uint8).reshape(h, in_row)
    dev_in = torch.from_numpy(host_in).to(device)
    dev_out = torch.full((h, out_row + pad_out), 0xA5, dtype=torch.uint8, device=device)
    cases.pointwise(which, dev_in, w, h, dev_out, pc.constants(which), pc.MATRIX)
    torch.cuda.synchronize()
    got = dev_out.cpu().numpy()
    assert np.all(got[:, out_row:] == 0xA5), "bytes beyond the rows were written"
    return np.ascontiguousarray(got[:, :out_row]).view(out_dtype).reshape(src.shape)


@pytest.mark.gpu
@pytest.mark.parametrize("which", ALL)
def test_operation_matches_the_oracle(device, which):
    # a size with partial runs at the row ends, rows that start on odd addresses for the narrow types, and special values
    for seed, (h, w, pad_in, pad_out) in enumerate(((7, 45, 0, 0), (33, 130, 3, 5))):
        if np.dtype(po.CASES[which][0]).itemsize > 1 or np.dtype(po.CASES[which][2]).itemsize > 1:
            pad_in, pad_out = pad_in * 4, pad_out * 4          # rows of wider elements stay aligned to their element
        src = pc.inputs(which, po.CASES, h, w, seed)
        want = po.run(which, src, pc.constants(which), pc.MATRIX)
        got = run_on_gpu(device, which, src, pad_in, pad_out)
        assert pc.same(which, got, want, po.INEXACT), (which, seed)


@pytest.mark.gpu
@pytest.mark.parametrize("which", [9, 6, 4, 14, 23, 13])
def test_widths_around_a_wave_of_runs(device, which):
    # A wave moves 256 elements of a row (64 lanes x 4).  Waves that lie wholly inside a row take the dense form of the
    # accesses for 32- to 64-byte runs, the wave at the row's end and rows narrower than a wave the per-lane form; odd
    # heights leave the last thread row half used; padded pitches of byte images put rows on odd addresses.
    in_dtype, _, out_dtype = po.CASES[which]
    wide = np.dtype(in_dtype).itemsize > 1 or np.dtype(out_dtype).itemsize > 1
    for seed, (w, h, pad) in enumerate(((255, 5, 0), (256, 4, 0), (257, 3, 1), (260, 5, 0), (511, 2, 3), (512, 5, 0), (515, 1, 0),
                                        (768, 3, 2), (1021, 5, 0), (1024, 2, 0), (1283, 3, 0))):
        src = pc.inputs(which, po.CASES, h, w, 40 + seed)
        want = po.run(which, src, pc.constants(which), pc.MATRIX)
        got = run_on_gpu(device, which, src, pad * (4 if wide else 1), pad * (4 if wide else 1))
        assert pc.same(which, got, want, po.INEXACT), (which, w, h, pad)


@pytest.mark.gpu
def test_full_size_properties(device):
    # 4K: Abs is idempotent, Max then Min with the same constants clamps, x ^ c ^ c = x, (x << 5) >> 5 keeps the low bits
    h, w = 2160, 3840
    x = pc.inputs(0, po.CASES, h, w // 3, 7)
    a1 = run_on_gpu(device, 0, x)
    assert run_on_gpu(device, 0, a1).tobytes() == a1.tobytes() and not np.any(a1[np.isfinite(a1)] < 0)
    u = pc.inputs(17, po.CASES, h, w, 8)
    assert run_on_gpu(device, 17, run_on_gpu(device, 17, u)).tobytes() == u.tobytes()
    sh = run_on_gpu(device, 19, u)
    assert np.array_equal(sh, (u << np.uint32(5)))
    f = pc.inputs(11, po.CASES, h, w // 3, 9)
    lo = run_on_gpu(device, 11, f)
    fin = ~np.isnan(f)
    assert np.all(lo[fin] >= np.broadcast_to(np.array(pc.constants(11)[:3], np.float32), f.shape)[fin])


@pytest.mark.gpu
@pytest.mark.parametrize("which", sorted(ol.SPLIT_WRITE_CASES))
def test_split_write_matches_the_oracle(device, which):
    # SplitWrite<_2D, T>: one image per channel, each with a pitch of its own (padding columns must stay untouched)
    import torch
    import test_oracle_pointwise as t
    in_dtype, cn, out_dtype = ol.SPLIT_WRITE_CASES[which]
    tdt = {np.uint8: torch.uint8, np.float32: torch.float32}[out_dtype]
    for seed, (h, w) in enumerate(((24, 40), (37, 53), (64, 256))):
        src = t._split_input(which, h, w, seed)
        dst = (29, 17) if which == 3 else None
        dw, dh = dst if dst else (w, h)
        c = (0.5, -2.0, 3.25, 0)
        want = ol.oracle_split_write(which, src, dst, c)
        dev_in = torch.from_numpy(np.ascontiguousarray(src).view(np.uint8).reshape(h, -1)).to(device)
        pads = (0, 3, 1, 2) if out_dtype == np.float32 else (0, 3, 5, 2)
        bufs = [torch.full((dh, dw + pads[k]), 77, dtype=tdt, device=device) for k in range(cn)]
        cases.split_write(which, dev_in, w, h, [b[:, :dw] for b in bufs], dst, c)
        torch.cuda.synchronize()
        for k in range(cn):
            got = bufs[k].cpu().numpy()
            assert got[:, :dw].tobytes() == want[k].tobytes(), (which, seed, k)
            assert np.all(got[:, dw:] == 77), "padding columns were written"


def _same_with_any_nan(got, want):
    """Bit-exact, except that a NaN the operation itself produced (inf - inf, 0 / 0 ...) counts as equal to any NaN: which
    quiet NaN an invalid operation returns is the platform's choice (x86 sets the sign bit, the GPU does not)."""
    if got.dtype != np.float32:
        return got.tobytes() == want.tobytes()
    gn, wn = np.isnan(got), np.isnan(want)
    return np.array_equal(gn, wn) and got[~gn].tobytes() == want[~wn].tobytes()


@pytest.mark.gpu
@pytest.mark.parametrize("which", sorted(po.DUAL_CASES))
def test_two_image_chain_matches_the_oracle(device, which):
    # DualSourceRead<_2D, T> -> the two-input form of Add / Sub / Mul / Div / AbsDiff / Max / Min / BwAnd / BwOr / BwXor -> write
    import torch
    in_dtype, cn, out_dtype = po.DUAL_CASES[which]
    for seed, (h, w, pad_a, pad_b) in enumerate(((6, 11, 0, 0), (19, 34, 0, 8), (64, 256, 4, 0))):
        a, b = pc.dual_inputs(which, po.DUAL_CASES, h, w, seed)
        want = po.run_dual(which, a, b)
        row = w * cn * np.dtype(in_dtype).itemsize
        devs = []
        for img, extra in ((a, pad_a), (b, pad_b)):
            buf = np.zeros((h, row + extra), np.uint8)
            buf[:, :row] = np.ascontiguousarray(img).view(np.uint8).reshape(h, row)
            devs.append(torch.from_numpy(buf).to(device))
        out_row = w * cn * np.dtype(out_dtype).itemsize
        dev_out = torch.full((h, out_row + 4), 0xA5, dtype=torch.uint8, device=device)
        cases.dual(which, devs[0], devs[1], w, h, dev_out)
        torch.cuda.synchronize()
        got = dev_out.cpu().numpy()
        assert np.all(got[:, out_row:] == 0xA5)
        got = np.ascontiguousarray(got[:, :out_row]).view(out_dtype).reshape(want.shape)
        assert _same_with_any_nan(got, want), (which, seed)


@pytest.mark.gpu
def test_two_image_and_split_properties_at_full_size(device):
    # 4K: (a ^ b) ^ b = a through two launches of the two-image chain; the planes SplitWrite leaves recombine to the image
    import torch
    h, w = 2160, 3840
    rng = np.random.default_rng(99)
    a = rng.integers(0, 2**32, (h, w), dtype=np.uint64).astype(np.uint32)
    b = rng.integers(0, 2**32, (h, w), dtype=np.uint64).astype(np.uint32)
    da, db = (torch.from_numpy(x.view(np.uint8).reshape(h, w * 4)).to(device) for x in (a, b))
    c = torch.zeros_like(da)
    back = torch.zeros_like(da)
    cases.dual(5, da, db, w, h, c)
    cases.dual(5, c, db, w, h, back)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint32).reshape(h, w), a ^ b)
    assert back.cpu().numpy().tobytes() == a.tobytes()
    img = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
    dimg = torch.from_numpy(img.reshape(h, w * 3)).to(device)
    planes = [torch.zeros((h, w), dtype=torch.uint8, device=device) for _ in range(3)]
    cases.split_write(0, dimg, w, h, planes)
    torch.cuda.synchronize()
    assert np.stack([p.cpu().numpy() for p in planes], axis=-1).tobytes() == img.tobytes()


@pytest.mark.gpu
def test_sweep_of_random_sizes(device):
    # 800 seeded cases (tests/pointwise_cases.py: sweep_case): every per-channel and two-image chain at random sizes and pitches
    import torch
    for i in range(800):
        two, which, w, h, pads = pc.sweep_case(i, po.CASES, po.DUAL_CASES)
        if not two:
            src = pc.inputs(which, po.CASES, h, w, i)
            want = po.run(which, src, pc.constants(which), pc.MATRIX)
            got = run_on_gpu(device, which, src, pads[0], pads[1])
            assert pc.same(which, got, want, po.INEXACT), (i, which, w, h, pads)
            continue
        in_dtype, cn, out_dtype = po.DUAL_CASES[which]
        a, b = pc.dual_inputs(which, po.DUAL_CASES, h, w, i)
        want = po.run_dual(which, a, b)
        row = w * cn * np.dtype(in_dtype).itemsize
        devs = []
        for img, extra in ((a, pads[0]), (b, pads[1])):
            buf = np.zeros((h, row + extra), np.uint8)
            buf[:, :row] = np.ascontiguousarray(img).view(np.uint8).reshape(h, row)
            devs.append(torch.from_numpy(buf).to(device))
        out_row = w * cn * np.dtype(out_dtype).itemsize
        dev_out = torch.full((h, out_row + 4), 0xA5, dtype=torch.uint8, device=device)
        cases.dual(which, devs[0], devs[1], w, h, dev_out)
        torch.cuda.synchronize()
        got = dev_out.cpu().numpy()
        assert np.all(got[:, out_row:] == 0xA5), (i, which, w, h, pads)
        got = np.ascontiguousarray(got[:, :out_row]).view(out_dtype).reshape(want.shape)
        assert _same_with_any_nan(got, want), (i, which, w, h, pads)
