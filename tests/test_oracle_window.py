"""CPU tests that pin the restatement of DivergentBatchTransformDPP launches and of the CircularTensor window
(reference data_parallel_patterns.h:286-381, circular_tensor.h:111-161) against the reference's CPU backend running
the same chain text (tests/cases/circular_chains.h), and against what the window means: plane z holds the image
given z updates ago (NewestFirst), or BATCH-1-z updates ago (OldestFirst)."""
import numpy as np
import pytest

import oracle_lib as ol

needs_ref = pytest.mark.skipif(not ol.have_ref(), reason="reference CPU backend (oracle/_ref) not built here")


def images(n, w, h, seed):
    r = np.random.default_rng(seed)
    return [r.integers(0, 256, (h, w, 3), dtype=np.uint8) for _ in range(n)]


@pytest.mark.parametrize("batch", [2, 3, 4, 15])
@pytest.mark.parametrize("oldest_first", [False, True])
def test_window_holds_the_last_images_in_order(batch, oldest_first):
    imgs = images(2 * batch + 3, 9, 5, batch)
    states = ol.oracle_circular(batch, oldest_first, imgs, 10.0)
    for i in range(len(imgs)):
        for z in range(batch):
            age = batch - 1 - z if oldest_first else z
            if age <= i:
                want = imgs[i - age].astype(np.float32).transpose(2, 0, 1)
                assert np.array_equal(states[i, z], want), (i, z)
            else:
                assert np.isnan(states[i, z]).all()      # copied from a hidden plane nothing was stored in yet


def test_circular_plane_index_known_answers():
    lib = ol.oracle()
    ol.OracleWindow(2, False, 1, 1, 0.0)      # sets the ctypes signatures
    assert [lib.fklo_circular_plane(0, 4, z, 3) for z in range(4)] == [3, 0, 1, 2]
    assert [lib.fklo_circular_plane(1, 4, z, 1) for z in range(4)] == [1, 0, 3, 2]
    assert [lib.fklo_window_sequence(0, 4, z) for z in range(4)] == [0, 1, 1, 1]
    assert [lib.fklo_window_sequence(1, 4, z) for z in range(4)] == [1, 1, 1, 0]


@needs_ref
@pytest.mark.parametrize("batch", [2, 3, 4, 15])
@pytest.mark.parametrize("oldest_first", [False, True])
def test_window_matches_reference_backend(batch, oldest_first):
    imgs = images(batch + 4, 11, 6, 40 + batch)
    a = ol.oracle_circular(batch, oldest_first, imgs, 10.0)
    b = ol.ref_circular(batch, oldest_first, imgs, 10.0)
    defined = ~np.isnan(a)
    assert defined.any() and np.array_equal(a[defined], b[defined])
    assert defined[batch - 1:].all()       # from the BATCH-th update on, every plane is defined


@needs_ref
def test_divergent_launches_match_reference_backend():
    r = np.random.default_rng(5)
    a = r.integers(0, 2**32, (32, 32), dtype=np.uint32)
    b = r.integers(0, 2**32, (32, 32), dtype=np.uint32)
    got = ol.ref_divergent_two(a, b, 3)
    assert np.array_equal(got[0], a + np.uint32(3)) and np.array_equal(got[1], b)     # uint32 addition wraps
    t = (r.random((4, 12, 20, 3), dtype=np.float32) * 10 - 5).astype(np.float32)
    img = r.integers(0, 256, (7, 9, 3), dtype=np.uint8)
    assert ol.oracle_divergent_mixed(t, 1.5, img).tobytes() == ol.ref_divergent_mixed(t, 1.5, img).tobytes()
