"""This repository's own TransformDPP<ParArch::CPU> executor (include/fused_kernel/core/execution_model/executors.h): the
lowered chain run element by element on the host with the device operations' element bodies.

oracle/libfkl_hostexec.so is the reference-backend harness (oracle/ref_chains.cpp: every chain spelled with the public
API) compiled against THIS repository's headers, so the ref_* wrappers of oracle_lib can be pointed at it.  The
checks are the ones that hold the oracle against the reference's CPU backend, run again with the wrappers redirected:
same chains, same inputs, results bit for bit those of the oracle (which the reference backend pins).  No GPU involved.
"""
import numpy as np
import pytest

import oracle_lib as ol
import test_oracle as t_core
import test_oracle_border as t_border
import test_oracle_color as t_color
import test_oracle_depth_and_transposed as t_depth
import test_oracle_window as t_window
import test_oracle_pointwise as t_pointwise

pytestmark = pytest.mark.skipif(not ol.have_hostexec(), reason="oracle/libfkl_hostexec.so not built (make -C oracle hostexec)")


def on_host_executor(fn, *args):
    with ol.host_executor():
        fn(*args)


def test_benchmark_chains_random_cases():
    # configurations 1, 3, 5 and the integer-only chain on random shapes
    on_host_executor(t_core.test_oracle_equals_live_reference_on_random_cases)


def test_pointwise_and_batched_chains():
    import workloads as wl
    with ol.host_executor():
        c = wl.config2(width=96, height=64)
        for n in (1, 2, 3, 10):
            for tf in (0, 1):
                assert ol.oracle_add_mul_chain(c["src"], n, c["add"], c["mul"]).tobytes() == \
                    ol.ref_add_mul_chain(c["src"], n, c["add"], c["mul"], tf=tf).tobytes(), (n, tf)
        c = wl.config4(batch=4, width=96, height=64)
        want = ol.oracle_batch_muladd_sat(c["srcs"], c["mul"], c["add"])
        got = ol.ref_batch_muladd_sat(c["srcs"], c["mul"], c["add"])
        assert all(np.array_equal(a, b) for a, b in zip(want, got))


def test_default_planes():
    on_host_executor(t_core.test_default_planes_match_reference_backend)


def test_warp():
    on_host_executor(t_core.test_warp_matches_reference_backend)


def test_deinterlace():
    on_host_executor(t_core.test_deinterlace_matches_reference_backend)


@pytest.mark.parametrize("pf,cr,cp", t_color.Y2R)
def test_yuv_to_rgb(pf, cr, cp):
    on_host_executor(t_color.test_yuv_to_rgb_matches_reference_backend, pf, cr, cp)


@pytest.mark.parametrize("pf,cr,cp", t_color.R2Y)
def test_rgb_to_yuv(pf, cr, cp):
    on_host_executor(t_color.test_rgb_to_yuv_matches_reference_backend, pf, cr, cp)


@pytest.mark.parametrize("pf", [ol.PF_NV21, ol.PF_UYVY, ol.PF_P010])
def test_yuv_resize(pf):
    on_host_executor(t_color.test_yuv_resize_matches_reference_backend, pf)


@pytest.mark.parametrize("cd,cr,cp", t_color.DEPTHS)
def test_depth_conversions(cd, cr, cp):
    on_host_executor(t_color.test_depth_conversions_match_reference_backend, cd, cr, cp)


@pytest.mark.parametrize("which", sorted(ol.COLOR_CODES))
def test_color_codes(which):
    on_host_executor(t_color.test_color_codes_match_reference_backend, which)


@pytest.mark.parametrize("which", [0, 1])
def test_normalize(which):
    on_host_executor(t_color.test_normalize_matches_reference_backend, which)


@pytest.mark.parametrize("bt", sorted(t_border.NUMPY_MODE))
def test_padding(bt):
    on_host_executor(t_border.test_padding_matches_reference_backend, bt)


@pytest.mark.parametrize("batch", [2, 3, 4, 15])
@pytest.mark.parametrize("oldest_first", [False, True])
def test_circular_window(batch, oldest_first):
    on_host_executor(t_window.test_window_matches_reference_backend, batch, oldest_first)


def test_divergent_launches():
    on_host_executor(t_window.test_divergent_launches_match_reference_backend)


@pytest.mark.parametrize("which", sorted(ol.DEPTH_OPS))
def test_depth_operations(which):
    on_host_executor(t_depth.test_depth_operations_match_reference_backend, which)


def test_transposed_tensor():
    on_host_executor(t_depth.test_transposed_tensor_matches_reference_backend, 3, 10, 6)
    on_host_executor(t_depth.test_transposed_tensor_matches_reference_backend, 4, 33, 5)


@pytest.mark.parametrize("batch", [2, 5])
@pytest.mark.parametrize("oldest_first", [False, True])
def test_transposed_window(batch, oldest_first):
    on_host_executor(t_depth.test_transposed_window_matches_reference_backend, batch, oldest_first)


@pytest.mark.parametrize("which", t_pointwise.ALL)
def test_per_channel_operations(which):
    # Abs ... MxVFloat3 (tests/cases/pointwise_chains.h): this repository's CPU executor against the numpy restatement
    on_host_executor(t_pointwise.test_oracle_equals_the_reference_backend, which)


def test_resize_geometry_of_every_aspect_ratio_mode():
    # Resize<INTER_LINEAR, AR>::build of this repository's headers (PRESERVE_AR, PRESERVE_AR_RN_EVEN, PRESERVE_AR_LEFT)
    on_host_executor(t_core.test_aspect_ratio_modes_match_the_live_reference_on_random_sizes)


@pytest.mark.parametrize("which", sorted(ol.SPLIT_WRITE_CASES))
def test_split_write(which):
    on_host_executor(t_pointwise.test_split_write_equals_the_reference_backend, which)


@pytest.mark.parametrize("which", sorted(t_pointwise.po.DUAL_CASES))
def test_two_image_chains(which):
    # DualSourceRead and the two-input forms of Add ... BwOr on this repository's CPU executor
    on_host_executor(t_pointwise.test_two_image_chains_equal_the_reference_backend, which)


def test_sweeps_of_random_cases():
    # the seeded sweeps that hold the oracle to the reference backend (and the GPU to the oracle), on this executor
    import test_oracle_random_batches as t_random
    on_host_executor(t_random.test_oracle_equals_the_reference_backend_on_the_sweep)
    on_host_executor(t_random.test_oracle_equals_the_reference_backend_on_the_reader_sweep)
    on_host_executor(t_random.test_oracle_equals_the_reference_backend_on_the_chain_sweep)
    on_host_executor(t_color.test_oracle_equals_the_reference_backend_on_the_sweep_of_random_sizes)
    on_host_executor(t_pointwise.test_oracle_equals_the_reference_backend_on_the_sweep_of_random_sizes)
