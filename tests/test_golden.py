"""Committed fixtures (tests/golden): the oracle on CPU, and the HIP scheduling-map kernel on the GPU, must both
reproduce them bit for bit."""

import json
import os

import numpy as np
import pytest

from gpu_ragged_dot_amd import workloads
from oracle import ragged_dot_oracle as oracle

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
MAPS = json.load(open(os.path.join(HERE, "sched_map_golden.json")))
SIZES = json.load(open(os.path.join(HERE, "workload_group_sizes.json")))


def test_workload_group_sizes_match_fixture_and_published_summary():
    for name, want in SIZES.items():
        assert workloads.group_sizes(name).tolist() == want
    assert SIZES["tiny"] == [116, 133, 132, 131]
    assert SIZES["mixtral_fwd"] == [2012, 2069, 2038, 2100, 2032, 2052, 2039, 2042]
    ds = np.array(SIZES["deepseek_fwd_bwd"])
    assert ds.sum() == 32768 and (ds == 0).sum() == 26 and ds.max() == 7099 and np.median(ds[ds > 0]) == 34
    assert sorted(ds)[-5:] == [1219, 1512, 2129, 3266, 7099]
    dec = np.array(SIZES["decode"])
    assert dec.sum() == 64 and (dec > 0).sum() == 53 and dec.max() == 3


@pytest.mark.parametrize("i", range(len(MAPS)))
def test_oracle_reproduces_map_fixture(i):
    fx = MAPS[i]
    md = oracle.make_gmm_group_metadata(np.array(fx["group_sizes"], np.int32), fx["m"], fx["chunk_m"])
    assert md.group_offsets.tolist() == fx["group_offsets"]
    assert md.row_it2group.tolist() == fx["row_it2group"]
    assert md.row_it2it_in_group.tolist() == fx["row_it2it_in_group"]
    assert int(md.total_row_its) == fx["total_row_its"]


@pytest.mark.gpu
@pytest.mark.parametrize("i", range(len(MAPS)))
def test_hip_map_reproduces_fixture(i):
    import torch

    import gpu_ragged_dot_amd as rd

    fx = MAPS[i]
    print("golden map", i, "g", len(fx["group_sizes"]), "m", fx["m"], "chunk", fx["chunk_m"], flush=True)
    offs, t2g, t2it, total = rd.make_group_metadata(torch.tensor(fx["group_sizes"], dtype=torch.int32), fx["m"], fx["chunk_m"])
    assert offs.cpu().tolist() == fx["group_offsets"]
    assert t2g.cpu().tolist() == fx["row_it2group"]
    assert t2it.cpu().tolist() == fx["row_it2it_in_group"]
    assert int(total.item()) == fx["total_row_its"]
