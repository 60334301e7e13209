"""Writes the committed fixtures in this directory.  Run from the repo root: python tests/golden/make_golden.py

The reference ships no golden vectors (its tests compare live against jax.lax.ragged_dot_general on a GPU), and
neither it nor JAX can be imported here, so these vectors come from the numpy oracle after it has been pinned by
tests/test_oracle.py.  They freeze (a) the benchmark configurations' seeded group sizes and (b) scheduling maps for
a few (group_sizes, m, chunk_m) triples, so a later change to either the generators or the map shows up as a diff.
"""

import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from gpu_ragged_dot_amd import workloads  # noqa: E402
from oracle import ragged_dot_oracle as oracle  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    sizes = {name: workloads.group_sizes(name).tolist() for name in workloads.WORKLOADS}
    with open(os.path.join(HERE, "workload_group_sizes.json"), "w") as f:
        json.dump(sizes, f)

    maps = []
    triples = [
        ([3, 0, 5], 8, 2),
        ([4, 1], 10, 512),
        (sizes["tiny"], 512, 512),
        (sizes["tiny"], 512, 64),
        (sizes["mixtral_fwd"], 16384, 512),
        (sizes["mixtral_fwd"], 16384, 256),
        (sizes["deepseek_fwd_bwd"], 32768, 512),
        (sizes["deepseek_fwd_bwd"], 32768, 64),
        (sizes["decode"], 64, 512),
        (oracle.generate_group_sizes(0, 16, 120).tolist(), 171, 8),
        ([0, 0, 0, 0], 64, 8),
    ]
    for gs, m, c in triples:
        md = oracle.make_gmm_group_metadata(np.array(gs, np.int32), m, c)
        maps.append(
            dict(group_sizes=list(map(int, gs)), m=m, chunk_m=c, group_offsets=md.group_offsets.tolist(),
                 row_it2group=md.row_it2group.tolist(), row_it2it_in_group=md.row_it2it_in_group.tolist(),
                 total_row_its=int(md.total_row_its))
        )
    with open(os.path.join(HERE, "sched_map_golden.json"), "w") as f:
        json.dump(maps, f)


if __name__ == "__main__":
    main()
