"""Writes the committed fixtures in this directory.  Run from the repo root: python tests/golden/make_golden.py

The reference ships no golden vectors (its tests compare live against jax.lax.ragged_dot_general on a GPU), and
neither it nor JAX can be imported here, so these vectors come from the numpy oracle after it has been pinned by
tests/test_oracle.py.  They freeze (a) the benchmark configurations' seeded group sizes and (b) scheduling maps for
a few (group_sizes, m, chunk_m) triples, so a later change to either the generators or the map shows up as a diff.
moe_route_golden.json freezes the routing (stable counting sort) of a few small expert-id tables, from
oracle/moe_glue_oracle.py after tests/test_moe_glue.py has pinned it against a brute-force loop.
"""

import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from gpu_ragged_dot_amd import workloads  # noqa: E402
from oracle import moe_glue_oracle  # noqa: E402
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

    routes = []
    rng = np.random.default_rng(7)
    tables = [
        (np.array([[2, 0], [1, 2], [0, 0], [3, 1]]), 4),
        (np.array([[5, -1, 2], [7, 2, 5], [9, 5, 0]]), 8),              # -1, 9: dropped
        (rng.integers(0, 6, size=(37, 2)), 6),
        (np.argsort(rng.standard_normal((8, 128)), axis=1)[:, :8], 128),  # 8 tokens x top-8 of 128, as the decode config
    ]
    for ids, g in tables:
        gs, ros, sor = moe_glue_oracle.route(ids.astype(np.int32), g)
        routes.append(dict(expert_ids=ids.astype(int).tolist(), g=g, group_sizes=gs.tolist(), row_of_slot=ros.tolist(),
                           slot_of_row=sor.tolist()))
    with open(os.path.join(HERE, "moe_route_golden.json"), "w") as f:
        json.dump(routes, f)


if __name__ == "__main__":
    main()
