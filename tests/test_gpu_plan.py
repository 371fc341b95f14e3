"""GPU: the plan (stable CSR / CSC build + schedule) is bit-exact with the numpy
oracle (stable argsort), through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import graph_prep as gp
from torchgt_amd import _lib, workloads
from torchgt_amd.plan import GraphPlan

pytestmark = pytest.mark.gpu


def _check_plan(ei_np, N, cuda):
    print(f"plan case N={N} E={ei_np.shape[1]}", flush=True)
    ei = torch.from_numpy(np.ascontiguousarray(ei_np)).to(cuda)
    plan = GraphPlan(ei, N)
    for by, ids in (("dst", (_lib.PLAN_ROWPTR_DST, _lib.PLAN_COL_DST, _lib.PLAN_EID_DST, _lib.PLAN_ITEMS_DST)),
                    ("src", (_lib.PLAN_ROWPTR_SRC, _lib.PLAN_COL_SRC, _lib.PLAN_EID_SRC, _lib.PLAN_ITEMS_SRC))):
        rowptr, col, eid = gp.build_csr(ei_np, N, by)
        np.testing.assert_array_equal(plan.export(ids[0]), rowptr)
        np.testing.assert_array_equal(plan.export(ids[2]), eid)
        np.testing.assert_array_equal(plan.export(ids[1]), col)
        # schedule: items tile every row exactly once, in order, segments <= limit
        items = plan.export(ids[3]).reshape(-1, 4)
        seg = plan.info()["segment_len"]
        assert np.all(items[:, 2] <= seg) and np.all(items[:, 2] >= 0)
        order = np.lexsort((items[:, 1], items[:, 0]))
        it = items[order]
        covered = np.zeros(N, dtype=np.int64)
        np.add.at(covered, it[:, 0], it[:, 2])
        np.testing.assert_array_equal(covered, np.diff(rowptr))
        first = np.ones(len(it), dtype=bool)
        first[1:] = it[1:, 0] != it[:-1, 0]
        np.testing.assert_array_equal(it[first, 1], rowptr[it[first, 0]])
        cont = ~first
        np.testing.assert_array_equal(it[cont, 1], it[np.nonzero(cont)[0] - 1, 1] + it[np.nonzero(cont)[0] - 1, 2])
        split = np.diff(rowptr) > seg
        assert np.all((it[:, 3] >= 0) == split[it[:, 0]])
        parts = np.sort(it[it[:, 3] >= 0, 3])
        np.testing.assert_array_equal(parts, np.arange(len(parts)))
    plan.close()
    return True


def test_plan_small_random(cuda):
    rng = np.random.default_rng(0)
    for N, E in ((1, 0), (1, 3), (7, 0), (5, 1), (100, 1000), (300, 5000), (257, 4097), (70000, 200000)):
        ei = rng.integers(0, N, (2, E))
        _check_plan(ei, N, cuda)


def test_plan_hub_and_duplicates(cuda):
    rng = np.random.default_rng(1)
    N = 3000
    ei = rng.integers(0, N, (2, 20000))
    ei[1, :9000] = 17                      # hub destination with 9000 in-edges (split row)
    ei[0, 9000:15000] = 5                  # hub source
    ei[:, 15000:16000] = ei[:, 16000:17000]   # duplicate edges
    _check_plan(ei, N, cuda)


def test_plan_config1_and_config2_graphs(cuda):
    e1, n1 = workloads.barabasi_albert()
    assert (n1, e1.shape[1]) == (4097, 45024)
    _check_plan(e1, n1, cuda)
    e2, n2 = workloads.power_law_graph()
    assert n2 == 64001 and abs(e2.shape[1] - 530000) < 0.02 * 530000
    _check_plan(e2, n2, cuda)


def test_plan_three_radix_passes(cuda):
    # N > 65536 needs three 8-bit passes; ids spread over the whole range
    rng = np.random.default_rng(2)
    N = 300000
    ei = rng.integers(0, N, (2, 400000))
    _check_plan(ei, N, cuda)


def test_plan_rejects_out_of_range(cuda):
    ei = torch.tensor([[0, 1, 9], [1, 2, 0]], device=cuda)
    with pytest.raises(_lib.TorchGTHipError) as exc:
        GraphPlan(ei, 5)
    assert exc.value.code == _lib.ERR_INDEX_RANGE
    ei = torch.tensor([[0, -1], [1, 2]], device=cuda)
    with pytest.raises(_lib.TorchGTHipError):
        GraphPlan(ei, 5)


def test_plan_is_reproducible(cuda):
    rng = np.random.default_rng(3)
    ei = torch.from_numpy(rng.integers(0, 5000, (2, 60000))).to(cuda)
    a, b = GraphPlan(ei, 5000), GraphPlan(ei, 5000)
    for which in range(8):
        np.testing.assert_array_equal(a.export(which), b.export(which))
