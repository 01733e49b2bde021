"""GPU results against the committed golden fixtures (tests/golden/replay_small.npz)."""
import os

import numpy as np
import pytest
import torch

from graph_sampling_amd import capi
from tests.util import to_dev

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "replay_small.npz"))


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
@pytest.mark.parametrize("name,algo", [("floyd", capi.ALGO_AUTO), ("reservoir", capi.ALGO_RESERVOIR)])
def test_uniform_sampling_golden(dev, idt, name, algo):
    sp, si, sel, _ = capi.sample_uniform(to_dev(GOLD["indptr"], dev), to_dev(GOLD["indices"], dev, idt),
                                         to_dev(GOLD["cols"], dev, idt), 5, False,
                                         replay=to_dev(GOLD[name + "_draws"], dev),
                                         replay_ptr=to_dev(GOLD[name + "_replay_ptr"], dev), algo=algo)
    n = int(sp[-1].item())
    assert np.array_equal(sp.cpu().numpy(), GOLD[name + "_sub_indptr"])
    assert np.array_equal(si[:n].cpu().numpy().astype(np.int64), GOLD[name + "_sub_indices"])
    assert np.array_equal(sel[:n].cpu().numpy(), GOLD[name + "_select_index"])


def test_weighted_walk_relabel_golden(dev):
    indptr, indices = to_dev(GOLD["indptr"], dev), to_dev(GOLD["indices"], dev)
    sp, si, sel, _ = capi.sample_weighted(indptr, indices, to_dev(GOLD["probs"], dev),
                                          to_dev(GOLD["cols"], dev), 4,
                                          replay=to_dev(GOLD["weighted_draws"], dev),
                                          replay_ptr=to_dev(GOLD["weighted_replay_ptr"], dev))
    n = int(sp[-1].item())
    assert np.array_equal(sel[:n].cpu().numpy(), GOLD["weighted_select_index"])
    assert np.array_equal(si[:n].cpu().numpy(), GOLD["weighted_sub_indices"])
    tr = capi.random_walk(indptr, indices, to_dev(GOLD["walk_seeds"], dev), 6,
                          replay=to_dev(GOLD["walk_draws"], dev))
    assert np.array_equal(tr.cpu().numpy(), GOLD["walk_trace"])
    rows = to_dev(GOLD["floyd_sub_indices"], dev)
    fr, num, outs = capi.unique_relabel([to_dev(GOLD["cols"], dev), rows], [rows])
    assert np.array_equal(fr[:int(num.item())].cpu().numpy(), GOLD["relabel_frontier"])
    assert np.array_equal(outs[0].cpu().numpy(), GOLD["relabel_rows"])
