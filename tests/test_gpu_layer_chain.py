"""GPU parity: a whole minibatch queued with no host read (gs_layer_sample + gs_layer_relabel
per layer, sizes handed from layer to layer on the device) against the CPU oracle, which runs
the layers one by one: sample_uniform on the frontier, then relabel of (frontier, sampled ids)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from graph_sampling_amd import capi
from tests.util import rmat_csc_np, to_dev

pytestmark = pytest.mark.gpu


def _oracle_layers(indptr, indices, seeds, fanouts, replace, seed):
    out = []
    cols = seeds
    for l, k in enumerate(fanouts):
        sp, _, si, _ = O.sample_uniform(indptr, indices, cols, k, replace, seed=seed + l,
                                        with_coo=False)
        frontier, (renamed,) = O.relabel([cols, si], [si])
        out.append((cols.size, sp, si, frontier, renamed))
        cols = frontier
    return out


def _check_layers(layers, want):
    for b, (S, sp, si, frontier, renamed) in zip(layers, want):
        E, U = (int(v) for v in b.counts.cpu())
        assert E == si.size and U == frontier.size, (E, si.size, U, frontier.size)
        assert np.array_equal(b.sub_indptr[:S + 1].cpu().numpy(), sp)
        assert np.array_equal(b.offsets_copy[:S + 1].cpu().numpy(), sp)
        assert np.array_equal(b.sub_indices[:E].cpu().numpy().astype(np.int64), si)
        assert np.array_equal(b.frontier[:U].cpu().numpy().astype(np.int64), frontier)
        assert np.array_equal(b.out_ids[:E].cpu().numpy().astype(np.int64), renamed)


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
@pytest.mark.parametrize("num_seeds,fanouts,replace", [
    (1024, (15, 10, 5), False),   # the benchmark's minibatch
    (512, (10, 5), False),
    (1, (3,), False),
    (0, (4, 4), False),
    (300, (4, 4, 4, 4), True),
    (3000, (32,), False),
    (257, (1, 1, 1), False),
    (1024, (16, 2), False),
    (1000, (16,), True),
])
def test_chain_matches_the_oracle_layer_by_layer(dev, idt, num_seeds, fanouts, replace):
    n = 1 << 14
    indptr, indices = rmat_csc_np(n, 1 << 19, seed=21)
    seeds = np.random.default_rng(num_seeds).permutation(n)[:num_seeds].astype(np.int64)
    t_ptr, t_idx, t_seeds = to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(seeds, dev, idt)
    bound = num_seeds
    for k in fanouts:
        bound *= 1 + k
    tables = [capi.RelabelTable(bound, torch.int32, dev) for _ in range(2)]
    box = capi.Mailbox()
    # several minibatches in a row on the same two tables: every one leaves them empty
    for seed in (40, 50):
        layers, ticket = capi.sample_layers(t_ptr, t_idx, t_seeds, fanouts, replace, seed=seed,
                                            mailbox=box, tables=tables)
        U_last = box.wait(ticket, dev)
        want = _oracle_layers(indptr, indices, seeds, fanouts, replace, seed)
        assert U_last == want[-1][3].size
        _check_layers(layers, want)
    torch.cuda.synchronize()
    for t in tables:
        assert bool((t.buf.view(torch.int64) == -1).all())


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
@pytest.mark.parametrize("with_edge_ids", [False, True])
@pytest.mark.parametrize("num_seeds,fanouts,replace", [
    (1024, (15, 10, 5), False),
    (700, (3, 40), True),      # fanout 40 with replacement: further rounds of a row's lanes
    (0, (4, 4), False),
    (257, (1, 6), False),
])
def test_chain_carries_the_edge_data_of_its_samples(dev, idt, with_edge_ids, num_seeds, fanouts,
                                                    replace):
    """With edge data the sampler leaves, per layer, the position of every sample in the graph's
    indices and data[e_ids[position]] (the gathers of the reference's src/graph.cc:544-557), at
    the same place as the sample's renamed id."""
    n = 1 << 13
    indptr, indices = rmat_csc_np(n, 1 << 18, seed=23)
    rng = np.random.default_rng(77)
    data = (1.0 - rng.random(indices.size)).astype(np.float32)
    e_ids = rng.permutation(indices.size).astype(np.int64) if with_edge_ids else None
    seeds = rng.permutation(n)[:num_seeds].astype(np.int64)
    layers, _ = capi.sample_layers(
        to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(seeds, dev, idt), fanouts, replace,
        seed=61, edge_data=to_dev(data, dev), edge_ids=None if e_ids is None else to_dev(e_ids, dev))
    want = _oracle_layers(indptr, indices, seeds, fanouts, replace, 61)
    _check_layers(layers, want)
    cols = seeds
    for l, (b, k) in enumerate(zip(layers, fanouts)):
        _, _, si, sel = O.sample_uniform(indptr, indices, cols, k, replace, seed=61 + l,
                                         with_coo=False)
        E = int(b.counts[0])
        assert E == sel.size
        assert np.array_equal(b.select_index[:E].cpu().numpy(), sel)
        assert np.array_equal(indices[sel], si)
        picked = data[sel] if e_ids is None else data[e_ids[sel]]
        assert np.array_equal(b.data[:E].cpu().numpy(), picked)
        cols = want[l][3]


@pytest.mark.parametrize("num_seeds", [5000, 1000])
def test_chain_with_repeated_seeds_and_hub_columns(dev, num_seeds):
    """Seeds that repeat (the frontier is shorter than the seed list), seeds that the sampled
    ids name again, and the graph's largest columns among them."""
    n = 1 << 13
    indptr, indices = rmat_csc_np(n, 1 << 18, seed=3)
    rng = np.random.default_rng(8)
    seeds = rng.integers(0, n, size=num_seeds).astype(np.int64)
    seeds[:16] = np.argsort(np.diff(indptr))[-16:]
    seeds[100:200] = seeds[0]
    seeds[300:400] = indices[indptr[seeds[0]]:indptr[seeds[0]] + 100]  # neighbours of a hub
    d = (to_dev(indptr, dev), to_dev(indices, dev, torch.int32), to_dev(seeds, dev, torch.int32))
    layers, _ = capi.sample_layers(*d, (6, 3), False, seed=9)
    _check_layers(layers, _oracle_layers(indptr, indices, seeds, (6, 3), False, 9))


def test_chain_with_seeds_that_are_no_columns(dev):
    """Seeds beyond the graph's last column are empty columns in every layer they reach.  (-1,
    the reference's mark of an empty table slot, unique_reindex.cu:52-54, is no id to relabel.)"""
    n = 1 << 12
    indptr, indices = rmat_csc_np(n, 1 << 16, seed=5)
    seeds = np.array([5, 1 << 20, n, 17, n + 100, 900, 5], dtype=np.int64)
    d = (to_dev(indptr, dev), to_dev(indices, dev, torch.int32), to_dev(seeds, dev, torch.int32))
    layers, _ = capi.sample_layers(*d, (3, 3), False, seed=2)
    want = _oracle_layers(indptr, indices, seeds, (3, 3), False, 2)
    for b, (S, sp, si, frontier, renamed) in zip(layers, want):
        E, U = (int(v) for v in b.counts.cpu())
        assert (E, U) == (si.size, frontier.size)
        assert np.array_equal(b.sub_indptr[:S + 1].cpu().numpy(), sp)
        assert np.array_equal(b.sub_indices[:E].cpu().numpy().astype(np.int64), si)
        assert np.array_equal(b.frontier[:U].cpu().numpy().astype(np.int32), frontier.astype(np.int32))
        assert np.array_equal(b.out_ids[:E].cpu().numpy().astype(np.int64), renamed)


@pytest.mark.parametrize("case", range(24))
def test_chain_on_seeded_random_shapes(dev, case):
    """Graph size, skew, seed count (with repeats), depth, fanouts and the replace flag drawn
    from a seeded generator: every case against the oracle, layer by layer."""
    rng = np.random.default_rng(1000 + case)
    n = int(rng.choice([64, 1 << 10, 1 << 13, 1 << 15]))
    e = int(n * rng.choice([1, 4, 30]))
    indptr, indices = rmat_csc_np(n, e, seed=case)
    num_seeds = int(rng.choice([1, 7, 100, 1500, 4000]))
    seeds = rng.integers(0, n, size=num_seeds).astype(np.int64)
    depth = int(rng.integers(1, 4))
    replace = bool(rng.integers(0, 2))
    fanouts = tuple(int(rng.choice([2, 3, 5, 8, 12, 20, 32])) for _ in range(depth))
    bound = num_seeds
    for k in fanouts:
        bound *= 1 + k
    if bound > 1 << 22:
        fanouts = fanouts[:1]
    idt = torch.int32 if case % 2 == 0 else torch.int64
    d = (to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(seeds, dev, idt))
    layers, _ = capi.sample_layers(*d, fanouts, replace, seed=case)
    _check_layers(layers, _oracle_layers(indptr, indices, seeds, fanouts, replace, case))


def test_chain_reports_an_id_beyond_32_bits(dev):
    """64-bit ids ride on one-word slots; one that does not fit is reported as -2, not truncated."""
    indptr = np.array([0, 2, 4, 6], dtype=np.int64)
    indices = np.array([1, 2, 0, (1 << 33) + 5, 0, 1], dtype=np.int64)
    seeds = np.array([0, 1, 2], dtype=np.int64)
    d = (to_dev(indptr, dev), to_dev(indices, dev), to_dev(seeds, dev))
    box = capi.Mailbox()
    layers, ticket = capi.sample_layers(*d, (2,), False, seed=1, mailbox=box)
    assert box.wait(ticket, dev) == -2
    assert int(layers[0].counts[1]) == -2
    torch.cuda.synchronize()
    capi._fused_state.clear()  # the error word of the look-back state is sticky
