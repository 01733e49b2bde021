"""GPU parity: unique / relabel through the C ABI vs the CPU oracle and closed forms."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from graph_sampling_amd import capi
from tests.util import to_dev

pytestmark = pytest.mark.gpu


def _closed_form_unique(x):
    u, first = np.unique(x, return_index=True)
    return u[np.argsort(first, kind="stable")]


def _run(mapping, queries, dev, idt):
    dm = [to_dev(m, dev, idt) for m in mapping]
    # a query that IS a mapping tensor must alias it (the slot-gather path)
    dq = []
    for q in queries:
        hit = [i for i, m in enumerate(mapping) if m is q]
        dq.append(dm[hit[0]] if hit else to_dev(q, dev, idt))
    frontier, num, outs = capi.unique_relabel(dm, dq)
    n = int(num.item())
    return frontier[:n].cpu().numpy().astype(np.int64), [o.cpu().numpy().astype(np.int64) for o in outs]


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
@pytest.mark.parametrize("n", [0, 1, 5, 2048, 2049, 100000])
def test_unique_first_occurrence(dev, idt, n):
    rng = np.random.default_rng(n)
    x = rng.integers(0, max(1, n // 3) + 5, size=n).astype(np.int64) * 7919 % 100003
    frontier, _ = _run([x], [], dev, idt)
    assert np.array_equal(frontier, _closed_form_unique(x))
    assert np.array_equal(frontier, O.unique(x))


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
def test_relabel_seeds_first(dev, idt):
    rng = np.random.default_rng(0)
    seeds = rng.permutation(50000)[:1024].astype(np.int64)
    rows = rng.integers(0, 50000, size=15000).astype(np.int64)
    other = rng.integers(0, 60000, size=777).astype(np.int64)  # holds ids absent from the mapping
    frontier, outs = _run([seeds, rows], [rows, other, seeds], dev, idt)
    want_frontier, want = O.relabel([seeds, rows], [rows, other, seeds])
    assert np.array_equal(frontier, want_frontier)
    for g, w in zip(outs, want):
        assert np.array_equal(g, w)
    assert np.array_equal(frontier[:1024], seeds)          # seeds occupy the head of the frontier
    assert np.array_equal(frontier[outs[0]], rows)         # frontier[relabelled] == original
    assert (outs[1] == -1).any() and np.array_equal(outs[2], np.arange(1024))


def test_relabel_reference_vector(dev):
    # reference tests/test_relabel.cc:7-26: slicing cols 1..3 of the 20x5 graph with relabel
    rows = np.arange(5, 20, dtype=np.int64)
    frontier, outs = _run([rows], [rows], dev, torch.int64)
    assert np.array_equal(frontier, rows)
    assert np.array_equal(outs[0], np.arange(15))


def test_unique_large_consecutive_and_clustered(dev):
    # consecutive ids (the case that clusters under an identity hash) plus heavy duplication
    x = np.concatenate([np.arange(300000), np.arange(300000)[::-1], np.full(1000, 42)]).astype(np.int64)
    frontier, outs = _run([x], [x], dev, torch.int64)
    assert np.array_equal(frontier, np.arange(300000))
    assert np.array_equal(frontier[outs[0]], x)


def test_four_mapping_spans(dev):
    rng = np.random.default_rng(4)
    spans = [rng.integers(0, 5000, size=s).astype(np.int64) for s in (10, 0, 3000, 2049)]
    frontier, outs = _run(spans, [spans[3], spans[0]], dev, torch.int64)
    want_frontier, want = O.relabel(spans, [spans[3], spans[0]])
    assert np.array_equal(frontier, want_frontier)
    for g, w in zip(outs, want):
        assert np.array_equal(g, w)


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
@pytest.mark.parametrize("n", [512 * 2048 - 1, 512 * 2048, 512 * 2048 + 1, 3_000_000])
def test_relabel_million_items(dev, idt, n):
    """Around 2^20 items (512 compaction tiles: several look-back bursts) and 3 M, with an aliased
    and a plain query, heavy and light repetition."""
    rng = np.random.default_rng(n)
    seeds = rng.permutation(5_000_000)[:1000].astype(np.int64)
    rows = np.concatenate([rng.integers(0, 2000, size=n // 2),            # hubs: heavy repetition
                           rng.integers(0, 5_000_000, size=n - 1000 - n // 2)]).astype(np.int64)
    rng.shuffle(rows)
    probe = rng.integers(0, 5_000_100, size=5000).astype(np.int64)        # some absent ids
    frontier, (rel_rows, rel_probe) = _run([seeds, rows], [rows, probe], dev, idt)
    want_frontier, (want_rows, want_probe) = O.relabel([seeds, rows], [rows, probe])
    assert np.array_equal(frontier, want_frontier)
    assert np.array_equal(rel_rows, want_rows)
    assert np.array_equal(rel_probe, want_probe)
    assert (want_probe == -1).any()


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
def test_relabel_every_item_the_same_key(dev, idt):
    """All tiles fight for one slot; one first occurrence in tile 0, every other tile has none."""
    x = np.full(300_000, 12345, dtype=np.int64)
    y = np.arange(300_000, dtype=np.int64) % 3
    frontier, (rx, ry) = _run([x, y], [x, y], dev, idt)
    assert np.array_equal(frontier, np.array([12345, 0, 1, 2]))
    assert (rx == 0).all() and np.array_equal(ry, y + 1)


def _batches(rng, B, n_nodes, max_seeds, max_ids, empty_every=0):
    seeds, ids, sp, ip = [], [], [0], [0]
    for b in range(B):
        ns = 0 if empty_every and b % empty_every == 1 else int(rng.integers(1, max_seeds + 1))
        ni = 0 if empty_every and b % empty_every == 2 else int(rng.integers(0, max_ids + 1))
        seeds.append(rng.permutation(n_nodes)[:ns])
        ids.append(rng.integers(0, n_nodes, size=ni))
        sp.append(sp[-1] + ns)
        ip.append(ip[-1] + ni)
    cat = lambda xs: np.concatenate(xs).astype(np.int64) if xs else np.empty(0, np.int64)  # noqa: E731
    return cat(seeds), np.array(sp, dtype=np.int64), cat(ids), np.array(ip, dtype=np.int64)


@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
@pytest.mark.parametrize("B,max_seeds,max_ids,empty_every", [(1, 50, 400, 0), (7, 30, 300, 3),
                                                               (64, 256, 4000, 0), (300, 8, 40, 5),
                                                               # both sides of the 511 batches whose
                                                               # offsets a workgroup keeps in LDS
                                                               (511, 6, 30, 7), (512, 6, 30, 7),
                                                               (1500, 4, 12, 4)])
def test_batch_csr_relabel_matches_oracle(dev, idt, B, max_seeds, max_ids, empty_every):
    """Every batch is relabelled on its own: the same id in two batches gets two ranks."""
    rng = np.random.default_rng(B)
    seeds, sp, ids, ip = _batches(rng, B, 3000, max_seeds, max_ids, empty_every)
    unique, unique_ptr, out_ids, num = capi.batch_csr_relabel(to_dev(seeds, dev, idt), to_dev(sp, dev),
                                                              to_dev(ids, dev, idt), to_dev(ip, dev))
    w_unique, w_ptr, w_out = O.batch_csr_relabel(seeds, sp, ids, ip)
    U = int(num.item())
    assert U == w_unique.size
    assert np.array_equal(unique_ptr.cpu().numpy(), w_ptr)
    assert np.array_equal(unique[:U].cpu().numpy().astype(np.int64), w_unique)
    assert np.array_equal(out_ids.cpu().numpy().astype(np.int64), w_out)
    # closed form per batch, independent of the oracle's hash table
    for b in range(B):
        x = np.concatenate([seeds[sp[b]:sp[b + 1]], ids[ip[b]:ip[b + 1]]])
        f = _closed_form_unique(x)
        assert np.array_equal(w_unique[w_ptr[b]:w_ptr[b + 1]], f)
        assert np.array_equal(f[w_out[ip[b]:ip[b + 1]]], ids[ip[b]:ip[b + 1]])


def _check_batch_relabel(dev, idt, seeds, sp, ids, ip, narrow, path):
    unique, unique_ptr, out_ids, num = capi.batch_csr_relabel(
        to_dev(seeds, dev, idt), to_dev(sp, dev), to_dev(ids, dev, idt), to_dev(ip, dev),
        narrow=narrow, path=path)
    w_unique, w_ptr, w_out = O.batch_csr_relabel(seeds, sp, ids, ip)
    U = int(num.item())
    assert U == w_unique.size
    assert np.array_equal(unique_ptr.cpu().numpy(), w_ptr)
    assert np.array_equal(unique[:U].cpu().numpy().astype(np.int64), w_unique)
    assert np.array_equal(out_ids.cpu().numpy().astype(np.int64), w_out)


@pytest.mark.parametrize("idt,narrow", [(torch.int32, False), (torch.int64, True)])
@pytest.mark.parametrize("B,max_seeds,max_ids,empty_every", [(1, 50, 400, 0), (7, 30, 300, 3),
                                                               (64, 256, 4000, 0), (300, 8, 40, 5),
                                                               (511, 6, 30, 7), (3, 3000, 50000, 0)])
def test_batch_csr_relabel_through_bins_small(dev, idt, narrow, B, max_seeds, max_ids, empty_every):
    """The binned relabel (hash classes + LDS tables) forced on inputs far below the size it is
    chosen for: same frontiers, offsets and ranks as the oracle, empty batches included."""
    rng = np.random.default_rng(B + 1)
    seeds, sp, ids, ip = _batches(rng, B, 3000, max_seeds, max_ids, empty_every)
    _check_batch_relabel(dev, idt, seeds, sp, ids, ip, narrow, "bins")


@pytest.mark.parametrize("idt,narrow", [(torch.int32, False), (torch.int64, True)])
@pytest.mark.parametrize("shape", ["even", "one_large", "hubs", "single", "all_same"])
def test_batch_csr_relabel_through_bins_at_size(dev, idt, narrow, shape):
    """From 2^19 items on the library takes the bins by itself: batches of equal size, one batch
    that holds nearly everything (thousands of classes) beside tiny and empty ones, ids that
    repeat tens of thousands of times, one batch only, one id only; the last batches empty."""
    rng = np.random.default_rng(len(shape))
    n_nodes = 1 << 21
    if shape == "even":
        sizes = [(1000, 60000)] * 16
    elif shape == "one_large":
        sizes = [(5, 40), (0, 0), (2000, 1_500_000), (1, 0), (0, 7), (300, 9000), (0, 0)]
    elif shape == "hubs":
        sizes = [(500, 200000)] * 4
    elif shape == "single":
        sizes = [(4096, 900000)]
    else:
        sizes = [(1, 300000), (1, 300000)]
    seeds, ids, sp, ip = [], [], [0], [0]
    for ns, ni in sizes:
        seeds.append(rng.permutation(n_nodes)[:ns])
        if shape == "hubs":     # a few ids hold most of the positions
            x = (rng.random(ni) ** 8 * n_nodes).astype(np.int64)
        elif shape == "all_same":
            x = np.full(ni, 77, dtype=np.int64)
        else:
            x = rng.integers(0, n_nodes, size=ni)
        ids.append(x)
        sp.append(sp[-1] + ns)
        ip.append(ip[-1] + ni)
    seeds = np.concatenate(seeds).astype(np.int64)
    ids = np.concatenate(ids).astype(np.int64)
    assert seeds.size + ids.size >= 1 << 19
    _check_batch_relabel(dev, idt, seeds, np.array(sp, dtype=np.int64), ids,
                         np.array(ip, dtype=np.int64), narrow, None)


def test_batch_csr_relabel_bins_report_what_they_cannot_take(dev):
    """An id beyond 32 bits among 64-bit ids promised to be narrow: -2, as on the hash regions.  A
    class with more distinct ids than its LDS table holds: -4 from the C ABI, and the host
    layer's operator repeats the call on hash regions by itself."""
    import graph_sampling_amd as gs
    gs.load_library()
    rng = np.random.default_rng(5)
    seeds = rng.permutation(1 << 20)[:100].astype(np.int64)
    ids = rng.integers(0, 1 << 20, size=(1 << 19) + 5).astype(np.int64)
    ids[1234] = (1 << 35) + 3
    sp, ip = np.array([0, 100], dtype=np.int64), np.array([0, ids.size], dtype=np.int64)
    num = capi.batch_csr_relabel(to_dev(seeds, dev), to_dev(sp, dev), to_dev(ids, dev),
                                 to_dev(ip, dev), narrow=True)[3]
    assert int(num.item()) == -2
    # one batch of 20 M distinct ids: 4096 classes of ~4900 distinct ids each, tables of 4096 slots
    n = 20_000_000
    ids = torch.randperm(n, device=dev, dtype=torch.int64).to(torch.int32)
    seeds = ids[:10].clone()
    t_sp = torch.tensor([0, 10], device=dev)
    t_ip = torch.tensor([0, n], device=dev)
    num = capi.batch_csr_relabel(seeds, t_sp, ids, t_ip)[3]
    assert int(num.item()) == -4
    uni, uni_ptr, rel, _ = torch.ops.gs_ops.BatchCSRRelabel(seeds, t_sp, ids, t_ip)
    # closed form: the seeds are the first ten ids, every other id is new, in order
    assert uni_ptr.cpu().tolist() == [0, n]
    assert torch.equal(uni, ids)
    assert torch.equal(rel, torch.arange(n, device=dev, dtype=torch.int32))


# a few tiles of the compaction, with keys all distinct, in long runs, and in between
@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
@pytest.mark.parametrize("n", [8191, 8192, 8193, 16383, 16384, 16385])
@pytest.mark.parametrize("spread", ["distinct", "few", "mixed"])
def test_relabel_few_tiles_by_key_spread(dev, idt, n, spread):
    rng = np.random.default_rng(n)
    if spread == "distinct":
        rows = (rng.permutation(1 << 20)[:n - 100].astype(np.int64) * 7 + 3)
    elif spread == "few":           # long runs of the same key
        rows = rng.integers(0, 17, size=n - 100).astype(np.int64) * 65537
    else:
        rows = rng.integers(0, n // 2, size=n - 100).astype(np.int64)
    seeds = rows[rng.permutation(rows.size)[:100]]
    other = rng.integers(0, 1 << 21, size=999).astype(np.int64)
    frontier, outs = _run([seeds, rows], [rows, other], dev, idt)
    want_frontier, want = O.relabel([seeds, rows], [rows, other])
    assert np.array_equal(frontier, want_frontier)
    for g, w in zip(outs, want):
        assert np.array_equal(g, w)


def test_64_bit_ids_on_one_word_slots(dev):
    """GS_NARROW_IDS: 64-bit ids that fit 32 bits give the same frontier and ranks as the
    two-array table, lookups of ids beyond 32 bits come back absent, and a mapping id beyond
    32 bits is reported (-2) rather than truncated."""
    rng = np.random.default_rng(12)
    a = rng.integers(0, 5000, 30000).astype(np.int64) + 4_000_000_000     # still below 2^32
    b = rng.integers(0, 5000, 20000).astype(np.int64) + 4_000_000_000
    q = np.concatenate([b[:1000], np.array([1 << 40, (1 << 32) + 5], dtype=np.int64)])
    for narrow in (False, True):
        frontier, num, outs = capi.unique_relabel([to_dev(a, dev), to_dev(b, dev)],
                                                  [to_dev(b, dev), to_dev(q, dev)], narrow=narrow)
        w_frontier, w_outs = O.relabel([a, b], [b, q])
        U = int(num.item())
        assert U == w_frontier.size
        assert np.array_equal(frontier[:U].cpu().numpy(), w_frontier)
        assert np.array_equal(outs[0].cpu().numpy(), w_outs[0])
        assert np.array_equal(outs[1].cpu().numpy(), w_outs[1])
        assert outs[1][-1].item() == -1 and outs[1][-2].item() == -1
    big = a.copy()
    big[777] = (1 << 36) + 1
    _, num, _ = capi.unique_relabel([to_dev(big, dev)], [], narrow=True)
    assert int(num.item()) == -2
    # the same with lookups queued behind the pass that gave up: void outputs, but the call ends
    t_big = to_dev(big, dev)
    _, num, _ = capi.unique_relabel([t_big], [t_big, to_dev(q, dev)], narrow=True)
    assert int(num.item()) == -2
    frontier, num, _ = capi.unique_relabel([to_dev(big, dev)], [], narrow=False)
    assert np.array_equal(frontier[:int(num.item())].cpu().numpy(), O.relabel([big], [])[0])
