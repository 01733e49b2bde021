"""GPU parity: the one-launch slice + sample (gs_sample_uniform_fused) and the result mailbox,
against the CPU oracle and against the two-phase calls."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from graph_sampling_amd import capi
from tests.util import graph_20x5, rmat_csc_np, to_dev, u32_draws

pytestmark = pytest.mark.gpu

ID_DTYPES = [torch.int64, torch.int32]


def _narrow(res):
    sub_indptr, sub_indices, select_index, coo_col = res[:4]
    nnz = int(sub_indptr[-1].item())
    return (sub_indptr, None if coo_col is None else coo_col[:nnz], sub_indices[:nnz],
            select_index[:nnz])


def _cmp(got, want):
    for g, w in zip(got, want):
        if w is None:
            assert g is None
            continue
        g = g.cpu().numpy().astype(np.int64)
        assert g.shape == w.shape, (g.shape, w.shape)
        assert np.array_equal(g, w)


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("replace", [False, True])
@pytest.mark.parametrize("k", [1, 4, 5, 8, 9, 15, 16, 17, 31, 32])
@pytest.mark.parametrize("fused_cols", [True, False])
def test_fused_matches_oracle(dev, idt, replace, k, fused_cols):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 17, seed=5)
    if fused_cols:
        cols = np.random.default_rng(k).integers(0, indptr.size - 1, size=3000).astype(np.int64)
        cols[:8] = np.argsort(np.diff(indptr))[-8:]
        dcols = to_dev(cols, dev, idt)
    else:
        cols, dcols = None, None
    got = _narrow(capi.sample_uniform_fused(to_dev(indptr, dev), to_dev(indices, dev, idt), dcols, k,
                                            replace, seed=99 + k, with_coo=True))
    _cmp(got, O.sample_uniform(indptr, indices, cols, k, replace, seed=99 + k, with_coo=True))


@pytest.mark.parametrize("replace", [False, True])
@pytest.mark.parametrize("k", [33, 70, 200])
def test_fused_large_fanout(dev, replace, k):
    """With replacement any fanout runs; without, fanouts above 32 are refused (two-phase path)."""
    indptr, indices = rmat_csc_np(1 << 10, 1 << 15, seed=8)
    cols = np.random.default_rng(3).integers(0, 1 << 10, size=500).astype(np.int64)
    args = (to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev), k, replace)
    if not replace:
        with pytest.raises(capi.GsError, match="exceeds 32"):
            capi.sample_uniform_fused(*args, seed=1)
        return
    _cmp(_narrow(capi.sample_uniform_fused(*args, seed=1, with_coo=True)),
         O.sample_uniform(indptr, indices, cols, k, replace, seed=1))


@pytest.mark.parametrize("S", [70001, 0, 1, 255, 256, 257, 16384, 16385, 300])
def test_fused_tile_boundaries_and_long_lookback(dev, S):
    """Row counts around the 256-row tile and past 64 tiles (more than one look-back window)."""
    indptr, indices = rmat_csc_np(1 << 13, 1 << 17, seed=2)
    cols = np.random.default_rng(S).integers(0, 1 << 13, size=S).astype(np.int64)
    d = (to_dev(indptr, dev), to_dev(indices, dev, torch.int32), to_dev(cols, dev, torch.int32))
    for replace in (False, True):
        got = _narrow(capi.sample_uniform_fused(*d, 7, replace, seed=S, with_coo=True))
        _cmp(got, O.sample_uniform(indptr, indices, cols, 7, replace, seed=S))


@pytest.mark.parametrize("idt", ID_DTYPES)
@pytest.mark.parametrize("k,replace", [(7, False), (16, False), (32, False), (3, True), (40, True)])
def test_fused_very_many_columns_take_the_row_per_lane_kernel(dev, idt, k, replace):
    """From 2^18 columns on, the launch runs one row per lane with an edge-parallel fill; same
    draws and outputs as below that size (the oracle knows one definition only)."""
    indptr, indices = rmat_csc_np(1 << 13, 1 << 17, seed=2)
    S = (1 << 18) + 77
    cols = np.random.default_rng(k).integers(0, 1 << 13, size=S).astype(np.int64)
    cols[::1000] = -5
    d = (to_dev(indptr, dev), to_dev(indices, dev, idt), to_dev(cols, dev, idt))
    got = _narrow(capi.sample_uniform_fused(*d, k, replace, seed=S + k, with_coo=True))
    _cmp(got, O.sample_uniform(indptr, indices, cols, k, replace, seed=S + k))


@pytest.mark.parametrize("with_edge_ids", [False, True])
@pytest.mark.parametrize("S,k,replace", [(3000, 15, False), (3000, 4, True), (3000, 70, True),
                                         ((1 << 18) + 77, 7, False), ((1 << 18) + 5, 3, True),
                                         (0, 5, False)])
def test_fused_carries_edge_data(dev, S, k, replace, with_edge_ids):
    """gs_sample_uniform_fused_data: the same samples as gs_sample_uniform_fused plus
    data[e_ids[select_index]] (reference src/graph.cc:544-557), by both kernels of the launch
    (G lanes per row; one row per lane from 2^18 columns on)."""
    indptr, indices = rmat_csc_np(1 << 13, 1 << 17, seed=6)
    rng = np.random.default_rng(S + k)
    cols = rng.integers(0, 1 << 13, size=S).astype(np.int64)
    data = (1.0 - rng.random(indices.size)).astype(np.float32)
    e_ids = rng.permutation(indices.size).astype(np.int64) if with_edge_ids else None
    d = (to_dev(indptr, dev), to_dev(indices, dev, torch.int32), to_dev(cols, dev, torch.int32))
    res = capi.sample_uniform_fused(*d, k, replace, seed=S + k, with_coo=True,
                                    edge_data=to_dev(data, dev),
                                    edge_ids=None if e_ids is None else to_dev(e_ids, dev))
    want = O.sample_uniform(indptr, indices, cols, k, replace, seed=S + k)
    _cmp(_narrow(res), want)
    sel = want[3]
    picked = data[sel] if e_ids is None else data[e_ids[sel]]
    assert np.array_equal(res[-1][:sel.size].cpu().numpy(), picked)


def test_fused_equals_two_phase_at_benchmark_shape(dev):
    """Layer-3-like shape: 45k seed columns, fanout 5; the two entry points agree bit for bit."""
    indptr, indices = rmat_csc_np(1 << 16, 1 << 21, seed=4)
    cols = np.random.default_rng(0).integers(0, 1 << 16, size=45000).astype(np.int64)
    d = (to_dev(indptr, dev), to_dev(indices, dev, torch.int32), to_dev(cols, dev, torch.int32))
    a = _narrow(capi.sample_uniform_fused(*d, 5, False, seed=11))
    b = capi.sample_uniform(*d, 5, False, seed=11)
    nnz = int(b[0][-1].item())
    assert torch.equal(a[0], b[0])
    assert torch.equal(a[2], b[1][:nnz]) and torch.equal(a[3], b[2][:nnz])


@pytest.mark.parametrize("replace", [False, True])
def test_fused_replay(dev, replace):
    indptr, indices = rmat_csc_np(1 << 12, 1 << 17, seed=6)
    cols = np.random.default_rng(1).integers(0, indptr.size - 1, size=2000).astype(np.int64)
    cols[:4] = np.argsort(np.diff(indptr))[-4:]
    _, replay_ptr = O.sample_count(indptr, cols, 15, replace, want_replay_ptr=True)
    replay = u32_draws(int(replay_ptr[-1]), seed=15)
    want = O.sample_uniform(indptr, indices, cols, 15, replace, replay=replay)
    got = _narrow(capi.sample_uniform_fused(to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev),
                                            15, replace, replay=to_dev(replay, dev),
                                            replay_ptr=to_dev(replay_ptr, dev), with_coo=True))
    _cmp(got, want)


def test_fused_reference_identity_vector(dev):
    """tests/test_colwise_sampling.cc:7-20 of the reference: fanout >= degree copies in order."""
    indptr, indices = graph_20x5()
    got = _narrow(capi.sample_uniform_fused(to_dev(indptr, dev), to_dev(indices, dev), None, 5, False))
    assert np.array_equal(got[0].cpu().numpy(), indptr)
    assert np.array_equal(got[2].cpu().numpy(), indices)


def test_fused_out_of_range_columns(dev):
    indptr, indices = rmat_csc_np(1 << 10, 1 << 14, seed=12)
    n = 1 << 10
    cols = np.random.default_rng(0).integers(0, n, size=600).astype(np.int64)
    cols[::7] = -1
    cols[3::11] = n
    cols[5::13] = n + 12345
    d = (to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev))
    for replace in (False, True):
        _cmp(_narrow(capi.sample_uniform_fused(*d, 6, replace, seed=3, with_coo=True)),
             O.sample_uniform(indptr, indices, cols, 6, replace, seed=3))


def test_epoch_wrap_rezeroes_state(dev):
    """More calls than there are epochs on one state buffer: the wrap zero-fills and restarts."""
    indptr, indices = rmat_csc_np(1 << 10, 1 << 14, seed=3)
    cols = np.random.default_rng(1).integers(0, 1 << 10, size=700).astype(np.int64)
    d = (to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev))
    want = O.sample_uniform(indptr, indices, cols, 3, False, seed=5, with_coo=False)
    key = (dev.index, torch.cuda.current_stream(dev).cuda_stream)
    capi.sample_uniform_fused(*d, 3, False, seed=5)
    buf, _ = capi._fused_state[key]
    capi._fused_state[key] = (buf, capi.MAX_EPOCH - 2)
    for _ in range(5):
        got = _narrow(capi.sample_uniform_fused(*d, 3, False, seed=5))
        _cmp(got, want)
    assert capi._fused_state[key][1] == 3


def test_mailbox_reports_totals(dev):
    """The kernels post {total, ticket} to pinned host memory; the host never syncs the stream."""
    indptr, indices = rmat_csc_np(1 << 12, 1 << 17, seed=5)
    d_ip, d_ix = to_dev(indptr, dev), to_dev(indices, dev, torch.int32)
    box = capi.Mailbox()
    for it in range(20):
        S = [0, 1, 300, 5000, 20000][it % 5]
        cols = np.random.default_rng(it).integers(0, 1 << 12, size=S).astype(np.int64)
        d_cols = to_dev(cols, dev, torch.int32)
        res = capi.sample_uniform_fused(d_ip, d_ix, d_cols, 10, False, seed=it, mailbox=box)
        nnz = box.wait(res[4], dev)
        want = O.sample_uniform(indptr, indices, cols, 10, False, seed=it)
        assert nnz == int(want[0][-1])
        sub = res[1][:nnz]
        frontier, num, outs, ticket = capi.unique_relabel([d_cols, sub], [sub], mailbox=box)
        U = box.wait(ticket, dev)
        f_want, r_want = O.relabel([cols, want[2]], [want[2]])
        assert U == f_want.size
        assert np.array_equal(frontier[:U].cpu().numpy().astype(np.int64), f_want)
        assert np.array_equal(outs[0].cpu().numpy().astype(np.int64), r_want[0])
        assert int(num.item()) == U


@pytest.mark.parametrize("idt", ID_DTYPES)
def test_relabel_with_device_side_length(dev, idt):
    """Sampler -> relabel with no host read in between: the relabel kernels take the length of the
    sampled ids from sub_indptr[S] on the device and treat the padded tail as absent."""
    indptr, indices = rmat_csc_np(1 << 12, 1 << 17, seed=5)
    d_ip, d_ix = to_dev(indptr, dev), to_dev(indices, dev, idt)
    box = capi.Mailbox()
    for it, S in enumerate([0, 1, 300, 5000, 20000, 7]):
        cols = np.random.default_rng(it).integers(0, 1 << 12, size=S).astype(np.int64)
        d_cols = to_dev(cols, dev, idt)
        sub_indptr, sub, sel, _ = capi.sample_uniform_fused(d_ip, d_ix, d_cols, 10, False, seed=it)
        frontier, num, outs, ticket = capi.unique_relabel([d_cols, sub], [sub], mailbox=box,
                                                          last_span_len=sub_indptr[S:])
        U = box.wait(ticket, dev)
        nnz = int(sub_indptr[S].item())
        want = O.sample_uniform(indptr, indices, cols, 10, False, seed=it)
        f_want, r_want = O.relabel([cols, want[2]], [want[2]])
        assert nnz == int(want[0][-1]) and U == f_want.size
        assert np.array_equal(frontier[:U].cpu().numpy().astype(np.int64), f_want)
        assert np.array_equal(outs[0][:nnz].cpu().numpy().astype(np.int64), r_want[0])


# ------------------------------ relabel behind the sampler on a persistent table
@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
@pytest.mark.parametrize("S,fanout,replace", [(1, 3, False), (700, 15, False), (5000, 5, False),
                                               (40000, 5, False), (3000, 4, True)])
def test_relabel_sampled_matches_the_one_call_relabel(dev, S, fanout, replace, idt):
    n = 1 << 14
    indptr, indices = rmat_csc_np(n, 1 << 19, seed=31)
    rng = np.random.default_rng(S)
    cols = rng.integers(0, n, size=S).astype(np.int64)            # duplicates among the seeds
    keys = cols + 1000                                            # the ids the columns go by
    t_ptr, t_idx = to_dev(indptr, dev), to_dev(indices, dev, idt)
    t_cols, t_keys = to_dev(cols, dev, idt), to_dev(keys, dev, idt)
    table = capi.RelabelTable(S + S * fanout + 100000, idt, dev)
    # several calls in a row on the same table: every call leaves it empty
    for seed in (5, 6, 7):
        sp, si, _, _ = capi.sample_uniform_fused(t_ptr, t_idx, t_cols, fanout, replace, seed=seed)
        copy = torch.full_like(sp, -7)
        frontier, num, out = capi.relabel_sampled(t_keys, sp, si, table, offsets_copy=copy)
        assert torch.equal(copy, sp)  # the sampler's offsets, copied by the last kernel
        w_sp, _, w_si, _ = O.sample_uniform(indptr, indices, cols, fanout, replace, seed=seed, with_coo=False)
        w_frontier, (w_out,) = O.relabel([keys, w_si], [w_si])
        E = int(w_sp[-1])
        assert np.array_equal(si[:E].cpu().numpy().astype(np.int64), w_si)
        assert int(num.item()) == w_frontier.size
        assert np.array_equal(frontier[:w_frontier.size].cpu().numpy().astype(np.int64), w_frontier)
        assert np.array_equal(out[:E].cpu().numpy().astype(np.int64), w_out)
    torch.cuda.synchronize()
    words = table.buf.view(torch.int64)
    if idt == torch.int32:
        assert bool((words == -1).all())
    else:
        slots = words.numel() * 8 // 12 // 1024 * 1024     # keys (8 B) then first indices (4 B)
        cap = 1 << (slots.bit_length() - 1)
        assert bool((words[:cap] == -1).all())


def test_relabel_sampled_narrow_slots_for_64_bit_ids(dev):
    """64-bit ids that fit 32 bits on the one-word slots: same frontier and renamed ids as the
    two-array table; an id beyond 32 bits is reported (-2) instead of being truncated."""
    n = 1 << 13
    indptr, indices = rmat_csc_np(n, 1 << 17, seed=9)
    cols = np.random.default_rng(4).integers(0, n, size=900).astype(np.int64)
    t_ptr, t_idx, t_cols = to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev)
    narrow = capi.RelabelTable(900 * 11 + 50000, torch.int64, dev, narrow=True)
    for shift in (0, 4_000_000_000, (1 << 33)):           # the last one does not fit 32 bits
        keys = cols + shift
        t_keys = to_dev(keys, dev)
        sp, si, _, _ = capi.sample_uniform_fused(t_ptr, t_idx, t_cols, 10, False, seed=3)
        w_sp, _, w_si, _ = O.sample_uniform(indptr, indices, cols, 10, False, seed=3, with_coo=False)
        frontier, num, out = capi.relabel_sampled(t_keys, sp, si, narrow)
        if shift == (1 << 33):
            assert int(num.item()) == -2
            break
        w_frontier, (w_out,) = O.relabel([keys, w_si], [w_si])
        E = int(w_sp[-1])
        assert int(num.item()) == w_frontier.size
        assert np.array_equal(frontier[:w_frontier.size].cpu().numpy(), w_frontier)
        assert np.array_equal(out[:E].cpu().numpy(), w_out)
    torch.cuda.synchronize()
    # the sticky error word of the look-back state must not leak into later calls of this process
    capi._fused_state.clear()


def test_bounded_wait_gives_up_and_the_error_sticks_until_the_state_is_cleared(dev):
    """The chained scan's wait for a predecessor is bounded.  gs_selftest_lookback leaves one tile
    out of the launch (every workgroup that does run reaches its end): the tiles behind it give
    up after the spin limit, the total reads -1, and the error word stays in the state -- a
    complete scan and the sampler itself report -1 on it -- until the state is zero-filled."""
    indptr, indices = rmat_csc_np(1 << 10, 1 << 14, seed=3)
    cols = np.random.default_rng(1).integers(0, 1 << 10, size=700).astype(np.int64)
    d = (to_dev(indptr, dev), to_dev(indices, dev), to_dev(cols, dev))
    want = O.sample_uniform(indptr, indices, cols, 3, False, seed=5, with_coo=False)
    key = (dev.index, torch.cuda.current_stream(dev).cuda_stream)
    state = torch.zeros(1 << 16, dtype=torch.uint8, device=dev)
    saved = capi._fused_state.get(key)
    try:
        assert int(capi.selftest_lookback(state, 1, 700, -1, 1 << 20)) == 700
        for missing in (0, 5, 698):
            state.zero_()
            assert int(capi.selftest_lookback(state, 2, 700, missing, 48)) == -1
        assert int(capi.selftest_lookback(state, 3, 700, -1, 1 << 20)) == -1      # sticky
        capi._fused_state[key] = (state, 3)
        got = capi.sample_uniform_fused(*d, 3, False, seed=5)
        assert int(got[0][-1]) == -1                                                # sticky
        state.zero_()
        capi._fused_state[key] = (state, 0)
        _cmp(_narrow(capi.sample_uniform_fused(*d, 3, False, seed=5)), want)
        assert int(capi.selftest_lookback(state, 9, 700, -1, 1 << 20)) == 700
    finally:
        if saved is None:
            capi._fused_state.pop(key, None)
        else:
            capi._fused_state[key] = saved
