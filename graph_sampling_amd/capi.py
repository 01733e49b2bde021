"""ctypes binding of the C ABI declared in ``include/gs_hip.h``.

torch is used for device memory and the current HIP stream only; every call
hands raw device pointers and sizes to ``libgs_hip.so``.  There is no fallback:
if the library is missing, importing a symbol raises.
"""
import ctypes
import os

import torch

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libgs_hip.so")

_lib = None


class GsError(RuntimeError):
    """A C-ABI call returned a negative gs_status."""


def lib():
    """The loaded kernel library (raises when it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise GsError("%s is missing: run `python -m graph_sampling_amd.build`" % LIB_PATH)
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.gs_status_string.restype = ctypes.c_char_p
        _lib.gs_status_string.argtypes = [ctypes.c_int]
        for name in ("gs_slice_workspace_bytes", "gs_sample_workspace_bytes",
                     "gs_sample_weighted_workspace_bytes", "gs_list_sample_workspace_bytes",
                     "gs_unique_workspace_bytes", "gs_row_slice_workspace_bytes",
                     "gs_sample_fused_state_bytes", "gs_batch_relabel_workspace_bytes",
                     "gs_coo2csc_workspace_bytes", "gs_col_row_slice_workspace_bytes",
                     "gs_index_search_workspace_bytes", "gs_relabel_table_bytes",
                     "gs_relabel_sampled_workspace_bytes", "gs_relabel_sampled_state_bytes",
                     "gs_segment_workspace_bytes", "gs_layer_workspace_bytes",
                     "gs_layer_sample_state_bytes", "gs_layer_relabel_state_bytes",
                     "gs_coo_sum_workspace_bytes", "gs_coo_pick_rows_workspace_bytes",
                     "gs_coo_block_values_workspace_bytes"):
            if hasattr(_lib, name):
                getattr(_lib, name).restype = ctypes.c_size_t
        _lib.gs_sorted_union_max.restype = ctypes.c_int64
    return _lib


def _check(status, what):
    if status != 0:
        raise GsError("%s failed (%d): %s" % (what, status, lib().gs_status_string(status).decode()))


def _ptr(t):
    if t is None:
        return ctypes.c_void_p(0)
    return ctypes.c_void_p(t.data_ptr())


def _i64(v):
    return ctypes.c_int64(int(v))


def _u64(v):
    return ctypes.c_uint64(int(v) & 0xFFFFFFFFFFFFFFFF)


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _id_bytes(t):
    if t.dtype == torch.int64:
        return 8
    if t.dtype == torch.int32:
        return 4
    raise GsError("node ids must be int64 or int32, got %s" % t.dtype)


def _need(t, dtype, name):
    if t.dtype != dtype:
        raise GsError("%s must be %s, got %s" % (name, dtype, t.dtype))
    if not t.is_cuda:
        raise GsError("%s must live on the GPU (there is no CPU path)" % name)
    if not t.is_contiguous():
        raise GsError("%s must be contiguous" % name)


def _ids(t, name, like=None):
    if not t.is_cuda:
        raise GsError("%s must live on the GPU (there is no CPU path)" % name)
    if not t.is_contiguous():
        raise GsError("%s must be contiguous" % name)
    b = _id_bytes(t)
    if like is not None and t.dtype != like.dtype:
        raise GsError("%s must have the dtype of the graph ids (%s), got %s" % (name, like.dtype, t.dtype))
    return b


def _replay(t):
    """Replay draws are raw uint32 values; torch carries them as int32 bit patterns."""
    if t.element_size() != 4 or not t.is_cuda or not t.is_contiguous():
        raise GsError("replay must be a contiguous 4-byte integer tensor on the GPU")


class _Workspace:
    """One growing scratch buffer per device (256-byte aligned by the torch allocator)."""

    def __init__(self):
        self._buf = {}

    def get(self, nbytes, device):
        nbytes = max(int(nbytes), 256)
        key = torch.device(device).index or 0
        buf = self._buf.get(key)
        if buf is None or buf.numel() < nbytes:
            buf = torch.empty(int(nbytes * 1.25) + 256, dtype=torch.uint8, device=device)
            self._buf[key] = buf
        return buf


_ws = _Workspace()


def workspace(nbytes, device):
    return _ws.get(nbytes, device)


# ---------------------------------------------------------------- slicing ----
def slice_count(indptr, column_ids):
    """gs_slice_count -> sub_indptr[S+1] (device); total still on the device."""
    _need(indptr, torch.int64, "indptr")
    idb = _ids(column_ids, "column_ids")
    S = column_ids.numel()
    sub_indptr = torch.empty(S + 1, dtype=torch.int64, device=indptr.device)
    nbytes = lib().gs_slice_workspace_bytes(_i64(S))
    ws = workspace(nbytes, indptr.device)
    _check(lib().gs_slice_count(_ptr(indptr), _i64(indptr.numel() - 1), _ptr(column_ids), idb, _i64(S), _ptr(sub_indptr),
                                _ptr(ws), ctypes.c_size_t(ws.numel()), _stream(indptr.device)),
           "gs_slice_count")
    return sub_indptr


def slice_fill(indptr, indices, column_ids, sub_indptr, nnz, with_coo):
    _need(indptr, torch.int64, "indptr")
    idb = _ids(indices, "indices")
    _ids(column_ids, "column_ids", like=indices)
    S = column_ids.numel()
    dev = indptr.device
    sub_indices = torch.empty(nnz, dtype=indices.dtype, device=dev)
    select_index = torch.empty(nnz, dtype=torch.int64, device=dev)
    coo_col = torch.empty(nnz, dtype=indices.dtype, device=dev) if with_coo else None
    _check(lib().gs_slice_fill(_ptr(indptr), _i64(indptr.numel() - 1), _ptr(indices), _ptr(column_ids), idb, _i64(S),
                               _ptr(sub_indptr), _i64(nnz), _ptr(sub_indices), _ptr(select_index),
                               _ptr(coo_col), _stream(dev)), "gs_slice_fill")
    return sub_indices, select_index, coo_col


# --------------------------------------------------------------- sampling ----
ALGO_AUTO, ALGO_RESERVOIR = 0, 1


def sample_uniform(indptr, indices, column_ids, fanout, replace, seed=0, replay=None,
                   replay_ptr=None, with_coo=False, algo=ALGO_AUTO):
    """gs_sample_count + gs_sample_uniform_fill on upper-bound buffers.

    Returns (sub_indptr, sub_indices_buf, select_index_buf, coo_col_buf); the
    buffers have capacity S*fanout and the caller narrows them to
    sub_indptr[S] once it has read that value."""
    _need(indptr, torch.int64, "indptr")
    idb = _ids(indices, "indices")
    dev = indptr.device
    if column_ids is None:
        S = indptr.numel() - 1
    else:
        _ids(column_ids, "column_ids", like=indices)
        S = column_ids.numel()
    if replay is not None:
        _replay(replay)
        _need(replay_ptr, torch.int64, "replay_ptr")
    sub_indptr = torch.empty(S + 1, dtype=torch.int64, device=dev)
    cap = S * int(fanout)
    sub_indices = torch.empty(cap, dtype=indices.dtype, device=dev)
    select_index = torch.empty(cap, dtype=torch.int64, device=dev)
    coo_col = torch.empty(cap, dtype=indices.dtype, device=dev) if with_coo else None
    nbytes = lib().gs_sample_workspace_bytes(_i64(S), _i64(fanout))
    ws = workspace(nbytes, dev)
    st = _stream(dev)
    _check(lib().gs_sample_count(_ptr(indptr), _i64(indptr.numel() - 1), _ptr(column_ids), idb, _i64(S), _i64(fanout),
                                 int(bool(replace)), _ptr(sub_indptr), _ptr(ws),
                                 ctypes.c_size_t(ws.numel()), st), "gs_sample_count")
    _check(lib().gs_sample_uniform_fill(_ptr(indptr), _i64(indptr.numel() - 1), _ptr(indices), _ptr(column_ids), idb, _i64(S),
                                        _i64(fanout), int(bool(replace)), int(algo), _u64(seed),
                                        _ptr(replay),
                                        _ptr(replay_ptr), _ptr(sub_indptr), _ptr(sub_indices),
                                        _ptr(select_index), _ptr(coo_col), _ptr(ws),
                                        ctypes.c_size_t(ws.numel()), st), "gs_sample_uniform_fill")
    return sub_indptr, sub_indices, select_index, coo_col


_fused_state = {}


MAX_EPOCH = (1 << 14) - 1


def fused_state(nbytes, device):
    """(state buffer, epoch) of gs_sample_uniform_fused for the current stream: zero-filled when
    (re)allocated and whenever the epoch counter wraps."""
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    buf, epoch = _fused_state.get(key, (None, 0))
    if buf is None or buf.numel() < nbytes:
        buf, epoch = torch.zeros(max(int(nbytes), 65536), dtype=torch.uint8, device=device), 0
    if epoch == MAX_EPOCH:
        buf.zero_()
        epoch = 0
    epoch += 1
    _fused_state[key] = (buf, epoch)
    return buf, epoch


def selftest_lookback(state, epoch, tiles, missing_tile, spin_limit):
    """gs_selftest_lookback on the caller's state buffer; returns the total as a device scalar."""
    total = torch.full((1,), -7, dtype=torch.int64, device=state.device)
    _check(lib().gs_selftest_lookback(_ptr(state), ctypes.c_size_t(state.numel()),
                                      ctypes.c_uint32(epoch), _i64(tiles), _i64(missing_tile),
                                      int(spin_limit), _ptr(total), _stream(state.device)),
           "gs_selftest_lookback")
    return total


class Mailbox:
    """gs_mailbox in pinned host memory plus the host side of the protocol."""

    def __init__(self):
        self.buf = torch.zeros(2, dtype=torch.int64).pin_memory()
        self.next_ticket = 1

    def ptr(self):
        return ctypes.c_void_p(self.buf.data_ptr())

    def ticket(self):
        t = self.next_ticket
        self.next_ticket += 1
        return t

    def wait(self, ticket, device, spins=200_000_000):
        words = (ctypes.c_int64 * 2).from_address(self.buf.data_ptr())
        stream = torch.cuda.current_stream(device)
        n = 0
        while words[1] != ticket:
            n += 1
            if n % 4096 == 0 and stream.query() and words[1] != ticket:
                raise GsError("the stream drained without posting mailbox ticket %d" % ticket)
            if n > spins:
                raise GsError("timed out waiting for mailbox ticket %d" % ticket)
        return int(words[0])


def sample_uniform_fused(indptr, indices, column_ids, fanout, replace, seed=0, replay=None,
                         replay_ptr=None, with_coo=False, mailbox=None, edge_data=None,
                         edge_ids=None):
    """gs_sample_uniform_fused: one launch.  Same return shape as sample_uniform; with a
    Mailbox also returns the ticket to wait on as a fifth element.  With edge_data (fp32, and
    optionally the int64 edge-id map edge_ids) the call is gs_sample_uniform_fused_data and the
    samples' edge data, at capacity, comes back as the last element."""
    _need(indptr, torch.int64, "indptr")
    idb = _ids(indices, "indices")
    dev = indptr.device
    if column_ids is None:
        S = indptr.numel() - 1
    else:
        _ids(column_ids, "column_ids", like=indices)
        S = column_ids.numel()
    if replay is not None:
        _replay(replay)
        _need(replay_ptr, torch.int64, "replay_ptr")
    sub_indptr = torch.empty(S + 1, dtype=torch.int64, device=dev)
    cap = S * int(fanout)
    sub_indices = torch.empty(cap, dtype=indices.dtype, device=dev)
    select_index = torch.empty(cap, dtype=torch.int64, device=dev)
    coo_col = torch.empty(cap, dtype=indices.dtype, device=dev) if with_coo else None
    state, epoch = fused_state(lib().gs_sample_fused_state_bytes(_i64(S)), dev)
    ticket = mailbox.ticket() if mailbox is not None else 0
    box = mailbox.ptr() if mailbox is not None else ctypes.c_void_p(0)
    if edge_data is not None:
        _need(edge_data, torch.float32, "edge_data")
        if edge_ids is not None:
            _need(edge_ids, torch.int64, "edge_ids")
        data_out = torch.empty(cap, dtype=torch.float32, device=dev)
        _check(lib().gs_sample_uniform_fused_data(
            _ptr(indptr), _i64(indptr.numel() - 1), _ptr(indices), _ptr(column_ids), idb, _i64(S),
            _i64(fanout), int(bool(replace)), _u64(seed), _ptr(replay), _ptr(replay_ptr),
            _ptr(sub_indptr), _ptr(sub_indices), _ptr(select_index), _ptr(coo_col), _i64(cap),
            _ptr(edge_data), _ptr(edge_ids), _ptr(data_out),
            _ptr(state), ctypes.c_size_t(state.numel()), ctypes.c_uint32(epoch),
            box, _i64(ticket), _stream(dev)), "gs_sample_uniform_fused_data")
        if mailbox is not None:
            return sub_indptr, sub_indices, select_index, coo_col, ticket, data_out
        return sub_indptr, sub_indices, select_index, coo_col, data_out
    _check(lib().gs_sample_uniform_fused(
        _ptr(indptr), _i64(indptr.numel() - 1), _ptr(indices), _ptr(column_ids), idb, _i64(S),
        _i64(fanout), int(bool(replace)), _u64(seed), _ptr(replay), _ptr(replay_ptr),
        _ptr(sub_indptr), _ptr(sub_indices), _ptr(select_index), _ptr(coo_col), _i64(cap),
        _ptr(state), ctypes.c_size_t(state.numel()), ctypes.c_uint32(epoch),
        box, _i64(ticket), _stream(dev)),
        "gs_sample_uniform_fused")
    if mailbox is not None:
        return sub_indptr, sub_indices, select_index, coo_col, ticket
    return sub_indptr, sub_indices, select_index, coo_col


def sample_uniform_fused_static(indptr, indices, column_ids, fanout, replace, out, seed=0,
                                replay=None, replay_ptr=None, mailbox=None):
    """gs_sample_uniform_fused_static: the one-launch sampler on the library's own state, for
    callers that cannot allocate.  `out` = (sub_indptr[S + 1], sub_indices[cap], select_index[cap]
    or None, coo_col[cap] or None), all the caller's; nothing is allocated here or in the call."""
    _need(indptr, torch.int64, "indptr")
    idb = _ids(indices, "indices")
    dev = indptr.device
    S = indptr.numel() - 1 if column_ids is None else column_ids.numel()
    sub_indptr, sub_indices, select_index, coo_col = out
    ticket = mailbox.ticket() if mailbox is not None else 0
    _check(lib().gs_sample_uniform_fused_static(
        _ptr(indptr), _i64(indptr.numel() - 1), _ptr(indices), _ptr(column_ids), idb, _i64(S),
        _i64(fanout), int(bool(replace)), _u64(seed), _ptr(replay), _ptr(replay_ptr),
        _ptr(sub_indptr), _ptr(sub_indices), _ptr(select_index), _ptr(coo_col),
        _i64(sub_indices.numel()),
        mailbox.ptr() if mailbox is not None else ctypes.c_void_p(0), _i64(ticket), _stream(dev)),
        "gs_sample_uniform_fused_static")
    return ticket


def static_init():
    """gs_sample_uniform_fused_static_init: resolves the library's state array on the current
    device (to be called before a stream capture that records the static sampler)."""
    _check(lib().gs_sample_uniform_fused_static_init(), "gs_sample_uniform_fused_static_init")


def static_reset():
    """gs_sample_uniform_fused_static_reset: the next static call starts from a zero-filled
    state (after a call that reported -1)."""
    _check(lib().gs_sample_uniform_fused_static_reset(), "gs_sample_uniform_fused_static_reset")


def static_debug_raise(device):
    """Raises the sticky error word in the library's own look-back state (test hook)."""
    _check(lib().gs_sample_uniform_fused_static_debug_raise(_stream(device)),
           "gs_sample_uniform_fused_static_debug_raise")


class RelabelTable:
    """The persistent hash table of gs_relabel_sampled (prepared once, left empty by every call)."""

    def __init__(self, max_items, id_dtype, device, narrow=False):
        """narrow: 64-bit ids on the one-word slots of 32-bit ids (gs_relabel_sampled_narrow)."""
        self.idb = 8 if id_dtype == torch.int64 else 4
        self.narrow = bool(narrow) and self.idb == 8
        nbytes = lib().gs_relabel_table_bytes(_i64(max_items), self.idb)
        self.buf = torch.empty(int(nbytes), dtype=torch.uint8, device=device)
        self.prepare()

    def prepare(self):
        _check(lib().gs_relabel_table_init(_ptr(self.buf), ctypes.c_size_t(self.buf.numel()),
                                           4 if self.narrow else self.idb,
                                           _stream(self.buf.device)),
               "gs_relabel_table_init")


def relabel_sampled(seed_keys, sub_indptr, sub_indices, table, mailbox=None, offsets_copy=None):
    """gs_relabel_sampled behind a sampler whose total is still on the device (sub_indptr[S]).
    Returns (frontier buffer, num_unique (device), relabelled sampled ids at capacity[, ticket]);
    `offsets_copy` (int64[S + 1]) receives a copy of sub_indptr."""
    idb = _ids(seed_keys, "seed_keys")
    _ids(sub_indices, "sampled ids", like=seed_keys)
    dev = seed_keys.device
    S, cap = seed_keys.numel(), sub_indices.numel()
    M = S + cap
    frontier = torch.empty(M, dtype=seed_keys.dtype, device=dev)
    out_ids = torch.empty(cap, dtype=seed_keys.dtype, device=dev)
    num_unique = torch.empty(1, dtype=torch.int64, device=dev)
    ws = workspace(lib().gs_relabel_sampled_workspace_bytes(_i64(M)), dev)
    state, epoch = fused_state(lib().gs_relabel_sampled_state_bytes(_i64(M)), dev)
    ticket = mailbox.ticket() if mailbox is not None else 0
    box = mailbox.ptr() if mailbox is not None else ctypes.c_void_p(0)
    if table.narrow:
        _check(lib().gs_relabel_sampled_narrow(
            _ptr(seed_keys), _i64(S), _ptr(sub_indices), _i64(cap),
            ctypes.c_void_p(sub_indptr.data_ptr() + 8 * S), _ptr(table.buf),
            ctypes.c_size_t(table.buf.numel()), _ptr(frontier), _ptr(out_ids), _ptr(num_unique),
            _ptr(offsets_copy), _ptr(ws), ctypes.c_size_t(ws.numel()), _ptr(state),
            ctypes.c_size_t(state.numel()), ctypes.c_uint32(epoch), box, _i64(ticket),
            _stream(dev)), "gs_relabel_sampled_narrow")
    else:
        _check(lib().gs_relabel_sampled(
            _ptr(seed_keys), _i64(S), _ptr(sub_indices), _i64(cap),
            ctypes.c_void_p(sub_indptr.data_ptr() + 8 * S), idb, _ptr(table.buf),
            ctypes.c_size_t(table.buf.numel()), _ptr(frontier), _ptr(out_ids), _ptr(num_unique),
            _ptr(offsets_copy), _ptr(ws), ctypes.c_size_t(ws.numel()), _ptr(state),
            ctypes.c_size_t(state.numel()), ctypes.c_uint32(epoch), box, _i64(ticket),
            _stream(dev)), "gs_relabel_sampled")
    if mailbox is not None:
        return frontier, num_unique, out_ids, ticket
    return frontier, num_unique, out_ids


# ----------------------------------- a whole minibatch queued with no host read ----
class LayerBuffers:
    """What one layer of sample_layers owns: outputs at their bounds, device-side counts."""

    def __init__(self, S_bound, fanout, id_dtype, device, with_data=False):
        self.S_bound = int(S_bound)
        self.fanout = int(fanout)
        self.capacity = self.S_bound * self.fanout
        self.sub_indptr = torch.empty(self.S_bound + 1, dtype=torch.int64, device=device)
        self.sub_indices = torch.empty(self.capacity, dtype=id_dtype, device=device)
        self.out_ids = torch.empty(self.capacity, dtype=id_dtype, device=device)
        self.frontier = torch.empty(self.S_bound + self.capacity, dtype=id_dtype, device=device)
        self.offsets_copy = torch.empty(self.S_bound + 1, dtype=torch.int64, device=device)
        self.counts = torch.zeros(2, dtype=torch.int64, device=device)  # num_edges, num_unique
        # only with edge data: positions of the samples in the graph's indices, and their data
        self.select_index = self.data = None
        if with_data:
            self.select_index = torch.empty(self.capacity, dtype=torch.int64, device=device)
            self.data = torch.empty(self.capacity, dtype=torch.float32, device=device)
        self.workspace = torch.empty(
            int(lib().gs_layer_workspace_bytes(_i64(self.S_bound), _i64(self.fanout))),
            dtype=torch.uint8, device=device)

    def num_edges_ptr(self):
        return ctypes.c_void_p(self.counts.data_ptr())

    def num_unique_ptr(self):
        return ctypes.c_void_p(self.counts.data_ptr() + 8)


def sample_layers(indptr, indices, seeds, fanouts, replace=False, seed=0, mailbox=None,
                  tables=None, edge_data=None, edge_ids=None):
    """gs_layer_sample + gs_layer_relabel for every layer of a minibatch, queued back to back:
    layer l + 1 takes its column ids and their number from layer l's frontier and num_unique on
    the device.  Layer l draws with seed + l.  Returns (layers: list of LayerBuffers, ticket of
    the last relabel or None); sizes are the device-side counts of each layer.  With edge_data
    (fp32; edge_ids: the optional int64 edge-id map) every layer also leaves the positions of
    its samples (select_index) and their edge data (data), both at capacity."""
    if edge_data is not None:
        _need(edge_data, torch.float32, "edge_data")
        if edge_ids is not None:
            _need(edge_ids, torch.int64, "edge_ids")
    _need(indptr, torch.int64, "indptr")
    idb = _ids(indices, "indices")
    _ids(seeds, "seeds", like=indices)
    dev = indptr.device
    L = lib()
    bounds = [seeds.numel()]
    for k in fanouts:
        bounds.append(bounds[-1] * (1 + int(k)))
    layers = [LayerBuffers(bounds[l], k, indices.dtype, dev, edge_data is not None)
              for l, k in enumerate(fanouts)]
    if tables is None:
        tables = [RelabelTable(bounds[-1], torch.int32, dev) for _ in range(2)]
    state_bytes = max(max(L.gs_layer_sample_state_bytes(_i64(b.S_bound)),
                          L.gs_layer_relabel_state_bytes(_i64(b.S_bound), _i64(b.fanout)))
                      for b in layers)
    cols, S_dev = seeds, ctypes.c_void_p(0)
    ticket = None
    null = ctypes.c_void_p(0)
    for l, b in enumerate(layers):
        table = tables[l % 2]
        state, epoch = fused_state(state_bytes, dev)
        _check(L.gs_layer_sample(
            _ptr(indptr), _i64(indptr.numel() - 1), _ptr(indices), _ptr(cols), idb,
            _i64(b.S_bound), S_dev, _i64(b.fanout), int(bool(replace)), _u64(seed + l), null, null,
            _ptr(b.sub_indptr), _ptr(b.sub_indices), _i64(b.capacity), b.num_edges_ptr(),
            _ptr(b.select_index), _ptr(edge_data), _ptr(edge_ids), _ptr(b.data),
            _ptr(table.buf), ctypes.c_size_t(table.buf.numel()), _ptr(b.workspace),
            ctypes.c_size_t(b.workspace.numel()), _ptr(state), ctypes.c_size_t(state.numel()),
            ctypes.c_uint32(epoch), null, _i64(0), _stream(dev)), "gs_layer_sample")
        state, epoch = fused_state(state_bytes, dev)
        last = l == len(layers) - 1
        box, ticket = null, None
        if last and mailbox is not None:
            ticket = mailbox.ticket()
            box = mailbox.ptr()
        prev = layers[l - 1] if l > 0 else None
        prev_S_dev = null if l < 2 else layers[l - 2].num_unique_ptr()
        _check(L.gs_layer_relabel(
            idb, _i64(b.S_bound), S_dev, _i64(b.capacity), b.num_edges_ptr(), _ptr(b.sub_indptr),
            _ptr(table.buf), ctypes.c_size_t(table.buf.numel()), _ptr(b.workspace),
            ctypes.c_size_t(b.workspace.numel()), _ptr(b.frontier), _ptr(b.out_ids),
            b.num_unique_ptr(), _ptr(b.offsets_copy), _ptr(state), ctypes.c_size_t(state.numel()),
            ctypes.c_uint32(epoch),
            _ptr(tables[(l - 1) % 2].buf) if prev else null,
            ctypes.c_size_t(tables[(l - 1) % 2].buf.numel() if prev else 0),
            _ptr(prev.workspace) if prev else null,
            ctypes.c_size_t(prev.workspace.numel() if prev else 0),
            _i64(prev.S_bound if prev else 0), prev_S_dev, _i64(prev.capacity if prev else 0),
            prev.num_edges_ptr() if prev else null, box, _i64(ticket or 0), _stream(dev)),
            "gs_layer_relabel")
        cols, S_dev = b.frontier, b.num_unique_ptr()
    b = layers[-1]
    _check(L.gs_layer_table_sweep(
        _ptr(tables[(len(layers) - 1) % 2].buf),
        ctypes.c_size_t(tables[(len(layers) - 1) % 2].buf.numel()), _ptr(b.workspace),
        ctypes.c_size_t(b.workspace.numel()), _i64(b.S_bound),
        null if len(layers) < 2 else layers[-2].num_unique_ptr(), _i64(b.capacity),
        b.num_edges_ptr(), _stream(dev)), "gs_layer_table_sweep")
    return layers, ticket


def sample_one_keepdim(indptr, indices, column_ids, seed=0, replay=None):
    _need(indptr, torch.int64, "indptr")
    idb = _ids(indices, "indices")
    _ids(column_ids, "column_ids", like=indices)
    dev = indptr.device
    S = column_ids.numel()
    sub_indptr = torch.empty(S + 1, dtype=torch.int64, device=dev)
    sub_indices = torch.empty(S, dtype=indices.dtype, device=dev)
    select_index = torch.empty(S, dtype=torch.int64, device=dev)
    _check(lib().gs_sample_one_keepdim(_ptr(indptr), _i64(indptr.numel() - 1), _ptr(indices), _ptr(column_ids), idb, _i64(S),
                                       _u64(seed), _ptr(replay), _ptr(sub_indptr), _ptr(sub_indices),
                                       _ptr(select_index), _stream(dev)), "gs_sample_one_keepdim")
    return sub_indptr, sub_indices, select_index


def sample_weighted(indptr, indices, probs, column_ids, fanout, seed=0, replay=None,
                    replay_ptr=None, with_coo=False):
    """gs_sample_count(replace=0) + gs_sample_weighted_fill; same return shape as sample_uniform."""
    _need(indptr, torch.int64, "indptr")
    _need(probs, torch.float32, "probs")
    idb = _ids(indices, "indices")
    dev = indptr.device
    if column_ids is None:
        S = indptr.numel() - 1
    else:
        _ids(column_ids, "column_ids", like=indices)
        S = column_ids.numel()
    sub_indptr = torch.empty(S + 1, dtype=torch.int64, device=dev)
    cap = S * int(fanout)
    sub_indices = torch.empty(cap, dtype=indices.dtype, device=dev)
    select_index = torch.empty(cap, dtype=torch.int64, device=dev)
    coo_col = torch.empty(cap, dtype=indices.dtype, device=dev) if with_coo else None
    nbytes = max(lib().gs_sample_workspace_bytes(_i64(S), _i64(fanout)),
                 lib().gs_sample_weighted_workspace_bytes(_i64(S), _i64(fanout)))
    ws = workspace(nbytes, dev)
    st = _stream(dev)
    _check(lib().gs_sample_count(_ptr(indptr), _i64(indptr.numel() - 1), _ptr(column_ids), idb, _i64(S), _i64(fanout), 0,
                                 _ptr(sub_indptr), _ptr(ws), ctypes.c_size_t(ws.numel()), st),
           "gs_sample_count")
    _check(lib().gs_sample_weighted_fill(_ptr(indptr), _i64(indptr.numel() - 1), _ptr(indices), _ptr(probs), _ptr(column_ids),
                                         idb, _i64(S), _i64(fanout), _u64(seed), _ptr(replay),
                                         _ptr(replay_ptr), _ptr(sub_indptr), _ptr(sub_indices),
                                         _ptr(select_index), _ptr(coo_col), _ptr(ws),
                                         ctypes.c_size_t(ws.numel()), st), "gs_sample_weighted_fill")
    return sub_indptr, sub_indices, select_index, coo_col


def sample_weighted_replace(indptr, indices, probs, column_ids, fanout, seed=0, replay=None,
                            with_coo=False):
    """gs_sample_count(replace=1) + gs_sample_weighted_replace; returns (sub_indptr, sub_indices,
    select_index, coo_col), the buffers at capacity S * fanout."""
    _need(indptr, torch.int64, "indptr")
    _need(probs, torch.float32, "probs")
    idb = _ids(indices, "indices")
    dev = indptr.device
    if column_ids is None:
        S = indptr.numel() - 1
        cdf_ptr, cdf_len = indptr, indices.numel()
    else:
        _ids(column_ids, "column_ids", like=indices)
        S = column_ids.numel()
        cdf_ptr = slice_count(indptr, column_ids)
        cdf_len = _total(cdf_ptr, cdf_ptr.numel() - 1)
    sub_indptr = torch.empty(S + 1, dtype=torch.int64, device=dev)
    cap = S * int(fanout)
    sub_indices = torch.empty(cap, dtype=indices.dtype, device=dev)
    select_index = torch.empty(cap, dtype=torch.int64, device=dev)
    coo_col = torch.empty(cap, dtype=indices.dtype, device=dev) if with_coo else None
    cdf = torch.empty(max(cdf_len, 1), dtype=torch.float32, device=dev)
    ws = workspace(lib().gs_sample_workspace_bytes(_i64(S), _i64(fanout)), dev)
    st = _stream(dev)
    _check(lib().gs_sample_count(_ptr(indptr), _i64(indptr.numel() - 1), _ptr(column_ids), idb,
                                 _i64(S), _i64(fanout), 1, _ptr(sub_indptr), _ptr(ws),
                                 ctypes.c_size_t(ws.numel()), st), "gs_sample_count")
    _check(lib().gs_sample_weighted_replace(_ptr(indptr), _i64(indptr.numel() - 1), _ptr(indices),
                                            _ptr(probs), _ptr(column_ids), idb, _i64(S),
                                            _i64(fanout), _u64(seed), _ptr(replay), _ptr(sub_indptr),
                                            _ptr(cdf_ptr), _ptr(cdf), _ptr(sub_indices),
                                            _ptr(select_index), _ptr(coo_col), st),
           "gs_sample_weighted_replace")
    return sub_indptr, sub_indices, select_index, coo_col


def list_sample_uniform(data, k, replace, seed=0, replay=None):
    idb = _ids(data, "data")
    dev = data.device
    n = data.numel()
    out_data = torch.empty(k, dtype=data.dtype, device=dev)
    out_index = torch.empty(k, dtype=torch.int64, device=dev)
    ws = workspace(lib().gs_list_sample_workspace_bytes(_i64(n), _i64(k)), dev)
    _check(lib().gs_list_sample_uniform(_ptr(data), idb, _i64(n), _i64(k), int(bool(replace)),
                                        _u64(seed), _ptr(replay), _ptr(out_data), _ptr(out_index),
                                        _ptr(ws), ctypes.c_size_t(ws.numel()), _stream(dev)),
           "gs_list_sample_uniform")
    return out_data, out_index


def list_sample_weighted(data, probs, k, seed=0, replay=None):
    idb = _ids(data, "data")
    _need(probs, torch.float32, "probs")
    dev = data.device
    n = data.numel()
    out_data = torch.empty(k, dtype=data.dtype, device=dev)
    out_index = torch.empty(k, dtype=torch.int64, device=dev)
    ws = workspace(lib().gs_list_sample_workspace_bytes(_i64(n), _i64(k)), dev)
    _check(lib().gs_list_sample_weighted(_ptr(data), idb, _ptr(probs), _i64(n), _i64(k), _u64(seed),
                                         _ptr(replay), _ptr(out_data), _ptr(out_index), _ptr(ws),
                                         ctypes.c_size_t(ws.numel()), _stream(dev)),
           "gs_list_sample_weighted")
    return out_data, out_index


# ---------------------------------------------------------- unique/relabel ----
class _Span(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("n", ctypes.c_int64)]


NARROW_IDS = 0x100  # GS_NARROW_IDS: 64-bit ids that fit 32 bits, on one-word table slots


def unique_relabel(mapping, queries, mailbox=None, last_span_len=None, narrow=False):
    """gs_unique_relabel[_notify].  mapping / queries: lists of 1-D id tensors (one dtype).

    Returns (frontier_buf, num_unique_dev, [relabelled query tensors]); frontier_buf has
    capacity sum(len(mapping)) and num_unique_dev is a 1-element int64 device tensor.  With a
    Mailbox the ticket to wait on is appended."""
    dev = mapping[0].device
    idb = _ids(mapping[0], "mapping[0]") | (NARROW_IDS if narrow else 0)
    for i, t in enumerate(list(mapping[1:]) + list(queries)):
        _ids(t, "relabel tensor %d" % (i + 1), like=mapping[0])
    M = sum(int(t.numel()) for t in mapping)
    frontier = torch.empty(M, dtype=mapping[0].dtype, device=dev)
    num_unique = torch.empty(1, dtype=torch.int64, device=dev)
    outs = [torch.empty_like(q) for q in queries]
    MapArr = _Span * max(len(mapping), 1)
    QArr = _Span * max(len(queries), 1)
    OutArr = ctypes.c_void_p * max(len(queries), 1)
    m_arr = MapArr(*[_Span(t.data_ptr(), t.numel()) for t in mapping])
    q_arr = QArr(*[_Span(t.data_ptr(), t.numel()) for t in queries]) if queries else QArr()
    o_arr = OutArr(*[t.data_ptr() for t in outs]) if queries else OutArr()
    ws = workspace(lib().gs_unique_workspace_bytes(_i64(M)), dev)
    if mailbox is not None or last_span_len is not None:
        # last_span_len: 1-element int64 device tensor holding the true length of mapping[-1]
        ticket = mailbox.ticket() if mailbox is not None else 0
        _check(lib().gs_unique_relabel_notify(m_arr, len(mapping), q_arr, o_arr, len(queries), idb,
                                              _ptr(frontier), _ptr(num_unique), _ptr(ws),
                                              ctypes.c_size_t(ws.numel()), _ptr(last_span_len),
                                              mailbox.ptr() if mailbox is not None
                                              else ctypes.c_void_p(0),
                                              _i64(ticket), _stream(dev)),
               "gs_unique_relabel_notify")
        return frontier, num_unique, outs, ticket
    _check(lib().gs_unique_relabel(m_arr, len(mapping), q_arr, o_arr, len(queries), idb,
                                   _ptr(frontier), _ptr(num_unique), _ptr(ws),
                                   ctypes.c_size_t(ws.numel()), _stream(dev)), "gs_unique_relabel")
    return frontier, num_unique, outs


RELABEL_REGIONS = 0x200
RELABEL_BINS = 0x400


def batch_csr_relabel(seeds, seeds_ptr, ids, ids_ptr, mailbox=None, narrow=False, path=None):
    """gs_batch_csr_relabel.  Returns (unique_buf, unique_ptr, relabelled ids, num_unique_dev
    [, ticket]); unique_buf has the capacity len(seeds) + len(ids).  path: None (the library
    chooses), "bins" or "regions"."""
    idb = _ids(seeds, "seeds") | (NARROW_IDS if narrow else 0)
    idb |= {None: 0, "bins": RELABEL_BINS, "regions": RELABEL_REGIONS}[path]
    _ids(ids, "ids", like=seeds)
    _need(seeds_ptr, torch.int64, "seeds_ptr")
    _need(ids_ptr, torch.int64, "ids_ptr")
    dev = seeds.device
    B = seeds_ptr.numel() - 1
    M = seeds.numel() + ids.numel()
    unique = torch.empty(M, dtype=seeds.dtype, device=dev)
    unique_ptr = torch.empty(B + 1, dtype=torch.int64, device=dev)
    out_ids = torch.empty_like(ids)
    num_unique = torch.empty(1, dtype=torch.int64, device=dev)
    ws = workspace(lib().gs_batch_relabel_workspace_bytes(_i64(M)), dev)
    ticket = mailbox.ticket() if mailbox is not None else 0
    _check(lib().gs_batch_csr_relabel(_ptr(seeds), _ptr(seeds_ptr), _ptr(ids), _ptr(ids_ptr), _i64(B),
                                      _i64(seeds.numel()), _i64(ids.numel()), idb, _ptr(unique),
                                      _ptr(unique_ptr), _ptr(out_ids), _ptr(num_unique), _ptr(ws),
                                      ctypes.c_size_t(ws.numel()),
                                      mailbox.ptr() if mailbox is not None else ctypes.c_void_p(0),
                                      _i64(ticket), _stream(dev)), "gs_batch_csr_relabel")
    if mailbox is not None:
        return unique, unique_ptr, out_ids, num_unique, ticket
    return unique, unique_ptr, out_ids, num_unique


def batch_coo_relabel(seeds, seeds_ptr, coo_row, coo_col, coo_ptr, narrow=False):
    """gs_batch_coo_relabel.  Returns (unique_buf, unique_ptr, out_row, out_col, num_unique_dev)."""
    idb = _ids(seeds, "seeds") | (NARROW_IDS if narrow else 0)
    _ids(coo_row, "coo_row", like=seeds)
    _ids(coo_col, "coo_col", like=seeds)
    _need(seeds_ptr, torch.int64, "seeds_ptr")
    _need(coo_ptr, torch.int64, "coo_ptr")
    dev = seeds.device
    B = seeds_ptr.numel() - 1
    M = seeds.numel() + coo_row.numel()
    unique = torch.empty(M, dtype=seeds.dtype, device=dev)
    unique_ptr = torch.empty(B + 1, dtype=torch.int64, device=dev)
    out_row, out_col = torch.empty_like(coo_row), torch.empty_like(coo_col)
    num_unique = torch.empty(1, dtype=torch.int64, device=dev)
    ws = workspace(lib().gs_batch_relabel_workspace_bytes(_i64(M)), dev)
    _check(lib().gs_batch_coo_relabel(_ptr(seeds), _ptr(seeds_ptr), _ptr(coo_row), _ptr(coo_col),
                                      _ptr(coo_ptr), _i64(B), _i64(seeds.numel()),
                                      _i64(coo_row.numel()), idb, _ptr(unique), _ptr(unique_ptr),
                                      _ptr(out_row), _ptr(out_col), _ptr(num_unique), _ptr(ws),
                                      ctypes.c_size_t(ws.numel()), ctypes.c_void_p(0), _i64(0),
                                      _stream(dev)), "gs_batch_coo_relabel")
    return unique, unique_ptr, out_row, out_col, num_unique


# ------------------------------------------------------- super-batch helpers ----
def batch_encode(data, ptr, encoding_size):
    idb = _ids(data, "data")
    _need(ptr, torch.int64, "ptr")
    out = torch.empty_like(data)
    _check(lib().gs_batch_encode(_ptr(data), idb, _i64(data.numel()), _ptr(ptr),
                                 _i64(ptr.numel() - 1), _i64(encoding_size), _ptr(out),
                                 _stream(data.device)), "gs_batch_encode")
    return out


def batch_decode(data, encoding_size):
    """Returns (decoded ids, batch numbers)."""
    idb = _ids(data, "data")
    out, batch = torch.empty_like(data), torch.empty_like(data)
    _check(lib().gs_batch_decode(_ptr(data), idb, _i64(data.numel()), _i64(encoding_size),
                                 _ptr(out), _ptr(batch), _stream(data.device)), "gs_batch_decode")
    return out, batch


def batch_offsets(data, num_batches, encoding_size):
    """Returns (offsets [num_batches+1], decoded ids) of encoded data sorted by batch."""
    idb = _ids(data, "data")
    ptr = torch.empty(num_batches + 1, dtype=torch.int64, device=data.device)
    out = torch.empty_like(data)
    _check(lib().gs_batch_offsets(_ptr(data), idb, _i64(data.numel()), _i64(num_batches),
                                  _i64(encoding_size), _ptr(ptr), _ptr(out), _stream(data.device)),
           "gs_batch_offsets")
    return ptr, out


def _ptr_array(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def batch_concat(datas, ptrs):
    """gs_batch_concat_{offsets,fill}.  Returns (total, key, total_ptr)."""
    idb = _ids(datas[0], "data")
    for d in datas:
        _ids(d, "data", like=datas[0])
    for p in ptrs:
        _need(p, torch.int64, "offsets")
    dev = datas[0].device
    B = ptrs[0].numel() - 1
    total_ptr = torch.empty(B + 1, dtype=torch.int64, device=dev)
    st = _stream(dev)
    _check(lib().gs_batch_concat_offsets(_ptr_array(ptrs), len(ptrs), _i64(B), _ptr(total_ptr), st),
           "gs_batch_concat_offsets")
    total = sum(int(d.numel()) for d in datas)
    out = torch.empty(total, dtype=datas[0].dtype, device=dev)
    key = torch.empty(total, dtype=datas[0].dtype, device=dev)
    _check(lib().gs_batch_concat_fill(_ptr_array(datas), _ptr_array(ptrs), len(ptrs), _i64(B),
                                      _i64(max(int(d.numel()) for d in datas)), idb,
                                      _ptr(total_ptr), _ptr(out), _ptr(key), st),
           "gs_batch_concat_fill")
    return out, key, total_ptr


def batch_split(data, data_ptr, data_key, out_ptrs):
    """gs_batch_split.  out_ptrs: offsets of every segment; returns the filled segments."""
    idb = _ids(data, "data")
    _need(data_ptr, torch.int64, "data_ptr")
    dev = data.device
    host = [int(p[-1].item()) for p in out_ptrs]
    outs = [torch.empty(n, dtype=data.dtype, device=dev) for n in host]
    _check(lib().gs_batch_split(_ptr(data), _ptr(data_ptr), _ptr(data_key), idb, _i64(data.numel()),
                                _i64(data_ptr.numel() - 1), _ptr_array(outs), _ptr_array(out_ptrs),
                                len(outs), _stream(dev)), "gs_batch_split")
    return outs


def coo_filter(key, row, col, ids, key_ptr=None, ids_ptr=None):
    """gs_coo_filter_{mark,compact}.  Returns (row, col, batch offsets | None, select_index)."""
    idb = _ids(key, "key")
    for t in (row, col, ids):
        _ids(t, "ids", like=key)
    dev = key.device
    E, n = key.numel(), ids.numel()
    B = 0 if key_ptr is None else key_ptr.numel() - 1
    num_kept = torch.empty(1, dtype=torch.int64, device=dev)
    ws = workspace(lib().gs_row_slice_workspace_bytes(_i64(n), _i64(E), _i64(0)), dev)
    st = _stream(dev)
    _check(lib().gs_coo_filter_mark(_ptr(key), idb, _i64(E), _ptr(key_ptr), _ptr(ids), _i64(n),
                                    _ptr(ids_ptr), _i64(B), _ptr(num_kept), _ptr(ws),
                                    ctypes.c_size_t(ws.numel()), st), "gs_coo_filter_mark")
    kept = _total(num_kept, 0)
    out_row = torch.empty(kept, dtype=key.dtype, device=dev)
    out_col = torch.empty(kept, dtype=key.dtype, device=dev)
    select_index = torch.empty(kept, dtype=torch.int64, device=dev)
    out_ptr = torch.empty(B + 1, dtype=torch.int64, device=dev) if B else None
    _check(lib().gs_coo_filter_compact(_ptr(row), _ptr(col), idb, _i64(E), _ptr(key_ptr), _i64(B),
                                       _ptr(out_row), _ptr(out_col), _ptr(select_index),
                                       _ptr(out_ptr), _ptr(ws), ctypes.c_size_t(ws.numel()), st),
           "gs_coo_filter_compact")
    return out_row, out_col, out_ptr, select_index


def index_search(data, keys):
    idb = _ids(data, "data")
    _ids(keys, "keys", like=data)
    out = torch.empty_like(keys)
    ws = workspace(lib().gs_index_search_workspace_bytes(_i64(data.numel())), data.device)
    _check(lib().gs_index_search(_ptr(data), _i64(data.numel()), _ptr(keys), _i64(keys.numel()), idb,
                                 _ptr(out), _ptr(ws), ctypes.c_size_t(ws.numel()),
                                 _stream(data.device)), "gs_index_search")
    return out


# ------------------------------------------------- layer-wise sampler tail ----
def sorted_union_max(id_bytes):
    return int(lib().gs_sorted_union_max(int(id_bytes)))


def sorted_union(a, b):
    """gs_sorted_union.  Returns (out with room for len(a) + len(b), count: device int64[1])."""
    idb = _ids(a, "a")
    _ids(b, "b", like=a)
    out = torch.empty(a.numel() + b.numel(), dtype=a.dtype, device=a.device)
    count = torch.empty(1, dtype=torch.int64, device=a.device)
    _check(lib().gs_sorted_union(_ptr(a), _i64(a.numel()), _ptr(b), _i64(b.numel()), idb, _ptr(out),
                                 _ptr(count), _stream(a.device)), "gs_sorted_union")
    return out, count


_boxes = {}


def _total(values, at):
    """values[at] read back through a mailbox (gs_post_total) instead of a blocking copy."""
    box = _boxes.get(values.device)
    if box is None:
        box = _boxes[values.device] = Mailbox()
    return post_total(values, at, box)


def post_total(values, at, box):
    """gs_post_total: values[at] (device int64) through the mailbox `box`; returns it."""
    _need(values, torch.int64, "values")
    ticket = box.ticket()
    _check(lib().gs_post_total(ctypes.c_void_p(values.data_ptr() + 8 * int(at)), box.ptr(),
                               _i64(ticket), _stream(values.device)), "gs_post_total")
    return box.wait(ticket, values.device)


def post_values(values, box):
    """gs_post_values: a device int64 array to pinned host memory; returns the pinned tensor once
    the mailbox says it has landed."""
    _need(values, torch.int64, "values")
    out = torch.empty(values.numel(), dtype=torch.int64).pin_memory()
    ticket = box.ticket()
    _check(lib().gs_post_values(_ptr(values), _i64(values.numel()),
                                ctypes.c_void_p(out.data_ptr()), box.ptr(), _i64(ticket),
                                _stream(values.device)), "gs_post_values")
    got = box.wait(ticket, values.device)
    if got != values.numel():
        raise GsError("gs_post_values posted %d values, expected %d" % (got, values.numel()))
    return out


def post_value_sets(sets, box):
    """gs_post_value_sets: several device int64 arrays of one length to pinned host memory by
    one launch; returns a pinned [len(sets), n] tensor once the mailbox says it has landed."""
    n = sets[0].numel() if sets else 0
    for t in sets:
        _need(t, torch.int64, "values")
        if t.numel() != n:
            raise ValueError("the arrays must have one length")
    out = torch.empty((len(sets), n), dtype=torch.int64).pin_memory()
    at = (ctypes.c_void_p * max(len(sets), 1))(*[t.data_ptr() for t in sets])
    ticket = box.ticket()
    dev = sets[0].device if sets else torch.device("cuda", torch.cuda.current_device())
    _check(lib().gs_post_value_sets(at, len(sets), _i64(n), ctypes.c_void_p(out.data_ptr()),
                                    box.ptr(), _i64(ticket), _stream(dev)), "gs_post_value_sets")
    got = box.wait(ticket, dev)
    if got != len(sets) * n:
        raise GsError("gs_post_value_sets posted %d values, expected %d" % (got, len(sets) * n))
    return out


def indptr_split(indptr, offsets, with_cuts=False):
    """gs_indptr_split / gs_indptr_split_cuts: the batches' offsets re-based and laid out back to
    back; with_cuts also returns indptr[offsets] from the same launch."""
    _need(indptr, torch.int64, "indptr")
    _need(offsets, torch.int64, "offsets")
    B = offsets.numel() - 1
    span = int(offsets[-1] - offsets[0]) if B >= 1 else 0
    total = span + B
    out = torch.empty(total, dtype=torch.int64, device=indptr.device)
    if not with_cuts:
        _check(lib().gs_indptr_split(_ptr(indptr), _ptr(offsets), _i64(B), _i64(total), _ptr(out),
                                     _stream(indptr.device)), "gs_indptr_split")
        return out
    cuts = torch.empty(B + 1, dtype=torch.int64, device=indptr.device)
    _check(lib().gs_indptr_split_cuts(_ptr(indptr), _ptr(offsets), _i64(B), _i64(total), _ptr(out),
                                      _ptr(cuts), _stream(indptr.device)), "gs_indptr_split_cuts")
    return out, cuts


def coo_pick_rows(row, col, nodes, count, max_nodes, box=None):
    """gs_coo_pick_rows.  Returns (kept_key, kept_pos, totals: device int64[2]); with a
    mailbox `box` the number of kept edges is waited for and returned as a fourth value."""
    idb = _ids(row, "row")
    _ids(col, "col", like=row)
    _ids(nodes, "nodes", like=row)
    _need(count, torch.int64, "count")
    E = row.numel()
    key = torch.empty(E, dtype=row.dtype, device=row.device)
    pos = torch.empty(E, dtype=row.dtype, device=row.device)
    totals = torch.empty(2, dtype=torch.int64, device=row.device)
    ws = workspace(lib().gs_coo_pick_rows_workspace_bytes(_i64(E)), row.device)
    ticket = box.ticket() if box is not None else 0
    _check(lib().gs_coo_pick_rows(_ptr(row), _ptr(col), idb, _i64(E), _ptr(nodes), _ptr(count),
                                  _i64(max_nodes), _ptr(key), _ptr(pos), _ptr(totals),
                                  box.ptr() if box is not None else ctypes.c_void_p(0),
                                  _i64(ticket), _ptr(ws),
                                  ctypes.c_size_t(ws.numel()), _stream(row.device)),
           "gs_coo_pick_rows")
    if box is not None:
        return key, pos, totals, box.wait(ticket, row.device)
    return key, pos, totals


def coo_block_values(kept_key, kept_pos, max_nodes, row, data, divisor, num_cols):
    """gs_coo_block_values.  Returns (out_row, out_value, out_indptr)."""
    idb = _ids(row, "row")
    _ids(kept_key, "kept_key", like=row)
    _ids(kept_pos, "kept_pos", like=row)
    _need(divisor, torch.float32, "divisor")
    if data is not None:
        _need(data, torch.float32, "data")
    kept = kept_key.numel()
    out_row = torch.empty(kept, dtype=row.dtype, device=row.device)
    out_value = torch.empty(kept, dtype=torch.float32, device=row.device)
    out_indptr = torch.empty(num_cols + 1, dtype=torch.int64, device=row.device)
    ws = workspace(lib().gs_coo_block_values_workspace_bytes(_i64(kept)), row.device)
    _check(lib().gs_coo_block_values(_ptr(kept_key), _ptr(kept_pos), _i64(kept), _i64(max_nodes),
                                     _ptr(row), idb, _ptr(data), _ptr(divisor), _i64(num_cols),
                                     _ptr(out_row), _ptr(out_value), _ptr(out_indptr), _ptr(ws),
                                     ctypes.c_size_t(ws.numel()), _stream(row.device)),
           "gs_coo_block_values")
    return out_row, out_value, out_indptr


# ------------------------------------------------------------------ walks ----
def random_walk(indptr, indices, seeds, length, seed=0, replay=None):
    _need(indptr, torch.int64, "indptr")
    idb = _ids(indices, "indices")
    _ids(seeds, "seeds", like=indices)
    dev = indptr.device
    n = seeds.numel()
    trace = torch.empty((int(length) + 1) * n, dtype=indices.dtype, device=dev)
    _check(lib().gs_random_walk(_ptr(indptr), _i64(indptr.numel() - 1), _ptr(indices), idb, _ptr(seeds), _i64(n), _i64(length),
                                _u64(seed), _ptr(replay), _ptr(trace), _stream(dev)),
           "gs_random_walk")
    return trace


def metapath_walk(indptr_table, indices_table, num_nodes_table, id_dtype, metapath, seeds, seed=0,
                  replay=None):
    """indptr_table / indices_table: device int64 tensors holding device addresses;
    num_nodes_table: device int64 tensor, columns per relation."""
    _need(num_nodes_table, torch.int64, "num_nodes_table")
    _need(metapath, torch.int64, "metapath")
    idb = _ids(seeds, "seeds")
    if seeds.dtype != id_dtype:
        raise GsError("seeds must have the dtype of the relation graphs' ids")
    dev = seeds.device
    n = seeds.numel()
    L = metapath.numel()
    trace = torch.empty((L + 1) * n, dtype=seeds.dtype, device=dev)
    _check(lib().gs_metapath_walk(_ptr(indptr_table), _ptr(indices_table), _ptr(num_nodes_table), idb, _ptr(metapath),
                                  _i64(L), _ptr(seeds), _i64(n), _u64(seed), _ptr(replay),
                                  _ptr(trace), _stream(dev)), "gs_metapath_walk")
    return trace


# ------------------------------------------------------------------ SDDMM ----
OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "copy_lhs": 4, "copy_rhs": 5, "dot": 6}


def sddmm_coo(op, row, col, e_ids, lhs, rhs, out, lhs_target, rhs_target, lhs_len, rhs_len,
              out_len, reduce_size, lhs_off=None, rhs_off=None):
    if op not in OPS:
        raise GsError("Unsupported SpMM/SDDMM binary operator: %s" % op)
    idb = _ids(row, "row")
    _ids(col, "col", like=row)
    _need(out, torch.float32, "out")
    dev = row.device
    _check(lib().gs_sddmm_coo(OPS[op], _ptr(row), _ptr(col), idb, _ptr(e_ids), _i64(row.numel()),
                              _ptr(lhs), _ptr(rhs), _ptr(out), int(lhs_target), int(rhs_target),
                              _i64(lhs_len), _i64(rhs_len), _i64(out_len), _i64(reduce_size),
                              _ptr(lhs_off), _ptr(rhs_off), _stream(dev)), "gs_sddmm_coo")


def sddmm_csc(op, indptr, indices, e_ids, nid_map, lhs, rhs, out, lhs_target, rhs_target, lhs_len,
              rhs_len, out_len, reduce_size, lhs_off=None, rhs_off=None):
    if op not in OPS:
        raise GsError("Unsupported SpMM/SDDMM binary operator: %s" % op)
    _need(indptr, torch.int64, "indptr")
    idb = _ids(indices, "indices")
    if nid_map is not None:
        _ids(nid_map, "nid_map", like=indices)
    _need(out, torch.float32, "out")
    dev = indptr.device
    _check(lib().gs_sddmm_csc(OPS[op], _ptr(indptr), _ptr(indices), idb, _ptr(e_ids), _ptr(nid_map),
                              _i64(indptr.numel() - 1), _i64(indices.numel()), _ptr(lhs), _ptr(rhs),
                              _ptr(out), int(lhs_target), int(rhs_target), _i64(lhs_len),
                              _i64(rhs_len), _i64(out_len), _i64(reduce_size), _ptr(lhs_off),
                              _ptr(rhs_off), _stream(dev)), "gs_sddmm_csc")


def segment_sum(indptr, e_ids, n_ids, data, powk, out):
    _need(indptr, torch.int64, "indptr")
    _need(data, torch.float32, "data")
    _need(out, torch.float32, "out")
    idb = _ids(n_ids, "n_ids") if n_ids is not None else 8
    nseg = indptr.numel() - 1
    nnz = e_ids.numel() if e_ids is not None else data.numel()
    ws = workspace(lib().gs_segment_workspace_bytes(_i64(nseg), _i64(nnz)), indptr.device)
    _check(lib().gs_segment_sum(_ptr(indptr), _ptr(e_ids), _ptr(n_ids), idb, _ptr(data),
                                _i64(nseg), _i64(nnz), _i64(powk), _ptr(out), _ptr(ws),
                                ctypes.c_size_t(ws.numel()), _stream(indptr.device)),
           "gs_segment_sum")


def coo_sum(target, e_ids, data, powk, out):
    idb = _ids(target, "target")
    _need(data, torch.float32, "data")
    _need(out, torch.float32, "out")
    _check(lib().gs_coo_sum(_ptr(target), idb, _ptr(e_ids), _ptr(data), _i64(target.numel()),
                            _i64(powk), _ptr(out), _stream(target.device)), "gs_coo_sum")


def coo_sum_binned(target, e_ids, data, powk, out):
    """`coo_sum` through the entry point that knows the number of targets (`out.numel()`) and
    brings a workspace: large inputs are binned by target and added up without atomics."""
    idb = _ids(target, "target")
    _need(data, torch.float32, "data")
    _need(out, torch.float32, "out")
    L = lib()
    ws = workspace(L.gs_coo_sum_workspace_bytes(_i64(target.numel()), _i64(out.numel())),
                   target.device)
    _check(L.gs_coo_sum_binned(_ptr(target), idb, _ptr(e_ids), _ptr(data), _i64(target.numel()),
                               _i64(powk), _i64(out.numel()), _ptr(out), _ptr(ws),
                               ctypes.c_size_t(ws.numel()), _stream(target.device)),
           "gs_coo_sum_binned")


def segment_normalize(indptr, e_ids, data, out):
    _need(indptr, torch.int64, "indptr")
    _need(data, torch.float32, "data")
    _need(out, torch.float32, "out")
    nseg = indptr.numel() - 1
    nnz = e_ids.numel() if e_ids is not None else data.numel()
    ws = workspace(lib().gs_segment_workspace_bytes(_i64(nseg), _i64(nnz)), indptr.device)
    _check(lib().gs_segment_normalize(_ptr(indptr), _ptr(e_ids), _ptr(data), _i64(nseg), _i64(nnz),
                                      _ptr(out), _ptr(ws), ctypes.c_size_t(ws.numel()),
                                      _stream(indptr.device)), "gs_segment_normalize")


def e_div_u_sum(row, col, data, divisor, out_data, out_sum):
    idb = _ids(row, "row")
    _ids(col, "col", like=row)
    _need(data, torch.float32, "data")
    _need(divisor, torch.float32, "divisor")
    _check(lib().gs_e_div_u_sum(_ptr(row), _ptr(col), idb, _ptr(data), _ptr(divisor),
                                _i64(row.numel()), _ptr(out_data), _ptr(out_sum),
                                _stream(row.device)), "gs_e_div_u_sum")


# ------------------------------------------------------------ row slicing ----
def row_slice_csc(indptr, indices, row_ids, with_coo):
    """Two-phase gs_row_slice_csc_*; returns (out_indptr, coo_col|None, out_indices, select_index)."""
    _need(indptr, torch.int64, "indptr")
    idb = _ids(indices, "indices")
    _ids(row_ids, "row_ids", like=indices)
    dev = indptr.device
    ncols, nnz, nr = indptr.numel() - 1, indices.numel(), row_ids.numel()
    out_indptr = torch.empty(ncols + 1, dtype=torch.int64, device=dev)
    ws = workspace(lib().gs_row_slice_workspace_bytes(_i64(nr), _i64(nnz), _i64(ncols)), dev)
    st = _stream(dev)
    _check(lib().gs_row_slice_csc_mark(_ptr(indptr), _ptr(indices), idb, _i64(ncols), _i64(nnz),
                                       _ptr(row_ids), _i64(nr), _ptr(out_indptr), _ptr(ws),
                                       ctypes.c_size_t(ws.numel()), st), "gs_row_slice_csc_mark")
    kept = _total(out_indptr, out_indptr.numel() - 1)
    out_indices = torch.empty(kept, dtype=indices.dtype, device=dev)
    select_index = torch.empty(kept, dtype=torch.int64, device=dev)
    coo_col = torch.empty(kept, dtype=indices.dtype, device=dev) if with_coo else None
    if kept == 0:
        return out_indptr, coo_col, out_indices, select_index
    _check(lib().gs_row_slice_csc_compact(_ptr(indptr), _i64(ncols), _i64(nnz), idb,
                                          _ptr(out_indices), _ptr(select_index), _ptr(coo_col),
                                          _ptr(ws), ctypes.c_size_t(ws.numel()), st),
           "gs_row_slice_csc_compact")
    return out_indptr, coo_col, out_indices, select_index


def row_slice_coo(key, other, ids):
    """Two-phase gs_row_slice_coo_*; returns (relabelled key, other, select_index)."""
    idb = _ids(key, "key")
    _ids(other, "other", like=key)
    _ids(ids, "ids", like=key)
    dev = key.device
    E, n = key.numel(), ids.numel()
    num_kept = torch.empty(1, dtype=torch.int64, device=dev)
    ws = workspace(lib().gs_row_slice_workspace_bytes(_i64(n), _i64(E), _i64(0)), dev)
    st = _stream(dev)
    _check(lib().gs_row_slice_coo_mark(_ptr(key), idb, _i64(E), _ptr(ids), _i64(n), _ptr(num_kept),
                                       _ptr(ws), ctypes.c_size_t(ws.numel()), st),
           "gs_row_slice_coo_mark")
    kept = _total(num_kept, 0)
    out_key = torch.empty(kept, dtype=key.dtype, device=dev)
    out_other = torch.empty(kept, dtype=key.dtype, device=dev)
    select_index = torch.empty(kept, dtype=torch.int64, device=dev)
    if kept == 0:
        return out_key, out_other, select_index
    _check(lib().gs_row_slice_coo_compact(_ptr(other), idb, _i64(E), _ptr(out_key),
                                          _ptr(out_other), _ptr(select_index), _ptr(ws),
                                          ctypes.c_size_t(ws.numel()), st), "gs_row_slice_coo_compact")
    return out_key, out_other, select_index


def col_row_slice(indptr, indices, column_ids, row_ids, col_ptr=None, row_ptr=None,
                  encoding_size=0):
    """gs_slice_count + gs_col_row_slice_{mark,compact}; returns (out_indptr, out_indices,
    select_index (position in the virtual column slice), parent_index (position in indices))."""
    _need(indptr, torch.int64, "indptr")
    idb = _ids(indices, "indices")
    _ids(column_ids, "column_ids", like=indices)
    _ids(row_ids, "row_ids", like=indices)
    dev = indptr.device
    S, nr = column_ids.numel(), row_ids.numel()
    B = 0
    if col_ptr is not None:
        _need(col_ptr, torch.int64, "col_ptr")
        _need(row_ptr, torch.int64, "row_ptr")
        B = col_ptr.numel() - 1
    sub_indptr = slice_count(indptr, column_ids)
    D = _total(sub_indptr, sub_indptr.numel() - 1)
    out_indptr = torch.empty(S + 1, dtype=torch.int64, device=dev)
    ws = workspace(lib().gs_col_row_slice_workspace_bytes(_i64(nr), _i64(D)), dev)
    st = _stream(dev)
    _check(lib().gs_col_row_slice_mark(_ptr(indptr), _i64(indptr.numel() - 1), _ptr(indices), idb,
                                       _ptr(column_ids), _i64(S), _ptr(sub_indptr), _i64(D),
                                       _ptr(row_ids), _i64(nr), _ptr(col_ptr), _ptr(row_ptr),
                                       _i64(B), _i64(encoding_size), _ptr(out_indptr), _ptr(ws),
                                       ctypes.c_size_t(ws.numel()), st), "gs_col_row_slice_mark")
    kept = _total(out_indptr, out_indptr.numel() - 1)
    out_indices = torch.empty(kept, dtype=indices.dtype, device=dev)
    select_index = torch.empty(kept, dtype=torch.int64, device=dev)
    parent_index = torch.empty(kept, dtype=torch.int64, device=dev)
    if kept > 0:
        _check(lib().gs_col_row_slice_compact(_i64(D), idb, _ptr(out_indices), _ptr(select_index),
                                              _ptr(parent_index), _ptr(ws),
                                              ctypes.c_size_t(ws.numel()), st),
               "gs_col_row_slice_compact")
    return out_indptr, out_indices, select_index, parent_index


# ------------------------------------------------------- format transform ----
def csc2coo(indptr, nnz, id_dtype=torch.int64):
    _need(indptr, torch.int64, "indptr")
    col = torch.empty(nnz, dtype=id_dtype, device=indptr.device)
    _check(lib().gs_csc2coo(_ptr(indptr), _i64(indptr.numel() - 1), _i64(nnz), _ptr(col),
                            _id_bytes(col), _stream(indptr.device)), "gs_csc2coo")
    return col


def dcsc2coo(indptr, nnz, ids):
    """Column of every edge of a doubly-compressed CSC: `ids[c]` for the edges of stored
    column c (`indptr` runs over the stored columns only)."""
    _need(indptr, torch.int64, "indptr")
    col = torch.empty(nnz, dtype=ids.dtype, device=indptr.device)
    _check(lib().gs_dcsc2coo(_ptr(indptr), _i64(indptr.numel() - 1), _i64(nnz), _ptr(ids),
                             _ptr(col), _id_bytes(col), _stream(indptr.device)), "gs_dcsc2coo")
    return col


def coo2csc(key, value, num_keys, is_sorted):
    """Returns (indptr, sorted value | value, perm | None)."""
    idb = _ids(key, "key")
    _ids(value, "value", like=key)
    dev = key.device
    E = key.numel()
    indptr = torch.empty(num_keys + 1, dtype=torch.int64, device=dev)
    out_value = None if is_sorted else torch.empty(E, dtype=value.dtype, device=dev)
    perm = None if is_sorted else torch.empty(E, dtype=torch.int64, device=dev)
    ws = workspace(lib().gs_coo2csc_workspace_bytes(_i64(E), _i64(num_keys)), dev)
    _check(lib().gs_coo2csc(_ptr(key), _ptr(value), idb, _i64(E), _i64(num_keys),
                            int(bool(is_sorted)), _ptr(indptr), _ptr(out_value), _ptr(perm), _ptr(ws),
                            ctypes.c_size_t(ws.numel()), _stream(dev)), "gs_coo2csc")
    return indptr, (value if is_sorted else out_value), perm
