"""Host-side scheduling helpers of the reference backend (binding.cpp:27,31-33,
106-119): rel_schedule, gen_edge_type_mag240m, topo_sort, and the dgSPARSE-style
GSpMM entry points, written as vectorised tensor index arithmetic."""
import enum

import torch

from . import _lib, _ops


def _rows_of_edges(ptr, n):
    return torch.repeat_interleave(torch.arange(n, device=ptr.device), ptr[1:n + 1] - ptr[:n])


def rel_schedule(csr_ptr, csr_idx, rel, num_node_in_layer, num_rel):
    """Per-relation sub-CSRs (src/cpp/src/schedule.cu:5-63).  For every relation r the
    rows that have at least one edge of type r: ptr_r, idx_r (edge order kept) and
    target_r (original row ids); then a [num_rel, L] table, L = len(num_node_in_layer)-1,
    whose entry [r, l] is the number of kept rows among the first num_node_in_layer[l]
    rows.  Returns the 3*num_rel + 1 tensors in that order, on the inputs' device
    (upstream works on CPU tensors); graphs on the GPU are handled for all relations at
    once after one stable sort by relation."""
    n = csr_ptr.shape[0] - 1
    num_rel = int(num_rel)
    if csr_ptr.is_cuda:
        return _rel_schedule_device(csr_ptr, csr_idx, rel, num_node_in_layer, num_rel, n)
    rows = _rows_of_edges(csr_ptr, n)
    e = rows.shape[0]
    idx = csr_idx[:e]
    rel = rel[:e]
    layers = [int(v) for v in num_node_in_layer.tolist()]
    num_layer = len(layers) - 1
    table = torch.zeros((num_rel, max(num_layer, 0)), dtype=torch.int64, device=csr_ptr.device)
    out = []
    for r in range(num_rel):
        m = rel == r
        cnt = torch.bincount(rows[m], minlength=n)
        keep = cnt > 0
        target = torch.nonzero(keep).flatten()
        sub_ptr = torch.cat([cnt.new_zeros(1), torch.cumsum(cnt[keep], 0)])
        out += [sub_ptr, idx[m], target]
        kept_before = torch.cumsum(keep.to(torch.int64), 0)
        # upstream walks rows in order and records layer l when it reaches row
        # num_node_in_layer[l]-1; a boundary that lies behind the walk is never met
        pos = -1
        for l in range(num_layer):
            i = layers[l] - 1
            if i <= pos or i >= n:
                break
            table[r, l] = kept_before[i]
            pos = i
    out.append(table)
    return out


def _rel_schedule_device(csr_ptr, csr_idx, rel, num_node_in_layer, num_rel, n):
    layers = [int(v) for v in num_node_in_layer.tolist()]
    num_layer = len(layers) - 1
    # upstream walks rows in order and records layer l when it reaches row
    # num_node_in_layer[l]-1; a boundary that lies behind the walk is never met
    reached, pos = [], -1
    for l in range(num_layer):
        i = layers[l] - 1
        if i <= pos or i >= n:
            break
        reached.append(i + 1)
        pos = i
    dev = csr_ptr.device
    table = torch.zeros((num_rel, max(num_layer, 0)), dtype=torch.int64, device=dev)
    e = int(csr_ptr[n].item()) if n > 0 else 0
    if e == 0:
        empty = torch.zeros(0, dtype=torch.int64, device=dev)
        out = []
        for r in range(num_rel):
            out += [torch.zeros(1, dtype=torch.int64, device=dev), empty, empty]
        out.append(table)
        return out
    # All relations at once.  A stable sort by relation keeps each relation's edges in
    # their original (row-major) order, so within a relation the rows of its edges are
    # non-decreasing: the kept rows and their edge counts are the runs of the combined
    # key relation * n + row.
    from . import _typed
    rel32 = rel[:e].to(torch.int32).contiguous()
    perm, seg = _typed.rel_segment(rel32, num_rel)
    rows = _ops.csr_row_ids(csr_ptr, n, e)
    r_rows = rows[perm]
    r_idx = csr_idx[:e][perm]
    key = rel32.to(torch.int64)[perm] * n + r_rows
    uniq, counts = torch.unique_consecutive(key, return_counts=True)
    bounds = torch.searchsorted(uniq, torch.arange(num_rel + 1, dtype=torch.int64, device=dev) * n)
    ends = torch.cat([counts.new_zeros(1), torch.cumsum(counts, 0)])
    target_all = uniq % n
    if reached:
        at = torch.tensor(reached, dtype=torch.int64, device=dev)
        q = torch.arange(num_rel, dtype=torch.int64, device=dev).unsqueeze(1) * n + at.unsqueeze(0)
        table[:, :len(reached)] = torch.searchsorted(uniq, q) - bounds[:num_rel].unsqueeze(1)
    seg_h, bounds_h = seg.tolist(), bounds.tolist()
    out = []
    for r in range(num_rel):
        e0, e1, u0, u1 = seg_h[r], seg_h[r + 1], bounds_h[r], bounds_h[r + 1]
        out += [ends[u0:u1 + 1] - e0, r_idx[e0:e1], target_all[u0:u1]]
    out.append(table)
    return out


_PAPER = 121751666
_PAPER_AUTHOR = 244134778


def gen_edge_type_mag240m(ptr, idx, sub_to_full):
    """Edge types of a MAG240M sub-graph from global id ranges
    (src/cpp/src/aggr.cu:516-566): paper<-paper 0, paper<-author 1, author<-paper 2,
    author<-institute 3, institute<-author 4."""
    n = ptr.shape[0] - 1
    rows = _rows_of_edges(ptr, n)
    e = rows.shape[0]
    center = sub_to_full[rows]
    nbr = sub_to_full[idx[:e]]

    def kind(v):
        return (v >= _PAPER).to(torch.int64) + (v >= _PAPER_AUTHOR).to(torch.int64)
    ck, nk = kind(center), kind(nbr)
    table = torch.tensor([[0, 1, -1], [2, -1, 3], [-1, 4, -1]], device=ptr.device)
    et = table[ck, nk]
    if bool((et < 0).any()):
        raise ValueError("edge between node kinds that MAG240M does not connect")
    out = torch.zeros_like(idx)
    out[:e] = et
    return out


def topo_sort(csr_ptr, csr_idx, degree):
    """Topological order of the nodes of a successor-list CSR on CPU tensors
    (src/cpp/src/schedule.cu:71-128): FIFO from the nodes with degree 0; cycles are
    broken by releasing the nodes with counter 1 and the first running-minimum node.
    Entries of nodes never reached are left uninitialised, as upstream does."""
    for t, name in ((csr_ptr, "csr_ptr"), (csr_idx, "csr_idx"), (degree, "degree")):
        if t.is_cuda or t.dtype != torch.int64 or t.dim() != 1:
            raise ValueError("%s must be a 1-D int64 CPU tensor" % name)
    n = degree.shape[0]
    if csr_ptr.shape[0] < n + 1:
        raise ValueError("csr_ptr needs %d entries" % (n + 1))
    ptr, idx, deg = csr_ptr.contiguous(), csr_idx.contiguous(), degree.contiguous()
    n_edges = int(ptr[n]) if n else 0
    if n_edges > idx.shape[0] or (n_edges and (int(idx[:n_edges].min()) < 0 or int(idx[:n_edges].max()) >= n)):
        raise ValueError("csr_idx does not match csr_ptr / the number of nodes")
    out = torch.empty(n, dtype=torch.int64)
    cnt = _lib.load().cxg_topo_sort_host_i64(ptr.data_ptr(), idx.data_ptr(), deg.data_ptr(), n, out.data_ptr())
    if cnt < 0:
        _lib.check(int(cnt))
    if cnt != n:
        print("Error: graph is not a DAG, %d %d" % (cnt, n))
    return out


class REDUCEOP(enum.IntEnum):
    SUM = 0
    MAX = 1
    MIN = 2
    MEAN = 3


class COMPUTEOP(enum.IntEnum):
    """Names in the order the reference exports them (binding.cpp:114-119), values
    of its C enum (dgsparse.h:14)."""
    ADD = 0
    MUL = 2
    DIV = 3
    SUB = 1


def _gspmm(rowptr, colind, val, b, red, comp):
    lib = _lib.load()
    for t, name in ((rowptr, "A_rowptr"), (colind, "A_colind")):
        _ops._req(t, name, torch.int32, 1)
    _ops._req(b, "B", torch.float32, 2)
    n = rowptr.shape[0] - 1
    if val is not None:
        _ops._req(val, "A_csrVal", torch.float32, 1)
        if val.shape[0] < colind.shape[0]:
            raise ValueError("A_csrVal shorter than A_colind")
    out = torch.empty((n, b.shape[1]), dtype=torch.float32, device=b.device)
    ws_bytes = lib.cxg_gspmm_workspace_bytes(colind.shape[0], b.shape[1])
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=b.device) if ws_bytes else None
    with torch.cuda.device(b.device):
        st = lib.cxg_gspmm_i32_f32(rowptr.data_ptr(), _lib.ptr(colind), _lib.ptr(val), _lib.ptr(b), _lib.ptr(out),
                                   n, colind.shape[0], b.shape[1], int(red), int(comp), _lib.ptr(ws), ws_bytes,
                                   _lib.current_stream(b.device))
    _lib.check(st)
    return out


def GSpMM_u(A_rowptr, A_colind, B, op):
    """int32-CSR SpMM without edge values (binding.cpp:97-104): sum / max / min / mean of
    the gathered rows; empty rows give 0."""
    op = REDUCEOP(int(op))
    if A_rowptr.dtype != torch.int32 or A_colind.dtype != torch.int32:
        raise ValueError("GSpMM_u takes int32 rowptr/colind")
    if op in (REDUCEOP.SUM, REDUCEOP.MEAN):
        return _ops.spmm(A_rowptr, A_colind, B, A_rowptr.shape[0] - 1, mean=(op == REDUCEOP.MEAN))
    return _gspmm(A_rowptr, A_colind, None, B, op, COMPUTEOP.MUL)


def GSpMM_u_e(A_rowptr, A_colind, A_csrVal, B, re_op, comp_op):
    """int32-CSR SpMM with edge values (binding.cpp:86-95):
    out[r] = REDUCE_e COMPUTE(val[e], B[col[e]]) with COMPUTE add val+b, sub b-val,
    mul val*b, div b/val (dgsparse.h:53-79)."""
    return _gspmm(A_rowptr, A_colind, A_csrVal, B, REDUCEOP(int(re_op)), COMPUTEOP(int(comp_op)))
