"""Pure-Python restatement of the reference's work-partition and ring-topology rules.

TEST INFRASTRUCTURE ONLY: the product's host library implements these in C++; this module is the
checker it is compared with.  Integer arithmetic throughout, so parity is bit-exact.

Pinned by (tests/test_oracle.py): the committed fixture sweep tests/golden/partition_golden.json,
which was produced by the compiled reference Partition.cc, the compiled reference itself
(oracle/_ref/libref_partition.so) where it has been built, the spot values quoted from a run of the
reference, and tiling invariants (every cell of [0,m) x [0,n) is owned by exactly one thread).
"""


def _ceil_div(a, b):
    return -(-a // b)


def work_per_socket(work, nsockets):
    """Partition.cc:25-27."""
    return _ceil_div(work, nsockets)


def partition_1d(work, nsockets, sid, T, t):
    """1-D split of `work` items over sockets, then threads (Partition.cc:30-48)."""
    wps = work_per_socket(work, nsockets)
    socket_begin = min(sid * wps, work)
    per_thread = _ceil_div(wps, T)
    b = min(t * per_thread, wps)
    e = min(b + per_thread, wps)
    return min(socket_begin + b, work), min(socket_begin + e, work)


def _block_extent(m, n, mb, nb, m_align):
    """Rows/cols per thread block for an mb x nb thread grid (Partition.cc:95-101)."""
    bm = _ceil_div(_ceil_div(m, 16), mb) * 16 if m_align else _ceil_div(m, mb)
    bn = _ceil_div(_ceil_div(n, 16), nb) * 16
    return bm, bn


def thread_grid(m, n, aspect_ratio, m_align, T):
    """Greedy search for the mb x nb thread grid whose block shape bm/bn is closest to
    aspect_ratio; stops at the first divisor of T that does not improve (Partition.cc:92-151).
    Returns (mb, nb, bm, bn)."""
    mb, nb = 1, T
    bm, bn = _block_extent(m, n, mb, nb, m_align)
    best = abs(bm / bn - aspect_ratio)
    for cand in range(2, T + 1):
        if T % cand:
            continue
        nb_c = T // cand
        rows = _ceil_div(m, cand)
        if m_align:
            if aspect_ratio < 1 and bm == 16 and rows < 16:
                continue
            if rows <= 8:
                continue
        if _ceil_div(n, nb_c) <= 8:
            continue
        bm_c, bn_c = _block_extent(m, n, cand, nb_c, m_align)
        delta = abs(bm_c / bn_c - aspect_ratio)
        if delta < best:
            best, mb, nb, bm, bn = delta, cand, nb_c, bm_c, bn_c
        else:
            break
    return mb, nb, bm, bn


def partition_2d_intra(m, n, aspect_ratio, m_align, T, t):
    """Block [m_begin,m_end) x [n_begin,n_end) of thread t inside one socket
    (Partition.cc:75-166)."""
    _, nb, bm, bn = thread_grid(m, n, aspect_ratio, m_align, T)
    mt, nt = divmod(t, nb)
    m_begin = min(mt * bm, m)
    m_end = min(m_begin + bm, m)
    n_begin = min(nt * bn, n)
    n_end = min(n_begin + bn, n)
    return m_begin, m_end, n_begin, n_end


def partition_2d(m, n, aspect_ratio, m_align, nsockets, sid, T, t):
    """Rows split over sockets first, then the intra-socket 2-D split (Partition.cc:193-222)."""
    mps = work_per_socket(m, nsockets)
    mb, me, nb_, ne = partition_2d_intra(mps, n, aspect_ratio, m_align, T, t)
    base = min(sid * mps, m)
    return min(base + mb, m), min(base + me, m), nb_, ne


# Two counter-rotating rings over the 8 sockets of a twisted hypercube
# (mlp_bench_common.cc:13-14).
RINGS = ((0, 1, 2, 4, 7, 6, 5, 3), (0, 3, 5, 6, 7, 4, 2, 1))


def ring_info(sid, task, nsockets):
    """(idx_in_ring, prev_sid, next_sid) for socket `sid`, ring chosen by task parity
    (mlp_bench_common.cc:170-190).  With fewer than 8 sockets the ring is plain +-1 order,
    reversed for odd tasks."""
    which = task % len(RINGS)
    if nsockets < 8:
        prev_sid = (sid - 1) % nsockets
        next_sid = (sid + 1) % nsockets
        if which:
            prev_sid, next_sid = next_sid, prev_sid
        return sid, prev_sid, next_sid
    ring = RINGS[which]
    idx = ring.index(sid)
    return idx, ring[(idx - 1) % nsockets], ring[(idx + 1) % nsockets]
