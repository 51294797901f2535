"""TEST INFRASTRUCTURE — numpy model of the device-side plan construction (bpt_amd/csrc/bptplan.hip).

Launch plans and row groups are this library's own construct (the reference has no counterpart: its kernels take
the CSR arrays of graph/base.py:71-86 as they are), so what pins them is (1) the structural invariants every plan
must satisfy (each item in one group, each edge one pair, masks / pair numbers / edge ids consistent), (2) a numpy
emulation of the kernels' walk over the plan against the oracle, and (3) for the base plan, equality with the host
builder (bptg_plan_fill).  This module restates the device algorithm step by step with stable sorts and prefix sums
so that the GPU result can be compared bit for bit.
"""
import numpy as np

FIXED_WORK = 24      # cost of a group beyond its pairs, in pair equivalents (same as the host builder)


def _excl(a):
    out = np.zeros(len(a) + 1, dtype=np.int64)
    np.cumsum(a, out=out[1:])
    return out


def base_plan(row, ipu, eid, indices, n_rows, n_index, seg_len):
    """rowptr, idx, eid (int32), items (n_items, 4) in locality order, heavy (n_heavy, 3), info dict."""
    row = np.asarray(row, dtype=np.int64); ipu = np.asarray(ipu, dtype=np.int64)
    U, E = len(row), len(eid)
    last = int(ipu[U]) if U else 0
    lb = np.searchsorted(row, np.arange(n_rows + 1), side="left")        # first unit of a row >= r
    rowptr = np.where(lb < U, ipu[np.minimum(lb, max(U - 1, 0))], last) if U else np.zeros(n_rows + 1, dtype=np.int64)
    deg = np.diff(rowptr)
    heavy_flag = deg > seg_len
    nseg = np.where(heavy_flag, -(-deg // seg_len), 1)
    item_base, heavy_base = _excl(nseg), _excl(heavy_flag)
    slot_base = _excl(np.where(heavy_flag, nseg, 0))
    n_items, n_heavy, n_slots = int(item_base[-1]), int(heavy_base[-1]), int(slot_base[-1])
    items = np.empty((n_items, 4), dtype=np.int32)
    heavy = np.empty((n_heavy, 3), dtype=np.int32)
    for r in range(n_rows):
        b, e = int(rowptr[r]), int(rowptr[r + 1])
        if not heavy_flag[r]:
            items[item_base[r]] = (r, b, e, -1)
        else:
            heavy[heavy_base[r]] = (r, slot_base[r], nseg[r])
            for s in range(int(nseg[r])):
                items[item_base[r] + s] = (r, b + s * seg_len, min(e, b + (s + 1) * seg_len), slot_base[r] + s)
    idx32 = (np.asarray(indices, dtype=np.int64) if indices is not None else np.zeros(E, dtype=np.int64)).astype(np.int32)
    eid32 = np.asarray(eid, dtype=np.int64).astype(np.int32)
    kmin = item_keys(items, idx32, n_index, np.min)
    items = items[np.argsort(kmin, kind="stable")]
    perm = bool(U > 0 and ipu[0] == 0 and last == E and len(np.unique(eid32)) == E) if E else (U == 0 or last == 0)
    return {"rowptr": rowptr.astype(np.int32), "idx": idx32, "eid": eid32, "items": items, "heavy": heavy,
            "seg_len": int(seg_len)}, {"n_items": n_items, "n_heavy": n_heavy, "n_slots": n_slots,
                                       "max_degree": int(deg.max()) if n_rows else 0, "perm": perm}


def item_keys(items, idx32, n_index, red):
    """Smallest / largest neighbour id of every item; an empty item: its own row id, clipped to n_index."""
    out = np.empty(len(items), dtype=np.int64)
    for i, (r, b, e, _) in enumerate(items.tolist()):
        out[i] = red(idx32[b:e]) if e > b else min(r, n_index)
    return out


def _entries_of(items, idx32, eid32, jorder, g_of_item, m_of_item, R):
    """One record per edge slot sorted by (group, neighbour, member), equal records in slot order; an entry per (group,
    neighbour) and per repeat of an edge in one member.  Returns ent_idx, ent_g, mask, slot_eid in that order."""
    E = len(eid32)
    key = np.zeros(E, dtype=np.int64)
    for j, it in enumerate(jorder.tolist()):
        b, e = items[it, 1], items[it, 2]
        key[b:e] = (g_of_item[j] << 35) | (idx32[b:e].astype(np.int64) << 4) | m_of_item[j]
    order = np.argsort(key, kind="stable")
    skey = key[order]
    t = np.zeros(E, dtype=np.int64)
    for i in range(1, E):
        t[i] = t[i - 1] + 1 if skey[i] == skey[i - 1] else 0
    head2 = np.ones(E, dtype=bool)
    head2[1:] = (skey[1:] >> 4) != (skey[:-1] >> 4)
    run = np.cumsum(head2) - 1
    n_runs = int(run[-1]) + 1 if E else 0
    mult = np.zeros(n_runs, dtype=np.int64)
    np.maximum.at(mult, run, t + 1)
    ebase = _excl(mult)
    n_entries = int(ebase[-1])
    u = ebase[run] + t
    ent_idx = np.zeros(n_entries, dtype=np.int64); ent_g = np.zeros(n_entries, dtype=np.int64)
    mask = np.zeros(n_entries, dtype=np.int64)
    slot_eid = np.full((n_entries, R), -1, dtype=np.int32)
    mem = skey & 15
    ent_idx[u] = (skey >> 4) & 0x7FFFFFFF
    ent_g[u] = skey >> 35
    np.bitwise_or.at(mask, u, 1 << mem)
    slot_eid[u, mem] = eid32[order]
    return ent_idx, ent_g, mask, slot_eid


def group_plan(arrays, n_index, R, by_mask):
    """Row groups: the items in the order of their largest neighbour, R consecutive ones per group; the groups
    numbered by locality (smallest neighbour), cut into 8 ranges of equal work, by decreasing work inside a range.
    Work: the group's pairs plus a fixed cost; for the tile plans (R = 16) its blocks of R entries, 4 * (blocks + 1) (what
    the matrix kernels pay for), known only once the entries of the locality-numbered groups are.
    by_mask: entry order inside a group: 0 / False ascending neighbour, 1 / True by member mask, 2 interleaved; + 4: the groups
    of a range keep their locality order instead of the order by decreasing work."""
    by_work = not (int(by_mask) & 4)
    by_mask = int(by_mask) & 3
    items, idx32, eid32 = arrays["items"], arrays["idx"], arrays["eid"]
    n_items, E = len(items), len(eid32)
    kmax = item_keys(items, idx32, n_index, np.max)
    jorder = np.argsort(kmax, kind="stable")
    ng = -(-n_items // R)
    lens = (items[:, 2] - items[:, 1]).astype(np.int64)
    w0 = np.zeros(ng, dtype=np.int64)
    np.add.at(w0, np.arange(n_items) // R, lens[jorder])
    w0 += FIXED_WORK
    # locality numbering of the groups: by the smallest neighbour id any member reads
    kmin = item_keys(items, idx32, n_index, np.min)
    gk = np.full(ng, np.iinfo(np.int64).max, dtype=np.int64)
    np.minimum.at(gk, np.arange(n_items) // R, kmin[jorder])
    lorder = np.argsort(gk, kind="stable")
    lpos = np.empty(ng, dtype=np.int64)
    lpos[lorder] = np.arange(ng)
    m_of_item = np.arange(n_items) % R
    if R == 16:
        _, prov_g, _, _ = _entries_of(items, idx32, eid32, jorder, lpos[np.arange(n_items) // R], m_of_item, R)
        w = 4 * (-(-np.bincount(prov_g, minlength=ng)[:ng] // R) + 1)
    else:
        w = w0[lorder]
    prefix, total = _excl(w)[:-1], int(w.sum())
    chunks = np.zeros(9, dtype=np.int32)
    for x in range(1, 8):
        chunks[x] = int(np.count_nonzero(prefix + w // 2 < total * x // 8))
    chunks[8] = ng
    chunk_of = np.searchsorted(chunks[1:8], np.arange(ng), side="right")
    gorder = np.argsort((chunk_of << 16) | ((0xFFFF - w) if by_work else 0), kind="stable")
    inv = np.empty(ng, dtype=np.int64)
    inv[gorder] = np.arange(ng)
    members = np.full((ng, R, 2), -1, dtype=np.int32)
    g_of_item = inv[lpos[np.arange(n_items) // R]]
    members[g_of_item, m_of_item, 0] = items[jorder, 0]
    members[g_of_item, m_of_item, 1] = items[jorder, 3]
    ent_idx, ent_g, mask, slot_eid = _entries_of(items, idx32, eid32, jorder, g_of_item, m_of_item, R)
    if int(by_mask) == 1:        # by member mask, larger first
        perm = np.argsort((ent_g << 16) | (0xFFFF ^ mask), kind="stable")
        ent_idx, ent_g, mask, slot_eid = ent_idx[perm], ent_g[perm], mask[perm], slot_eid[perm]
    elif int(by_mask) == 2:      # by (neighbour mod 16, neighbour): groups that share rows read them at about the same step
        perm = np.argsort((ent_g << 35) | ((ent_idx & 15) << 31) | ent_idx, kind="stable")
        ent_idx, ent_g, mask, slot_eid = ent_idx[perm], ent_g[perm], mask[perm], slot_eid[perm]
    grp_ptr = np.searchsorted(ent_g, np.arange(ng + 1), side="left").astype(np.int32)
    pop = np.array([bin(int(m)).count("1") for m in mask], dtype=np.int64)
    first = _excl(pop)[:-1]
    entries = np.stack([ent_idx, mask, first, np.zeros_like(first)], axis=1).astype(np.int32).reshape(-1, 4)
    pair_eid = slot_eid[slot_eid >= 0].astype(np.int32)           # row-major: entry by entry, members ascending
    return {"members": members, "grp_ptr": grp_ptr, "entries": entries, "pair_eid": pair_eid, "slot_eid": slot_eid,
            "chunks": chunks, "R": R}


def link_groups(grp_dst, grp_src, n_edges, pad_entries):
    """grp_pairs of the destination side: position entry' * R + member' of the same edge on the source side."""
    Rd, Rs = grp_dst["R"], grp_src["R"]
    spare = (len(grp_src["entries"]) + pad_entries) * Rs - 1
    pos = np.full(n_edges, spare, dtype=np.int64)
    ss = grp_src["slot_eid"].reshape(-1)
    pos[ss[ss >= 0]] = np.nonzero(ss >= 0)[0]
    out = np.full((len(grp_dst["entries"]) + pad_entries) * Rd, spare, dtype=np.int32)
    sd = grp_dst["slot_eid"].reshape(-1)
    out[:len(sd)][sd >= 0] = pos[sd[sd >= 0]]
    return out
