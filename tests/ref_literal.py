"""Literal pure-Python models of the reference's beam search and insert, for pinning the CPU oracle.

Each function follows the reference's data structures as they are laid out there (one flat queue of
`queue_capacity` slots, a whole-queue sort per iteration, the expanded flag in the top bit of the id,
the open-addressing table) instead of the merged form the oracle and the kernels use, so that a
misreading shared by oracle and kernels shows up as a difference.  Threads of a block are played one
after the other in index order (one legal interleaving of the reference's atomics).

The `fixes` argument switches on, one by one, the behaviours in which the library's default mode
departs from the reference; with no fixes the model is the reference as written.
"""
import numpy as np

INVALID = 0xFFFFFFFF
MSB = 0x80000000
FLT_MAX = np.float32(3.40282e38)
M64 = (1 << 64) - 1

# behaviours of the library's default mode that the reference does not have
FIX_SEEDS = 1          # seeds that are duplicates or fail the filter are not queued
FIX_RESTORE_ORDER = 2  # the visited set is rebuilt after the sort of that iteration, not before it
FIX_EMPTY_SLOTS = 4    # unfilled result slots are -1 instead of 0x7FFFFFFF
FILTER_FIRST = 8       # the filter is tested before the visited-set insert (rows outside never enter the table)


def next_power_of_2(n):  # src/index/smem_cal.cuh:13-23
    if n == 0:
        return 1
    return 1 << (n - 1).bit_length()


def queue_capacity(itopk, sw, degree):  # src/index/cagra.cu:871-873
    return max(256, next_power_of_2(itopk + sw * degree))


class Table:
    """src/index/hashmap.cuh:30-117."""

    def __init__(self, bitlen):
        self.bitlen = bitlen
        self.size = 1 << bitlen
        self.slots = [INVALID] * self.size
        self.used = 0
        self.full_hits = 0  # inserts attempted while no slot was free (they fail whether or not the key is there)

    def init(self):
        self.slots = [INVALID] * self.size
        self.used = 0

    def insert(self, key):
        if self.used == self.size:
            self.full_hits += 1
        mask = self.size - 1
        idx = (key ^ (key >> self.bitlen)) & mask
        for _ in range(self.size):
            old = self.slots[idx]
            if old == INVALID:
                self.slots[idx] = key
                self.used += 1
                return True
            if old == key:
                return False
            idx = (idx + 1) & mask
        return False

    def restore(self, indices, itopk, skip_invalid):
        for i in range(itopk):
            if skip_invalid and indices[i] == INVALID:
                continue
            node = indices[i] & 0x7FFFFFFF
            if node != INVALID:  # always true once the top bit is stripped (hashmap.cuh:109-113)
                self.insert(node)


def l2_exact(a, b):
    """Squared L2 in float64; exact, hence order-independent, on the integer-valued inputs the tests use."""
    d = a.astype(np.float64) - b.astype(np.float64)
    return np.float32(np.dot(d, d))


def search_one(data, graph, q, topk, itopk, sw, max_iter, bitlen, num_seeds, seeds, mask, variant="plain",
               active_degree=None, ts=None, window=None, fixes=0, dist=l2_exact):
    """One query of search_kernel / search_kernel_bucket / search_kernel_range
    (src/index/search.cu:149-370, 375-586, 589-798).

    variant: "plain" (compute_distance_to_child_nodes), "strided" (…_strided, local slots only),
    "range" (…_range, timestamps tested after the visited-set insert, skipped slots left as they are).
    Returns ids (python ints), float32 distances and counters
    {iterations, S, P, F_all, F_fresh, D, full}.
    """
    n, degree = data.shape[0], graph.shape[1]
    cap = queue_capacity(itopk, sw, degree)
    assert cap in (256, 512, 1024, 2048) and itopk % 32 == 0
    ridx = [INVALID] * cap
    rdist = [FLT_MAX] * cap
    table = Table(bitlen)
    ctr = dict(iterations=0, S=0, P=0, F_all=0, F_fresh=0, D=0, full=0)

    def in_window(node):
        return window[0] <= int(ts[node]) < window[1]

    filtered = variant == "range"
    # --- seeds: compute_distance_to_random_nodes / _init_nodes (compute_distance.cuh:144-269)
    for i in range(num_seeds):
        node = INVALID
        if seeds is not None and i < len(seeds):
            node = int(seeds[i])
        if node >= n:
            node = ((mask * (i + 1)) & M64) % n
        if fixes & FIX_SEEDS:
            if filtered and (fixes & FILTER_FIRST):
                ctr["F_all"] += 1
                ctr["F_fresh"] += 1
                if not in_window(node):
                    continue
            if not table.insert(node):
                continue
            if filtered and not (fixes & FILTER_FIRST):
                ctr["F_all"] += 1
                ctr["F_fresh"] += 1
                if not in_window(node):
                    continue
            ridx[i], rdist[i] = node, dist(q, data[node])
        else:
            ridx[i], rdist[i] = node, dist(q, data[node])  # slot i is written whatever the insert says
            table.insert(node)
        ctr["S"] += 1

    def sort_queue():
        # load_sort_store over the whole capacity, by distance alone (search.cu:287-298); stable
        order = sorted(range(cap), key=lambda j: rdist[j])
        ri = [ridx[j] for j in order]
        rd = [rdist[j] for j in order]
        ridx[:], rdist[:] = ri, rd

    def rebuild_table():
        table.init()
        table.restore(ridx, itopk, skip_invalid=bool(fixes & FIX_RESTORE_ORDER))

    it = 0
    while it < max_iter:
        reset = it > 0 and it % 30 == 0
        if reset and not (fixes & FIX_RESTORE_ORDER):
            rebuild_table()  # search.cu:273-283: before the sort, so this iteration's candidates are forgotten
        sort_queue()
        if reset and (fixes & FIX_RESTORE_ORDER):
            rebuild_table()

        # --- pickup_next_parents (search.cu:38-107), 32 lanes at a time
        parents = [INVALID] * sw
        found = 0
        for base in range(0, itopk, 32):
            votes = [(ridx[base + lane] & MSB) == 0 and ridx[base + lane] != INVALID for lane in range(32)]
            for lane in range(32):
                if votes[lane]:
                    rank = found + sum(votes[:lane])
                    if rank < sw:
                        parents[rank] = ridx[base + lane]
                        ridx[base + lane] |= MSB
            found += sum(votes)
            if found >= sw:
                break
        if found == 0:
            break
        ctr["iterations"] += 1

        # --- expansion into the slots behind the first itopk
        for task in range(sw * degree):
            p_idx, off = task // degree, task % degree
            slot = itopk + task

            def skip():
                if variant != "range":  # the range variant leaves the slot as the sort left it
                    ridx[slot], rdist[slot] = INVALID, FLT_MAX

            if variant == "strided" and off >= active_degree:
                skip()
                continue
            parent = parents[p_idx]
            if parent == INVALID:
                skip()
                continue
            if off == 0:
                ctr["P"] += 1
            nb = int(graph[parent, off])
            if nb == INVALID:
                skip()
                continue
            if filtered and (fixes & FILTER_FIRST):
                ctr["F_all"] += 1
                ctr["F_fresh"] += 1
                if not in_window(nb):
                    continue
                if not table.insert(nb):
                    continue
            else:
                fresh = table.insert(nb)
                if filtered:
                    ctr["F_all"] += 1  # d_ts[nb] is read whether or not nb is new (compute_distance.cuh:580)
                    ctr["F_fresh"] += int(fresh)
                    if not in_window(nb):
                        continue
                if not fresh:
                    skip()
                    continue
            ridx[slot], rdist[slot] = nb, dist(q, data[nb])
            ctr["D"] += 1
        it += 1

    sort_queue()
    ids, dists = [], []
    for i in range(topk):
        if (fixes & FIX_EMPTY_SLOTS) and ridx[i] == INVALID:
            ids.append(-1)
        else:
            ids.append(ridx[i] & 0x7FFFFFFF)  # search.cu:351
        dists.append(rdist[i])
    ctr["full"] = table.full_hits
    return ids, np.array(dists, np.float32), ctr


def search_wrapper_plan(k, itopk_param, sw, degree):
    """cagra::search (src/index/cagra.cu:861-887): list length, number of random seeds."""
    itopk = max(k, itopk_param)
    if itopk < 64:
        itopk = 64
    return itopk, itopk_param // 4


def striped_warp_sort(dists, ids, search_k):
    """insert_sort_kernel (src/index/insert.cu:80-133): lane l loads elements l, l+32, … but the network
    treats a lane's registers as the consecutive elements l*N … l*N+N-1, and the result goes back the way
    it was loaded."""
    per_lane = 2 if search_k <= 64 else 4 if search_k <= 128 else 8 if search_k <= 256 else 16
    total = 32 * per_lane
    key = [FLT_MAX] * total
    val = [INVALID] * total
    for lane in range(32):
        for i in range(per_lane):
            src = lane + i * 32
            if src < search_k:
                key[lane * per_lane + i] = dists[src]
                val[lane * per_lane + i] = ids[src] & 0xFFFFFFFF
    order = sorted(range(total), key=lambda j: (key[j], val[j]))
    out_d, out_i = list(dists), list(ids)
    for lane in range(32):
        for i in range(per_lane):
            dst = lane + i * 32
            if dst < search_k:
                j = order[lane * per_lane + i]
                out_d[dst], out_i[dst] = key[j], val[j]
    return out_d, out_i


def insert_batch(data, n_existing, n_new, graph, itopk_param, sw, max_iter, bitlen, masks, striped=True, fixes=0,
                 dist=l2_exact):
    """cagra::insert (src/index/cagra.cu:938-1015): find_near_nodes (src/index/insert.cu:140-219) in groups of
    64 new rows, one `rand_xor_mask` per group (`masks`), then update_topology_gpu_v1 (:225-440).
    `striped=False` sorts the result list properly (the blocked layout the network expects)."""
    degree = graph.shape[1]
    search_k = 2 * degree
    g = graph.copy()
    itopk, n_seeds = search_wrapper_plan(search_k, itopk_param, sw, degree)
    found = []
    for i in range(n_new):
        q = data[n_existing + i]
        ids, _, _ = search_one(data[:n_existing], graph[:n_existing], q, search_k, itopk, sw, max_iter, bitlen, n_seeds,
                               None, masks[i // 64], fixes=fixes, dist=dist)
        # insert_refine_kernel_warp: exact distance, FLT_MAX for ids outside [0, n_existing)
        d = [dist(q, data[t]) if 0 <= t < n_existing else FLT_MAX for t in ids]
        if striped:
            _, ids = striped_warp_sort(d, ids, search_k)
        else:
            order = sorted(range(search_k), key=lambda j: (d[j], ids[j] & 0xFFFFFFFF))
            ids = [ids[j] & 0xFFFFFFFF for j in order]
        found.append(ids)
    # fill_new_nodes_kernel (:225-257)
    for i in range(n_new):
        for k in range(degree):
            v = INVALID
            if k < search_k and 0 <= found[i][k] < n_existing:
                v = found[i][k]
            g[n_existing + i, k] = v
    # generate_update_requests_kernel (:263-290), sort by target (:422-424), apply (:296-368)
    req = []
    for t in range(n_new * search_k):
        nb = found[t // search_k][t % search_k]
        req.append((nb, n_existing + t // search_k) if 0 <= nb < n_existing else (INVALID, INVALID))
    req.sort(key=lambda r: r[0])  # stable
    total = len(req)
    protected = degree // 2
    unprotected = degree - protected
    for tid in range(total):
        target = req[tid][0]
        if target == INVALID:
            continue
        if tid != 0 and req[tid - 1][0] == target:
            continue
        rng = (target * 0x9e3779b97f4a7c15 + tid) & M64
        idx = tid
        while idx < total and req[idx][0] == target:
            new_id = req[idx][1]
            if new_id not in g[target].tolist():
                rng = (rng * 6364136223846793005 + 1) & M64
                r1 = rng >> 32
                rng = (rng * 6364136223846793005 + 1) & M64
                r2 = rng >> 32
                slot = (r2 % protected) if r1 % 10 == 0 else protected + (r2 % unprotected)
                g[target, slot] = new_id
            idx += 1
    return g
