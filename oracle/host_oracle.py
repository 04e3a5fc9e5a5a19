"""Integer restatement of the reference's host-side planner and block-table
logic. TEST INFRASTRUCTURE (see binding.py). Plain loops; every function names
the reference lines it follows. These are the bit-exact parts of the path:
the product's C++ planner, run with the reference's constants, must produce
identical records.
"""


def plan_tiles(trees, Hkv, split, groups=256, min_chunk=32):
    """plan_tiles without the sparse-attention branch: src/model/impl/forest.h:1378-1433.
    trees: list of (base, P, table, M). Returns (tiles, combine, parts); tile =
    (tree, r0, k0, k1, part, last, 0, 0), combine = (r0, rows, part0, nparts)."""
    tiles, combine, parts = [], [], 0
    n_tiles = sum((t[3] + 7) // 8 for t in trees)
    budget = max(1, groups // max(1, Hkv * n_tiles))
    for ti, (base, P, _table, M) in enumerate(trees):
        ns = 1
        if split > 0 and budget > 1 and P >= 64:
            chunk = max(max(32, min_chunk), min(split, ((P + budget - 1) // budget + 31) // 32 * 32))
            ns = min((P + chunk - 1) // chunk, budget, 64)
        for r in range(0, M, 8):
            if ns == 1:
                tiles.append((ti, base + r, 0, P, -1, 1, 0, 0))
                continue
            per = (P + ns - 1) // ns
            step = (per + 31) // 32 * 32
            part0, used, k = parts, 0, 0
            while k < P:
                k1 = min(P, k + step)
                tiles.append((ti, base + r, k, k1, parts, 1 if k1 >= P else 0, 0, 0))
                parts += 1
                k += step
                used += 1
            combine.append((base + r, min(8, M - r), part0, used))
    return tiles, combine, parts


def g4_plan_tiles(trees, groups, split, window, pos, rows=8):
    """g4_plan_tiles: src/model/impl/gemma.h:77-116. pos: flat int list, 4 per row
    (pos[4 * row] = position). Returns (tiles, combine, parts, rows_used)."""
    tiles, combine, parts = [], [], 0
    n_tiles = sum((t[3] + 7) // 8 for t in trees)
    budget = max(1, 256 // max(1, groups * n_tiles))
    arows = rows if budget == 1 else 8
    for ti, (base, P, _table, M) in enumerate(trees):
        for r in range(0, M, arows):
            k0 = b0 = 0
            if window > 0:
                minpos = min(pos[4 * (base + i)] for i in range(r, min(M, r + arows)))
                k0 = min(max(minpos - window + 1, 0), P)
                b0 = max(0, minpos - window + 1 - P)
            span = P - k0
            ns = 1
            if split > 0 and budget > 1 and span >= 64:
                chunk = max(32, min(split, ((span + budget - 1) // budget + 31) // 32 * 32))
                ns = min((span + chunk - 1) // chunk, budget, 64)
            if ns == 1:
                tiles.append((ti, base + r, k0, P, -1, 1, b0, 0))
                continue
            per = (span + ns - 1) // ns
            step = (per + 31) // 32 * 32
            part0, used, k = parts, 0, k0
            while k < P:
                k1 = min(P, k + step)
                tiles.append((ti, base + r, k, k1, parts, 1 if k1 >= P else 0, b0, 0))
                parts += 1
                k += step
                used += 1
            combine.append((base + r, min(8, M - r), part0, used))
    return tiles, combine, parts, arows


class Pool:
    """KV block allocator: src/model/impl/forest.h:60-62 (free list order),
    src/model/impl/model.h:722-737 (alloc / retain / release)."""

    def __init__(self, n_blocks, bt):
        self.bt = bt
        self.ref = [0] * n_blocks
        self.free_list = list(range(n_blocks - 1, -1, -1))

    def alloc(self):
        if not self.free_list:
            raise RuntimeError("KV cache full")
        b = self.free_list.pop()
        self.ref[b] = 1
        return b

    def retain(self, b):
        self.ref[b] += 1

    def release(self, b):
        self.ref[b] -= 1
        if self.ref[b] == 0:
            self.free_list.append(b)


def target_blocks(pool, parent_blocks, P, w0, end, in_place):
    """Forest::target_blocks: src/model/impl/forest.h:1785-1811. Returns (blocks, cow pairs)."""
    bt = pool.bt
    out, cow = [], []
    keep = w0 // bt
    for i in range(min(keep, len(parent_blocks))):
        out.append(parent_blocks[i])
        pool.retain(parent_blocks[i])
    need = (end + bt - 1) // bt
    for i in range(keep, need):
        has_parent = i < len(parent_blocks) and i * bt < P
        if has_parent and in_place and pool.ref[parent_blocks[i]] == 1:
            out.append(parent_blocks[i])
            pool.retain(parent_blocks[i])
            continue
        nb = pool.alloc()
        if has_parent:
            cow.append((parent_blocks[i], nb))
        out.append(nb)
    return out, cow


def target_new_blocks(pool, parent_blocks, P, w0, end, in_place):
    """target_new_blocks: src/model/impl/forest.h:1821-1829 (parent_blocks None: no parent)."""
    bt = pool.bt
    i = w0 // bt
    n = (end + bt - 1) // bt - i
    if (n > 0 and in_place and parent_blocks is not None and i < len(parent_blocks) and i * bt < P
            and pool.ref[parent_blocks[i]] == 1):
        n -= 1
    return max(n, 0)


def host_leaves(leaf_tokens, leaf_offsets):
    """Leaf hosting: src/model/impl/forest.h:2201-2220. Returns (host, off, leaf_rows)."""
    NL = len(leaf_offsets) - 1

    def ln(i):
        return leaf_offsets[i + 1] - leaf_offsets[i]

    host, off = [-1] * NL, [0] * NL
    for i in range(NL):
        h = i
        ti = leaf_tokens[leaf_offsets[i]:leaf_offsets[i] + ln(i)]
        for j in range(NL):
            if j == i or ln(j) < ln(i):
                continue
            if ln(j) == ln(i) and j > i:
                continue
            if ln(j) < ln(h) or (ln(j) == ln(h) and j >= h):
                continue
            if leaf_tokens[leaf_offsets[j]:leaf_offsets[j] + ln(i)] == ti:
                h = j
        host[i] = h
    leaf_rows = 0
    for i in range(NL):
        if host[i] == i:
            off[i] = leaf_rows
            leaf_rows += ln(i)
    return host, off, leaf_rows


def tree_rows(base, Tr, next_pos, leaf_tokens, leaf_offsets, noncausal=False):
    """desc / pos of a tree's rows: src/model/impl/forest.h:2376-2443 (text rows, no
    explicit positions, no images). Returns (desc rows, pos rows, M), row = 4 ints."""
    desc, pos = [], []
    pmax = next_pos - 1
    for j in range(Tr):
        pt = next_pos + j
        pos.append((pt, pt, pt, 0))
        pmax = max(pmax, pt)
        desc.append((0, 0, Tr if noncausal else 0, 0))
    next_root = pmax + 1
    host, off, leaf_rows = host_leaves(leaf_tokens, leaf_offsets)
    desc += [None] * leaf_rows
    pos += [None] * leaf_rows
    for i in range(len(host)):
        if host[i] != i:
            continue
        start = Tr + off[i]
        for j in range(leaf_offsets[i + 1] - leaf_offsets[i]):
            pos[start + j] = (next_root + j,) * 3 + (0,)
            desc[start + j] = (start, 0, Tr, 0)
    return desc, pos, Tr + leaf_rows


def kv_saves(base, P, n, blocks, bt):
    """add_saves: src/model/impl/forest.h:2490-2494."""
    return [(base + i, blocks[(P + i) // bt], (P + i) % bt, 0) for i in range(n)]


def kv_row_table(saves, rows):
    """kv_row_table: src/model/impl/forest.h:1737-1749. saves: (src_row, block, pos, _) tuples."""
    t = [[-1, -1, -1, -1] for _ in range(max(rows, 1))]
    for (row, block, pos, _pad) in saves:
        e = t[row]
        j = 0 if e[0] < 0 else 2
        if j == 2 and e[2] >= 0:
            raise ValueError("a row saved into more than two slots")
        e[j], e[j + 1] = block, pos
    return t[:rows]



def ring_plan(trees, window, ring_blocks, bt):
    """The sliding layers' view of a pass: src/model/impl/forest.h:2657-2659 (trees) and 2679-2700 (saves,
    copies). Slot s owns ring blocks [s * ring_blocks, (s + 1) * ring_blocks); position p lives in block
    (p / bt) % ring_blocks. trees: (base, P, M, parent slot or -1, [(target slot, rows saved), ...]).
    Returns (tree records (base, P, table, M), saves (src_row, block, pos, 0), copies (src, dst))."""
    recs, saves, copies = [], [], []
    for base, P, M, parent, targets in trees:
        recs.append((base, P, parent * ring_blocks if parent >= 0 else 0, M))
        for slot, S in targets:
            if slot != parent and P > 0:
                seen = set()
                b = max(0, P + S - window + 1) // bt
                while b * bt < P:
                    if b % ring_blocks not in seen:
                        seen.add(b % ring_blocks)
                        copies.append((parent * ring_blocks + b % ring_blocks, slot * ring_blocks + b % ring_blocks))
                    b += 1
            for p in range(max(P, P + S - window + 1), P + S):
                saves.append((base + (p - P), slot * ring_blocks + (p // bt) % ring_blocks, p % bt, 0))
    return recs, saves, copies
