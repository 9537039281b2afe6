"""Host model of every GLOBAL address the direct-to-LDS kernels touch (emerging-optimizers_amd/csrc/gemm_fast.hpp with
its launcher, launch_impl.hpp, and the tile enumerations of gemm_engine.hpp).

The fast kernel's loaders have no bounds checks of their own: a tile that lies wholly inside its operand is fetched
through precomputed lane offsets, and only the lower-triangle product of K-contiguous operands has a variant with
clamped rows for tiles that overhang the matrix.  Whether a launch is safe is therefore decided on the host.  This
model replays, for every tile configuration x operand layout x product the library instantiates,
  * the launcher's decisions (tile counts, the padded lower-triangle grid, edge variant or refusal),
  * workgroup id -> tile (``tri_block_decode`` with the XCD chunking, ``gemm_tile_of``),
  * every 16-byte operand load of every wavefront for the first and the last K tile (``FastLoader``),
  * the addend loads and every store of both epilogues (row-wise and mirrored write-out, GEMM staging),
  * the per-workgroup partial-sum slot,
  * the stream-K schedule of the 256 x 256 lower-triangle kernel (ranges of K tiles per workgroup, who parks an
    accumulator image where, whom an owner waits for),
over a grid of shapes (multiples of 8 on both sides of every tile size, batches, split-K slices, the tail split of
the wide GEMM) and asserts that each access lies inside the matrix it belongs to.  It also checks that the tile
enumerations visit every tile exactly once.  No GPU is involved.
"""

import itertools

import numpy as np
import pytest

NW, BK, MI = 4, 64, 16
LANES = np.arange(64)

# name -> (TILE_M, TILE_N, WGM, WGN, ring slots)
CFGS = {
    "CfgM128": (128, 256, 1, 4, 2),
    "CfgT128": (128, 128, 2, 2, 3),
    "CfgT128x2": (128, 128, 2, 2, 2),
    "CfgBig": (256, 256, 2, 2, 2),
    "CfgHalfN": (256, 128, 2, 2, 3),
    "CfgSyrk192": (192, 192, 2, 2, 3),
}
# (cfg, P K-strided, Q K-strided, mode) exactly as the inst_*.hip files instantiate them
INSTANCES = [
    ("CfgSyrk192", False, False, "syrk"), ("CfgT128", False, False, "syrk"), ("CfgBig", False, False, "syrk"),
    ("CfgT128x2", False, False, "syrk"), ("CfgBig", True, True, "syrk"), ("CfgT128", True, True, "syrk"),
    ("CfgT128x2", True, True, "syrk"), ("CfgBig", False, True, "gemm"), ("CfgHalfN", False, True, "gemm"),
    ("CfgM128", False, True, "gemm"), ("CfgBig", False, False, "gemm"), ("CfgT128", False, False, "gemm"),
]


def kc_slot(row, c):
    return c ^ ((row >> 1) & 7)


def ks_rot(k):
    return 2 * (k & 7) + 8 * (k >> 3)


# ------------------------------------------------------------------ tile enumerations
def tri_block_decode(s, T, block=6):
    r = 0
    while (r + 1) * (r + 2) // 2 <= s:
        r += 1
    bi = r // block
    row0 = bi * block
    h = min(T - row0, block)
    u = s - row0 * (row0 + 1) // 2
    rect = h * block
    if u < bi * rect:
        bj, v = divmod(u, rect)
        return row0 + v // block, bj * block + v % block
    u -= bi * rect
    lr = 0
    while (lr + 1) * (lr + 2) // 2 <= u:
        lr += 1
    return row0 + lr, row0 + (u - lr * (lr + 1) // 2)


def gemm_tile_of(pid, tiles_m, tiles_n, xcds=8, block_m=8):
    if tiles_n % xcds != 0 or tiles_m % block_m != 0:
        return pid % tiles_m, pid // tiles_m
    xcd, local = pid % xcds, pid // xcds
    cols_per_xcd = tiles_n // xcds
    block = block_m * cols_per_xcd
    rb, r = divmod(local, block)
    return rb * block_m + r % block_m, xcd * cols_per_xcd + r // block_m


def round_size(cfg, cus=256):
    """Workgroups of a configuration that the chip holds at once (two per CU when two rings fit its 160 KB of LDS)."""
    tile_m, tile_n, _, _, slots = CFGS[cfg]
    per_cu = 2 if 2 * slots * (tile_m + tile_n) * BK * 2 <= 160 * 1024 else 1
    return max(cus * per_cu // 8 * 8, 8)


def syrk_grid_tiles(tiles_m, batch=1, g=256, limit=None):
    """Workgroup id -> (batch entry, tile) of the one-dimensional lower-triangle grid over a whole batch (None: padding
    workgroup that exits at once): whole rounds of g workgroups, then a last round shared evenly between the XCDs."""
    tri = tiles_m * (tiles_m + 1) // 2
    total = tri * batch if limit is None else min(limit, tri * batch)
    full = total // g * g
    last = (total - full + 7) // 8
    out = []
    for bid in range(full + 8 * last):
        if bid < full:
            tile = bid // g * g + (bid % 8) * (g // 8) + (bid % g) // 8
        else:
            j, rest = bid - full, total - full
            lo, hi = rest * (j % 8) // 8, rest * (j % 8 + 1) // 8
            if j // 8 >= hi - lo:
                out.append(None)
                continue
            tile = full + lo + j // 8
        out.append((tile // tri, tri_block_decode(tile % tri, tiles_m)))
    return out


@pytest.mark.parametrize("tiles_m", list(range(1, 70)))
def test_lower_triangle_grid_visits_every_tile_once(tiles_m):
    for batch, g in ((1, 256), (3, 256), (5, 512), (2, 8), (7, 304)):
        grid = syrk_grid_tiles(tiles_m, batch, g)
        seen = [t for t in grid if t is not None]
        assert sorted(seen) == [(b, (i, j)) for b in range(batch) for i in range(tiles_m) for j in range(i + 1)]
        # every XCD (workgroup id % 8) gets the same number of tiles, give or take one
        per_xcd = [sum(1 for t in grid[x::8] if t is not None) for x in range(8)]
        assert max(per_xcd) - min(per_xcd) <= 1
    # a limited launch (the whole rounds of a split-tail product) computes exactly the first tiles of that order
    tri = tiles_m * (tiles_m + 1) // 2
    lim = 3 * tri // 2
    seen = sorted(t for t in syrk_grid_tiles(tiles_m, 3, 256, limit=lim) if t is not None)
    assert seen == sorted((b, tri_block_decode(s, tiles_m)) for b in range(3) for s in range(tri) if b * tri + s < lim)


@pytest.mark.parametrize("tiles_m,tiles_n", [(4, 9), (8, 16), (16, 48), (16, 56), (8, 32), (1, 2), (3, 3), (16, 8), (24, 40), (7, 16)])
def test_gemm_grid_visits_every_tile_once(tiles_m, tiles_n):
    seen = [gemm_tile_of(pid, tiles_m, tiles_n) for pid in range(tiles_m * tiles_n)]
    assert sorted(seen) == [(i, j) for i in range(tiles_m) for j in range(tiles_n)]


# ------------------------------------------------------------------ operand loads
class Matrix:
    """A row-major (rows x cols) matrix inside a batch; every access must name an in-range row and a run of columns
    that ends inside the row."""

    def __init__(self, name, rows, cols, ld=None):
        self.name, self.rows, self.cols, self.ld = name, rows, cols, cols if ld is None else ld

    def check(self, rows, cols, width, what):
        rows, cols = np.asarray(rows), np.asarray(cols)
        ok = (rows >= 0) & (rows < self.rows) & (cols >= 0) & (cols + width <= self.cols)
        assert ok.all(), f"{what}: {self.name}[{rows[~ok][:4]}, {cols[~ok][:4]} + {width}] outside {self.rows} x {self.cols}"


def loader_accesses(rows_tile, ks, clamp, row0, rows_valid, kt, wave):
    """(row, k) of the first element of every 16-byte load that `wave` issues for K tile `kt` of one operand tile
    (rows = the operand's row index, k = its position along K), as FastLoader computes them."""
    lpt = rows_tile * BK * 2 // 1024 // NW
    out_r, out_k = [], []
    b0 = wave * lpt
    if clamp:
        assert not ks
        for i in range(lpt):
            b = b0 + i
            row = 8 * b + LANES // 8
            c = kc_slot(row, LANES % 8)
            gr = np.minimum(row0 + row, rows_valid - 1)
            out_r.append(gr)
            out_k.append(c * 8 + BK * kt)
        return np.concatenate(out_r), np.concatenate(out_k)
    if not ks:
        period, nv = 2, 2
        assert lpt % period == 0 and b0 % period == 0  # the phase of load i is i % 2 for every wavefront
        for i in range(lpt):
            v = i % nv
            lr = LANES // 8
            c = kc_slot(8 * v + lr, LANES % 8)
            out_r.append(row0 + 8 * (b0 + i) + lr)
            out_k.append(c * 8 + BK * kt)
    else:
        chunks, rows_per_kb = rows_tile // 8, 512 // rows_tile
        period = max(chunks // rows_per_kb, 1)
        periodic = lpt % period == 0
        for i in range(lpt):
            v = (i % min(period, lpt)) if periodic else b0 + i
            kr = LANES // chunks
            c = ((LANES % chunks) - ks_rot(rows_per_kb * v + kr)) & (chunks - 1)
            if periodic:  # the offset registers are shared by all wavefronts: the phase must not depend on b0
                c_true = ((LANES % chunks) - ks_rot(rows_per_kb * (b0 + i) + kr)) & (chunks - 1)
                assert (c == c_true).all()
            out_k.append(rows_per_kb * (b0 + i) + kr + BK * kt)
            out_r.append(row0 + c * 8)
    return np.concatenate(out_r), np.concatenate(out_k)


_COVERED = set()


def check_operand(mat_rows, K, ks, rows_tile, clamp, row0, kts, what, k_off=0, k_total=None):
    """All loads of one operand tile.  The operand is (mat_rows x k_total) K-contiguous or (k_total x mat_rows)
    K-strided in memory; the product covers k in [k_off, k_off + K)."""
    k_total = K if k_total is None else k_total
    mem = Matrix(what, k_total, mat_rows) if ks else Matrix(what, mat_rows, k_total)
    for kt in kts:
        for wave in range(NW):
            r, k = loader_accesses(rows_tile, ks, clamp, row0, mat_rows, kt, wave)
            if ks:
                mem.check(k + k_off, r, 8, what)     # 8 consecutive rows of the operand at one k
            else:
                mem.check(r, k + k_off, 8, what)     # 8 consecutive k of one row
            if not clamp:
                assert (r >= row0).all() and (r < row0 + rows_tile).all()
    # the tile is covered: every (row, k-chunk) of a K tile is fetched by exactly one lane (the lane arithmetic does
    # not depend on the tile's position: checked once per layout)
    if not clamp and (rows_tile, ks) not in _COVERED:
        _COVERED.add((rows_tile, ks))
        hits = np.zeros((rows_tile, BK), dtype=np.int32)
        for wave in range(NW):
            r, k = loader_accesses(rows_tile, ks, clamp, row0, mat_rows, 0, wave)
            if ks:   # 8 consecutive rows at one k
                for e in range(8):
                    np.add.at(hits, (r - row0 + e, k), 1)
            else:    # 8 consecutive k of one row
                for e in range(8):
                    np.add.at(hits, (r - row0, k + e), 1)
        assert (hits == 1).all()


# ------------------------------------------------------------------ epilogues
def syrk_epilogue_accesses(cfg, M, m0, n0, diag, guard, skip_upper, addends, out, cmat):
    tile, _, wgm, wgn, ns = CFGS[cfg]
    tm = tile // wgm
    fm = tm // MI
    ldt = tile + 8
    rp, npass = tile, 1          # the whole tile is staged at once (the kernel sizes its LDS for it)
    assert rp * ldt * 2 <= 160 * 1024 - 256 and ns >= 2
    cprw = tile // 8
    nt = NW * 64
    assert rp * cprw % nt == 0
    # addends: a 256 x 256 tile copies them row-wise (16 bytes per lane) into the staging area ...
    if fm * fm * 2 > 80 and addends:
        nt_, cprw_ = NW * 64, tile // 8
        assert tile * cprw_ % (nt_ * 8) == 0   # batches of 8 chunks per thread
        for it in range(tile * cprw_ // nt_):
            c = np.arange(nt_) + it * nt_
            row, c8 = c // cprw_, c % cprw_
            gr, gc = m0 + row, n0 + c8 * 8
            on = (gr < M) & (gc < M) if guard else np.ones(nt_, bool)
            cmat.check(gr[on], gc[on], 8, "addend copy")
            assert ((row * ldt + c8 * 8) * 2 + 16 <= tile * ldt * 2).all()
    # ... smaller tiles read them in accumulator layout
    for wave in range(NW):
        wm, wn = wave % wgm, wave // wgm
        for i in range(fm):
            for j in range(fm):
                m = m0 + wm * tm + i * MI + (LANES & 15)
                n = n0 + wn * tm + j * MI + 4 * (LANES >> 4)
                if guard:
                    # every lane loads (the K loop counts these loads in its vmcnt waits): quads beyond the matrix
                    # read a clamped address
                    m, n = np.minimum(m, M - 1), np.where(n + 4 <= M, n, M - 4)
                if addends:
                    cmat.check(m, n, 4, "addend fetch")
    # store counts in the tile's own window (rows from m0, columns from n0) and in the mirrored window
    direct = np.zeros((tile, tile), dtype=np.int32)
    mirror = direct if diag else np.zeros((tile, tile), dtype=np.int32)

    def store(gr, gc, on):
        gr, gc = gr[on], gc[on]
        out.check(gr, gc, 8, "store")
        in_direct = (gr >= m0) & (gr < m0 + tile) & (gc >= n0) & (gc + 8 <= n0 + tile)
        in_mirror = (gr >= n0) & (gr < n0 + tile) & (gc >= m0) & (gc + 8 <= m0 + tile)
        if diag:
            assert in_direct.all(), "store outside the tile"
        else:
            assert (in_direct ^ in_mirror).all(), "store outside the tile and its mirror image"
        for e in range(8):
            np.add.at(direct, (gr[in_direct] - m0, gc[in_direct] - n0 + e), 1)
            if not diag:
                np.add.at(mirror, (gr[in_mirror] - n0, gc[in_mirror] - m0 + e), 1)

    tids = np.arange(nt)
    sym = diag and not skip_upper
    for h in range(npass):
        for it in range(rp * cprw // nt):
            c = tids + it * nt
            row, c8 = c // cprw, c % cprw
            gr, gc = m0 + h * rp + row, n0 + c8 * 8
            held = (c8 * 8 < ((h * rp + row) // tm + 1) * tm) if diag else np.ones(nt, bool)
            on = held & ((gr < M) & (gc < M) if guard else True)
            store(gr, gc, on)
        if skip_upper:
            continue

        def mirror_out(rows, ccols, r_lo, grow0, gcol0):
            nb = rows // 32
            units = ccols // 4 * nb
            for it in range((units + 15) // 16):
                for wave in range(NW):
                    unit = it * 16 + wave * 4 + (LANES >> 4)
                    on = unit < units
                    u = np.minimum(unit, units - 1)
                    cq, rb = u // nb, u % nb
                    l16 = LANES & 15
                    gr, gc = grow0 + 4 * cq + (l16 & 3), gcol0 + 32 * rb + 8 * (l16 >> 2)
                    if guard:
                        on = on & (gr < M) & (gc < M)
                    store(gr, gc, on)

        if not diag:
            mirror_out(rp, tile, 0, n0, m0 + h * rp)
        elif (h + 1) * rp > tm:
            lo = tm if npass == 1 else 0
            mirror_out(tm, tm, lo, n0, m0 + h * rp + lo)
    return direct, mirror


def gemm_epilogue_accesses(cfg, M, N, m0, n0, xmat, out):
    tile_m, tile_n, wgm, wgn, _ = CFGS[cfg]
    tm, tn = tile_m // wgm, tile_n // wgn
    assert tn in (32, 64, 128)
    lpr = tn // 8
    rpi = 64 // lpr
    nit = MI // rpi
    hits = np.zeros((tile_m, tile_n // 8), dtype=np.int32)
    for wave in range(NW):
        wm, wn = wave % wgm, wave // wgm
        rr, cc = LANES // lpr, (LANES % lpr) * 8
        for i in range(tm // MI):
            for t in range(nit):
                m = m0 + wm * tm + i * MI + t * rpi + rr
                n = n0 + wn * tn + cc
                xmat.check(m, n, 8, "Cin fetch")
                out.check(m, n, 8, "store")
                np.add.at(hits, (m - m0, (n - n0) // 8), 1)
    assert (hits == 1).all()


# ------------------------------------------------------------------ the launcher
def launch_fast(cfg, p_ks, q_ks, mode, M, N, K):
    """Mirrors launch_fast: ('refused', why) or ('ok', edge, tiles_m, tiles_n, grid)."""
    tile_m, tile_n = CFGS[cfg][:2]
    if K < BK or K % BK:
        return ("refused", "K")
    tiles_m, tiles_n = -(-M // tile_m), -(-N // tile_n)
    grid = tiles_m * (tiles_m + 1) // 2 if mode == "syrk" else tiles_m * tiles_n
    if mode == "syrk":
        g = round_size(cfg)
        grid = grid // g * g + 8 * ((grid % g + 7) // 8)
    edge = M % tile_m != 0 or N % tile_n != 0
    if edge and not (mode == "syrk" and not p_ks and not q_ks):
        return ("refused", "edge")
    return ("ok", edge, tiles_m, tiles_n, grid)


def sample(seq, limit):
    """First, last and an evenly spread selection of `seq` (the checks are per tile; the extremes matter most)."""
    seq = list(seq)
    if len(seq) <= limit:
        return seq
    idx = sorted(set([0, 1, len(seq) - 2, len(seq) - 1] + list(range(0, len(seq), max(len(seq) // limit, 1)))))
    return [seq[i] for i in idx]


SYRK_NS = [256, 384, 512, 768, 1024, 1032, 1096, 1152, 1280, 1536, 1792, 1800, 2048, 2304, 3072, 4096, 5120, 8192, 8184]
SYRK_KS = [64, 128, 192, 1024, 14336]


@pytest.mark.parametrize("cfg,p_ks,q_ks,mode", [i for i in INSTANCES if i[3] == "syrk"])
def test_lower_triangle_launches_stay_inside_their_matrices(cfg, p_ks, q_ks, mode):
    tile = CFGS[cfg][0]
    launched = refused = 0
    for n, k in itertools.product(SYRK_NS, SYRK_KS):
        res = launch_fast(cfg, p_ks, q_ks, mode, n, n, k)
        if res[0] == "refused":
            assert n % tile != 0 and p_ks  # the only refusals: a K-strided operand whose last tile would overhang
            refused += 1
            continue
        _, edge, tiles_m, _, grid = res
        launched += 1
        assert edge == (n % tile != 0)
        tiles = [t if t is None else t[1] for t in syrk_grid_tiles(tiles_m, 1, round_size(cfg))]
        assert len(tiles) == grid
        nk = k // BK
        out = Matrix("D", n, n)
        cmat = Matrix("C", n, n)
        real = [t for t in tiles if t is not None]
        # corner tiles, the last block row (where the overhang is), diagonal and off-diagonal ones
        last_row = [t for t in real if t[0] == tiles_m - 1]
        picks = [(0, 0), (min(1, tiles_m - 1), 0), last_row[0], last_row[len(last_row) // 2], last_row[-1]] + sample(real, 4)
        for tm_, tn_ in dict.fromkeys(picks):
            m0, n0 = tm_ * tile, tn_ * tile
            for ks, row0, what in ((p_ks, m0, "P"), (q_ks, n0, "Q")):
                check_operand(n, k, ks, tile, edge, row0, sorted({0, nk - 1}), what)
            if k != SYRK_KS[0]:
                continue  # the epilogue does not depend on K
            for skip_upper, addends in ((False, True), (True, False)):
                diag = tm_ == tn_
                direct, mirror = syrk_epilogue_accesses(cfg, n, m0, n0, diag, edge, skip_upper, addends, out, cmat)
                # what ends up stored, each element once: the part of the tile inside the matrix (on a diagonal tile
                # with the upper triangle skipped: without the block above the diagonal blocks) and, unless skipped,
                # its mirror image
                rr, cc = np.meshgrid(np.arange(tile), np.arange(tile), indexing="ij")
                inside = (m0 + rr < n) & (n0 + cc < n)
                if diag and skip_upper:
                    inside &= cc < (rr // (tile // 2) + 1) * (tile // 2)
                assert (direct == inside).all()
                if not diag:
                    want_mirror = ((n0 + rr < n) & (m0 + cc < n)) if not skip_upper else np.zeros_like(inside)
                    assert (mirror == want_mirror).all()
    assert launched > 0
    assert (refused > 0) == p_ks


GEMM_SHAPES = [(1024, 1024), (1024, 2304), (2048, 4096), (4096, 4096), (4096, 14336), (1792, 4096), (1280, 1536), (128, 512),
               (384, 768), (896, 256), (128, 4096), (256, 1024), (1000, 2048), (1024, 1032), (1032, 2048)]


@pytest.mark.parametrize("cfg,p_ks,q_ks,mode", [i for i in INSTANCES if i[3] == "gemm"])
def test_gemm_launches_stay_inside_their_matrices(cfg, p_ks, q_ks, mode):
    """GEMM+AXPY  OUT = beta X + alpha B X.  x_trans == 0: P = B (m x m, K-contiguous), Q[j][k] = X[k][j] (K-strided),
    OUT and Cin are (m x n).  x_trans != 0: P = X^T (n x m), Q = B, OUT (n x m).  Shapes the tiles do not divide are
    refused by the launcher (the callers never send them)."""
    tile_m, tile_n = CFGS[cfg][:2]
    launched = 0
    for m, n in GEMM_SHAPES:
        M, N, K = (m, n, m) if q_ks else (n, m, m)
        res = launch_fast(cfg, p_ks, q_ks, mode, M, N, K)
        if res[0] == "refused":
            assert M % tile_m or N % tile_n or K % BK
            continue
        _, edge, tiles_m, tiles_n, grid = res
        assert not edge and grid == tiles_m * tiles_n
        launched += 1
        nk = K // BK
        out = Matrix("OUT", M, N)
        pids = sample(range(grid), 10)
        for pid in pids:
            tm_, tn_ = gemm_tile_of(pid, tiles_m, tiles_n)
            assert 0 <= tm_ < tiles_m and 0 <= tn_ < tiles_n
            m0, n0 = tm_ * tile_m, tn_ * tile_n
            check_operand(M, K, p_ks, tile_m, False, m0, sorted({0, nk - 1}), "P")
            check_operand(N, K, q_ks, tile_n, False, n0, sorted({0, nk - 1}), "Q")
            gemm_epilogue_accesses(cfg, M, N, m0, n0, Matrix("Cin", M, N), out)
    assert launched > 0


def test_tail_split_of_the_wide_gemm():
    """batch 1, m = 4096, n = 14336 on 256 CUs: the last 2048 columns run as 256 x 128 tiles on pointers advanced by
    `main_cols` elements; every access of both launches must stay inside the original matrices."""
    m, n, cus = 4096, 14336, 256
    tm, tn = m // 256, n // 256
    rem = (tm * tn) % cus
    assert rem > 0 and rem * 2 <= cus and rem % tm == 0 and tn > rem // tm
    tail_cols = (rem // tm) * 256
    main_cols = n - tail_cols
    tiles_main, tiles_tail = tm * (main_cols // 256), tm * (tail_cols // 128)
    assert (tiles_main, tiles_tail) == (768, 256)
    nk = m // BK
    for cfg, width, col_off in (("CfgBig", main_cols, 0), ("CfgHalfN", tail_cols, main_cols)):
        tile_m, tile_n = CFGS[cfg][:2]
        res = launch_fast(cfg, False, True, "gemm", m, width, m)
        assert res[0] == "ok" and not res[1]
        _, _, tiles_m, tiles_n, grid = res
        xfull = Matrix("X", m, n)   # Q is X (k x columns) with ld = n; the tail launch starts `col_off` columns in
        for pid in sample(range(grid), 12):
            tm_, tn_ = gemm_tile_of(pid, tiles_m, tiles_n)
            m0, n0 = tm_ * tile_m, tn_ * tile_n
            check_operand(m, m, False, tile_m, False, m0, [0, nk - 1], "B")
            for kt in (0, nk - 1):
                for wave in range(NW):
                    r, k = loader_accesses(tile_n, True, False, n0, width, kt, wave)
                    xfull.check(k, r + col_off, 8, "X")
        # partial-sum slots of both launches share one array of tiles_main + tiles_tail entries
        base = 0 if cfg == "CfgBig" else tiles_main
        assert base + grid <= tiles_main + tiles_tail


def test_tail_split_by_rows_of_a_batched_gemm():
    """8 x (1792 x 4096) on 256 CUs: 896 tiles of 256 x 256 leave half a round, which is the last tile row of every
    matrix; it runs as 256 x 128 tiles on pointers advanced by `main_rows` rows.  Every access of both launches must stay
    inside the matrices of its batch entry."""
    m, n, batch, cus = 1792, 4096, 8, 256
    tm, tn = m // 256, n // 256
    rem = (tm * tn * batch) % cus
    assert rem == 128 and rem % (tm * batch) != 0 and rem % (tn * batch) == 0
    tail_rows = rem // (tn * batch) * 256
    main_rows = m - tail_rows
    tiles_main, tiles_tail = (main_rows // 256) * tn, (tail_rows // 256) * (n // 128)
    assert (tiles_main * batch) % cus == 0 and (tiles_main, tiles_tail) == (96, 32)
    nk = m // BK
    for cfg, rows, row_off in (("CfgBig", main_rows, 0), ("CfgHalfN", tail_rows, main_rows)):
        tile_m, tile_n = CFGS[cfg][:2]
        res = launch_fast(cfg, False, True, "gemm", rows, n, m)
        assert res[0] == "ok" and not res[1]
        _, _, tiles_m, tiles_n, grid = res
        assert grid == (tiles_main if cfg == "CfgBig" else tiles_tail)
        bfull, xfull = Matrix("B", m, m), Matrix("X", m, n)
        for pid in sample(range(grid), 12):
            tm_, tn_ = gemm_tile_of(pid, tiles_m, tiles_n)
            m0, n0 = tm_ * tile_m, tn_ * tile_n
            for kt in (0, nk - 1):
                for wave in range(NW):
                    r, k = loader_accesses(tile_m, False, False, m0, rows, kt, wave)
                    bfull.check(r + row_off, k, 8, "B")          # P starts `row_off` rows into B
                    r, k = loader_accesses(tile_n, True, False, n0, n, kt, wave)
                    xfull.check(k, r, 8, "X")
            # Cin and Out are X and X' advanced by the same rows
            gemm_epilogue_accesses(cfg, rows, n, m0, n0, Matrix("Cin", m - row_off, n), Matrix("OUT", m - row_off, n))
        base = 0 if cfg == "CfgBig" else tiles_main
        assert base + grid <= tiles_main + tiles_tail


@pytest.mark.parametrize("batch,m,n", [(32, 128, 4096), (2, 256, 1536), (4, 128, 1024), (1, 256, 1024)])
def test_split_k_gram_partials(batch, m, n):
    """Short, wide matrices: K slices of 512 columns run as extra batch entries of a 128 x 128-tile product whose
    operand offset is outer * (m n) + inner * 512; every load must stay inside its matrix and inside its slice."""
    splits = n // 512
    assert m % 128 == 0 and n % 512 == 0
    K = n // splits
    res = launch_fast("CfgT128", False, False, "gemm", m, m, K)
    assert res[0] == "ok" and not res[1]
    _, _, tiles_m, tiles_n, grid = res
    for y in sample(range(batch * splits), 8):
        outer, inner = divmod(y, splits)
        assert outer < batch
        for pid in range(grid):
            tm_, tn_ = gemm_tile_of(pid, tiles_m, tiles_n)
            for row0, what in ((tm_ * 128, "P"), (tn_ * 128, "Q")):
                check_operand(m, K, False, 128, False, row0, [0, K // BK - 1], what, k_off=inner * K, k_total=n)
            gemm_epilogue_accesses("CfgT128", m, m, tm_ * 128, tn_ * 128, Matrix("none", m, m), Matrix("partial", m, m))


def test_k_strided_edge_tiles_are_refused_not_clamped():
    """A K-strided tile that overhangs the matrix would read past the end of each k-row (16-byte loads cannot be
    clamped per element): the launcher must refuse it, and the loader has no such variant."""
    for cfg, p_ks, q_ks, mode in INSTANCES:
        tile_m, tile_n = CFGS[cfg][:2]
        if p_ks or q_ks:
            assert launch_fast(cfg, p_ks, q_ks, mode, 4096 + 8, 4096 + 8, 1024) == ("refused", "edge")
        assert launch_fast(cfg, p_ks, q_ks, mode, 4096, 4096, 1000)[0] == "refused"   # K tail
    with pytest.raises(AssertionError):
        loader_accesses(256, True, True, 0, 1000, 0, 0)


# ------------------------------------------------------------------ split-tail (stream-K) launch of the 256 x 256 lower-triangle kernel
MAX_STREAMK_SPLITS = 8


def streamk_plan(tiles, k_tiles, cus):
    rounds, rem = divmod(tiles, cus)
    splits = min(cus // rem, MAX_STREAMK_SPLITS, k_tiles) if rem else 0
    return rounds, rem, (splits if splits >= 2 else 0)


def streamk_launches(tiles, nk_full, cus):
    """Replays launch_streamk's geometry and the workgroup decoding of gemm_fast_kernel<..., SK_WHOLE / SK_PARTS /
    SK_FINISH>: (whole, parts, finish) with whole = [(workgroup, tile)], parts = [(workgroup, tile, k_first, nk, image
    slot)], finish = [(workgroup, tile, [image slots in the order they are added])]; padding workgroups left out."""
    rounds, rem, splits = streamk_plan(tiles, nk_full, cus)
    split = splits > 1
    sk_whole = rounds * cus if split else tiles  # (computed whole by an ordinary launch limited to these tiles)
    tpx = (rem + 7) // 8 if split else 1
    whole, parts, finish = [(bid, bid) for bid in range(sk_whole)], [], []
    if split:
        for bid in range(8 * tpx * splits):
            t, sp = (bid % 8) * tpx + (bid // 8) % tpx, (bid // 8) // tpx
            if t >= rem or sp >= splits:
                continue
            k_first = nk_full * sp // splits
            parts.append((bid, sk_whole + t, k_first, nk_full * (sp + 1) // splits - k_first, sp * rem + t))
        for bid in range(4 * rem):  # four workgroups per left-over tile, one per 128 x 128 quarter
            if bid % 4 == 0:
                finish.append((bid, sk_whole + bid // 4, [sp * rem + bid // 4 for sp in range(splits)]))
    return whole, parts, finish, (rounds, rem, splits)


def test_split_tail_image_layout():
    """SK_PARTS (256 x 256 tile, 2 x 2 wavefronts of 128 x 128, 8 x 8 fragments each) stores fragment (I, J) of thread t
    at float4 ((I 8 + J) 256 + t) of the image; SK_FINISH (128 x 128 tile = one quarter, 2 x 2 wavefronts of 64 x 64,
    4 x 4 fragments each) reads fragment (i, j) of its wavefront (wm, wn) from ((wm 4 + i) 8 + wn 4 + j) 256 + quarter
    64 + lane.  Both must name the same element of the tile, every element once, inside the image."""
    lane = np.arange(64)
    where = {}
    for wave in range(4):  # SK_PARTS: wavefront = row half + 2 * column half
        WM, WN = wave % 2, wave // 2
        for I in range(8):
            for J in range(8):
                idx = (I * 8 + J) * 256 + wave * 64 + lane
                rows = WM * 128 + 16 * I + (lane & 15)
                cols = WN * 128 + 16 * J + 4 * (lane >> 4)
                for a, r, c in zip(idx, rows, cols):
                    where[int(a)] = (int(r), int(c))
    assert sorted(where) == list(range(256 * 64))  # 65536 float4 = one image
    seen = set()
    for quarter in range(4):
        qm, qn = quarter % 2, quarter // 2
        for wave in range(4):
            wm, wn = wave % 2, wave // 2
            for i in range(4):
                for j in range(4):
                    idx = ((wm * 4 + i) * 8 + wn * 4 + j) * 256 + quarter * 64 + lane
                    rows = qm * 128 + wm * 64 + 16 * i + (lane & 15)
                    cols = qn * 128 + wn * 64 + 16 * j + 4 * (lane >> 4)
                    for a, r, c in zip(idx, rows, cols):
                        assert where[int(a)] == (int(r), int(c))
                        seen.add(int(a))
    assert len(seen) == 256 * 64


@pytest.mark.parametrize("batch,n,k", [(16, 2048, 8192), (1, 1024, 8192), (3, 1280, 1024), (2, 1536, 4096), (1, 4096, 14336),
                                       (7, 1024, 64), (1, 2048, 128), (5, 1792, 448), (5, 1024, 448), (64, 1024, 256)])
@pytest.mark.parametrize("cus", [256, 248, 8, 304])
def test_split_tail_schedule(batch, n, k, cus):
    t, nk_full = n // 256, k // 64
    tiles = t * (t + 1) // 2 * batch
    whole, parts, finish, (rounds, rem, splits) = streamk_launches(tiles, nk_full, cus)
    assert splits == 0 or (2 <= splits and rem * splits <= cus)  # the split round is a single round
    # every K tile of every tile is multiplied exactly once, inside the K range of the operands
    cover = np.zeros((tiles, nk_full), dtype=np.int32)
    for _, tile in whole:
        assert 0 <= tile < tiles
        cover[tile] += 1
    for _, tile, k0, cnt, _ in parts:
        assert 0 <= tile < tiles and 0 <= k0 and cnt > 0 and (k0 + cnt) * 64 <= k
        cover[tile, k0:k0 + cnt] += 1
    assert (cover == 1).all()
    # every part has an image slot of its own inside the workspace the launcher asks for, and the finishing
    # workgroup of a tile adds exactly the images of that tile's parts, every left-over tile once
    n_images = rem * splits
    assert sorted(slot for *_, slot in parts) == list(range(n_images))
    assert sorted(tile for _, tile, _ in finish) == sorted({tile for _, tile, *_ in parts})
    for _, tile, slots in finish:
        assert sorted(slots) == sorted(slot for _, tl, _, _, slot in parts if tl == tile)
    # the workgroups of one XCD (workgroup id % 8) that run at the same time work on neighbouring tiles
    if splits:
        for x in range(8):
            mine = [tile for bid, tile, k0, *_ in parts if bid % 8 == x and k0 == 0]
            assert mine == list(range(mine[0], mine[0] + len(mine))) if mine else True


# ------------------------------------------------------------------ per-head slab kernel (inst_head_apply.hip)
@pytest.mark.parametrize("batch,n", [(32, 4096), (3, 1024), (1, 2048), (5, 512)])
def test_head_apply_global_accesses(batch, n):
    """One workgroup of 512 threads per (matrix, 512-column slice): every global access of S (128 x 128), of X and X'
    (128 x n), of the partial Gram matrices ([batch][slices][128][128] float32) and of the partial sums of squares
    ([batch][slices]) lies inside its array, every element of X' is written once, and the partial Gram matrix of
    every slice has its lower triangle written once."""
    m, split, w = 128, 512, 128
    splits = n // split
    assert n % split == 0
    tid = np.arange(512)
    lane, wave = tid & 63, tid >> 6
    # S fragments: 16 bytes at row 16 wave + lane % 16, k = 32 q + 8 (lane / 16)
    for q in range(4):
        row, k = 16 * wave + (lane & 15), 32 * q + 8 * (lane >> 4)
        assert (row < m).all() and (k + 8 <= m).all()
    written = np.zeros((batch, m, n), dtype=np.int32)
    for wg in sample(range(batch * splits), 6):
        b, s = divmod(wg, splits)
        assert b < batch
        for t in range(split // w):
            for u in range(4):  # slab <-> threads, loads of X and stores of the bf16 X'
                row, col = (tid >> 4) + 32 * u, s * split + t * w + 8 * (tid & 15)
                assert (row < m).all() and (col + 8 <= n).all()
                for r, c in zip(row, col):
                    written[b, r, c:c + 8] += 1
            for j in range(8):  # float32 stores of the last group: row 16 wave + lane % 16, four columns
                row, col = 16 * wave + (lane & 15), s * split + t * w + 16 * j + 4 * (lane >> 4)
                assert (row < m).all() and (col + 4 <= n).all()
        assert (written[b, :, s * split:(s + 1) * split] == 1).all()
        # partial Gram matrix of slice (b, s): wavefront w, column blocks 0 .. w
        g = np.zeros((m, m), dtype=np.int32)
        for wv in range(8):
            for j in range(wv + 1):
                for ln in range(64):
                    r, c = 16 * wv + (ln & 15), 16 * j + 4 * (ln >> 4)
                    off = (b * splits + s) * m * m + r * m + c
                    assert 0 <= off and off + 4 <= batch * splits * m * m
                    g[r, c:c + 4] += 1
        assert (np.tril(g) == np.tril(np.ones_like(g))).all() and g.max() == 1
        assert b * splits + s < batch * splits  # slot of the partial sum of squares


@pytest.mark.parametrize("batch,n", [(32, 4096), (3, 1024), (1, 2048), (5, 512)])
def test_head_front_global_accesses(batch, n):
    """The input pass of 128-row matrices (head_front_kernel), one workgroup of 512 threads per (matrix, 512-column
    slice): a thread reads two 16-byte groups of float32 (eight columns) per 32 rows and slab and writes the 16 bytes
    of bf16 they become; every element of x is read once and every element of the copy written once, inside their
    arrays; the partial sums ([batch][slices] float64) and the partial Gram matrices are indexed as the consumers
    index them."""
    m, split, w = 128, 512, 128
    splits = n // split
    tid = np.arange(512)
    ck, cc = tid >> 4, tid & 15
    for wg in sample(range(batch * splits), 6):
        b, s = divmod(wg, splits)
        seen = np.zeros((m, split), dtype=np.int32)
        base = b * m * n + s * split + 8 * cc
        for t in range(split // w):
            for u in range(4):
                at = base + (ck + 32 * u) * n + t * w
                for h in range(2):
                    lo = at + 4 * h
                    assert (lo >= b * m * n).all() and (lo + 4 <= (b + 1) * m * n).all() and (lo % 4 == 0).all()
                assert (at % 8 == 0).all()  # 16-byte alignment of the bf16 store
                rows, cols = (at - b * m * n) // n, (at - b * m * n) % n - s * split
                assert (cols >= 0).all() and (cols + 8 <= split).all()
                for r, c in zip(rows, cols):
                    seen[r, c:c + 8] += 1
        assert (seen == 1).all()
        assert 0 <= b * splits + s < batch * splits


def transposed_store_elements(cfg, m0, n0, ldo, base):
    """Element offsets (into the transposed float32 result, element (m, n) at n * ldo + m) of the 16-byte stores that
    the staged GEMM epilogue issues for the tile at (m0, n0) when p.out_transposed is set: per wavefront and 16-row
    block, lane l takes rows 4 (l / 16) .. + 3 of column 16 t + l % 16."""
    tile_m, tile_n, wgm, wgn, _ = CFGS[cfg]
    tm, tn = tile_m // wgm, tile_n // wgn
    col, g4 = LANES & 15, 4 * (LANES >> 4)
    out = []
    for wave in range(NW):
        wm, wn = wave % wgm, wave // wgm
        for i in range(tm // MI):
            for t in range(tn // 16):
                out.append(base + (n0 + wn * tn + 16 * t + col) * ldo + m0 + wm * tm + i * MI + g4)
    return np.concatenate(out)


@pytest.mark.parametrize("m,n,batch", [(4096, 14336, 1), (1792, 4096, 8), (1024, 1024, 1), (1024, 2304, 2), (256, 512, 3)])
def test_transposed_output_of_the_staged_gemm_epilogue(m, n, batch):
    """Tall inputs: the last product writes its float32 result transposed, (n x m) row-major.  Over the launches of
    one product (one, or a main and a tail launch whose output pointer is advanced by main_cols * ldo or by main_rows
    elements) every element of every transposed matrix is written exactly once, by a 16-byte aligned store."""
    cus, ldo = 256, m
    tm, tn = m // 256, n // 256
    launches = []  # (cfg, rows, cols, element offset of the launch's output inside a batch entry)
    if m >= 1024:
        rem = (tm * tn * batch) % cus
        tail_cols = tail_rows = 0
        if rem > 0 and rem * 2 <= cus:
            if rem % (tm * batch) == 0 and rem // (tm * batch) < tn:
                tail_cols = rem // (tm * batch) * 256
            elif rem % (tn * batch) == 0 and rem // (tn * batch) < tm:
                tail_rows = rem // (tn * batch) * 256
        if tail_cols:
            launches = [("CfgBig", m, n - tail_cols, 0), ("CfgHalfN", m, tail_cols, (n - tail_cols) * ldo)]
        elif tail_rows:
            launches = [("CfgBig", m - tail_rows, n, 0), ("CfgHalfN", tail_rows, n, m - tail_rows)]
        else:
            launches = [("CfgBig", m, n, 0)]
        assert (m, n, batch) != (4096, 14336, 1) or tail_cols == 2048
        assert (m, n, batch) != (1792, 4096, 8) or tail_rows == 256
    else:
        launches = [("CfgM128", m, n, 0)]
    b = batch - 1
    written = np.zeros(n * m, dtype=np.int32)
    for cfg, rows, cols, off in launches:
        tile_m, tile_n = CFGS[cfg][:2]
        assert rows % tile_m == 0 and cols % tile_n == 0 and ldo >= m and ldo % 4 == 0
        for m0 in range(0, rows, tile_m):
            for n0 in range(0, cols, tile_n):
                at = transposed_store_elements(cfg, m0, n0, ldo, off)
                assert (at % 4 == 0).all() and (at >= 0).all() and (at + 4 <= n * m).all()
                for e in range(4):
                    np.add.at(written, at + e, 1)
    assert (written == 1).all()
    assert (b * n * m + n * m) <= batch * n * m
