"""Host model of the fast kernel's operand staging (emerging-optimizers_amd/csrc/gemm_fast.hpp).

The direct-to-LDS loader (``FastLoader``, uniform-base form) and the fragment readers (``fast_frag``,
``fast_frag16_ks``) are written independently in the kernel; they only work together if every 16-byte chunk a
load drops into LDS is the one the MFMA fragment read of that position expects.  This model restates both sides
lane by lane and checks, for every configuration the library instantiates,
  * every global offset stays inside the operand tile and every chunk of the tile is fetched exactly once,
  * the K-contiguous fragment read returns (row, k-chunk) of its lane,
  * the LDS transpose read (result lane i, element e <- source lane 4e + i/4, element i%4 of a 16-lane group)
    hands lane i the four k-values of its own row,
  * the compact address form of the 16 x 16 shape equals the direct formula,
  * one pass of a read instruction (16 lanes of a 16-byte read, 32 lanes of an 8-byte read) touches every LDS
    bank at most once.
No GPU is involved: this is the check that runs before a new layout is allowed on the device.
"""
import itertools

import pytest


def kc_slot(bk, row, c):
    return c ^ ((row >> 1) & 7) if bk == 64 else c ^ ((row >> 2) & 3)


def ks_rot(mi, k):
    return 4 * k if mi == 32 else 2 * (k & 7) + 8 * (k >> 3)


def run_model(mi, bk, nw, ks, rows, ld=5000):
    ki = 16 if mi == 32 else 32
    lpt = rows * bk * 2 // 1024 // nw
    cpr, rpkb, ksc, ksr = bk // 8, 1024 // (bk * 2), rows // 8, 512 // rows
    if ks:
        period = max(ksc // (4 * ksr), 1) if mi == 32 else max(ksc // ksr, 1)
    else:
        period = 2 if bk == 64 else 1
    periodic = lpt % period == 0
    nv = min(period, lpt) if periodic else lpt

    def lane_part(b, lane):
        if not ks:
            lr = lane // cpr
            return lr * ld + kc_slot(bk, rpkb * b + lr, lane % cpr) * 8
        kr = lane // ksc
        return kr * ld + (((lane % ksc) - ks_rot(mi, ksr * b + kr)) & (ksc - 1)) * 8

    lds = {}
    for wave in range(nw):
        b0 = wave * lpt
        for i in range(lpt):
            b = b0 + i
            for lane in range(64):
                v = (i % nv) if periodic else i
                off = lane_part(v if periodic else b0 + v, lane)
                first = (ksr * b0) * ld if ks else (rpkb * b0) * ld
                g = first + i * (ksr if ks else rpkb) * ld + off
                if not ks:
                    row, col = divmod(g, ld)
                    assert 0 <= row < rows and 0 <= col < bk and col % 8 == 0
                    ident = (row, col // 8)
                else:
                    k, col = divmod(g, ld)
                    assert 0 <= k < bk and 0 <= col < rows and col % 8 == 0
                    ident = ("ks", k, col // 8)
                pos = (b * 1024 + lane * 16) // 16
                assert pos not in lds
                lds[pos] = ident
    assert len(lds) == rows * bk * 2 // 16 == len(set(lds.values()))

    worst = 1
    for row_base in range(0, rows, mi):
        for q in range(bk // ki):
            addrs = []
            for lane in range(64):
                kgrp = lane >> 5 if mi == 32 else lane >> 4
                if not ks:
                    row = row_base + (lane & (mi - 1))
                    chunk = (ki // 8) * q + kgrp
                    byte = row * (bk * 2) + kc_slot(bk, row, chunk) * 16
                    assert lds[byte // 16] == (row, chunk)
                    addrs.append([byte])
                else:
                    i16 = lane & 15
                    col = row_base + (16 * ((lane >> 4) & 1) if mi == 32 else 0) + 4 * (i16 & 3)
                    kb = ki * q + 8 * kgrp + (i16 >> 2)
                    both = []
                    for k in (kb, kb + 4):
                        slot = ((col >> 3) + ks_rot(mi, k)) & (ksc - 1)
                        byte = k * rows * 2 + slot * 16 + (col & 7) * 2
                        assert lds[byte // 16] == ("ks", k, col >> 3)
                        both.append(byte)
                    addrs.append(both)
            if ks:
                for lane in range(64):
                    grp, i = lane & ~15, lane & 15
                    kgrp = lane >> 5 if mi == 32 else lane >> 4
                    for h in (0, 1):
                        for e in range(4):
                            src = grp + 4 * e + i // 4
                            s16 = src & 15
                            col = row_base + (16 * ((src >> 4) & 1) if mi == 32 else 0) + 4 * (s16 & 3) + (i % 4)
                            k = ki * q + 8 * kgrp + (s16 >> 2) + 4 * h
                            assert col == row_base + (lane & (mi - 1))
                            assert k == ki * q + 8 * kgrp + 4 * h + e
                for h in (0, 1):
                    for p0 in (0, 32):
                        banks = [((addrs[lane][h] + 4 * w) // 4) % 64 for lane in range(p0, p0 + 32) for w in range(2)]
                        worst = max(worst, max(banks.count(x) for x in set(banks)))
            else:
                for p0 in range(0, 64, 16):
                    banks = [((addrs[lane][0] + 4 * w) // 4) % 64 for lane in range(p0, p0 + 16) for w in range(4)]
                    worst = max(worst, max(banks.count(x) for x in set(banks)))
    return worst


CONFIGS = [
    (mi, bk, nw, ks, rows)
    for mi, bk, nw, ks, rows in itertools.product((16,), (64,), (4,), (False, True), (256, 128, 192))
    if not (ks and rows == 192) and rows * bk * 2 % (1024 * nw) == 0
]


@pytest.mark.parametrize("mi,bk,nw,ks,rows", CONFIGS)
def test_loader_and_fragment_reads_agree_and_are_conflict_free(mi, bk, nw, ks, rows):
    assert run_model(mi, bk, nw, ks, rows) == 1


@pytest.mark.parametrize("rows", [256, 128])
def test_compact_transpose_read_address_equals_direct_formula(rows):
    ch, rowb = rows // 8, rows * 2
    for wb in range(0, rows, 32):
        for lane in range(64):
            g, i16 = lane >> 4, lane & 15
            kk, cq = i16 >> 2, i16 & 3
            s = (wb // 8 + (cq >> 1) + 2 * kk + 8 * g) * 16 + (cq & 1) * 8
            r0 = (8 * g + kk) * rowb
            for r in range((rows - wb) // 16):
                for q in (0, 1):
                    a0 = (((s + 2 * r * 16) & (rowb - 1)) | r0) + 32 * q * rowb
                    a1 = (((s + (2 * r + 8) * 16) & (rowb - 1)) | r0) + (32 * q + 4) * rowb
                    col, kb = wb + 16 * r + 4 * (i16 & 3), 32 * q + 8 * g + (i16 >> 2)
                    ref = [k * rowb + (((col >> 3) + ks_rot(16, k)) & (ch - 1)) * 16 + (col & 7) * 2 for k in (kb, kb + 4)]
                    assert [a0, a1] == ref


# ---- SYRK-mode epilogue: tile assembled row-major in LDS, mirror image formed with the LDS transpose read ----
#
# Restates `syrk_epilogue_lds` lane by lane: staging of the accumulator quads, the in-LDS fill of the upper 4 x 4
# blocks of a diagonal wavefront block, the row-wise write-out and the transposed write-out.  The check is that
# global memory ends up holding exactly the lower-triangle values and their mirror image, every element written
# once, for every tile shape the library instantiates.


def tr_read(lds, addr_of_lane):
    """ds_read_b64_tr_b16: result lane i, element e <- source lane 4e + i/4, element i%4 (per 16-lane group)."""
    out = []
    for lane in range(64):
        grp, i = lane & ~15, lane & 15
        out.append([lds.get(addr_of_lane[grp + 4 * e + i // 4] + 2 * (i % 4)) for e in range(4)])
    return out


def syrk_epilogue_model(tile, mi, npass, diag, skip_upper=False):
    tm = tile // 2
    ldt, rp = tile + 8, tile // npass
    g_cnt = 4 if mi == 32 else 1
    fm = tm // mi
    sym, mirror = diag and not skip_upper, not skip_upper
    m0, n0 = (tile, tile) if diag else (2 * tile, 0)
    out = {}

    def value(ml, nl):  # what the accumulators of the wavefront owning (ml, nl) hold
        return ("v", ml, nl)

    def store(row, col, vals):
        for t, v in enumerate(vals):
            assert (row, col + t) not in out, "element written twice"
            out[(row, col + t)] = v

    for h in range(npass):
        lds = {}

        def put(row, col, v):
            assert 0 <= row < rp and 0 <= col < tile
            lds[(row * ldt + col) * 2] = v

        # staging
        for wave in range(4):
            wm, wn = wave // 2, wave % 2
            mw, nw = wm * tm, wn * tm
            if mw // rp != h:
                continue
            for lane in range(64):
                frow, fk = lane & (mi - 1), lane // mi
                for i in range(fm):
                    for j in range(fm):
                        for g in range(g_cnt):
                            ml, nl = mw + i * mi + frow, nw + j * mi + (8 * g if mi == 32 else 0) + 4 * fk
                            quad = [value(ml, nl + r) for r in range(4)]
                            if not sym or wm > wn:
                                for r in range(4):
                                    put(ml - h * rp, nl + r, quad[r])
                            elif wm == wn:
                                if i > j or (i == j and nl < (ml & ~3)):
                                    for r in range(4):
                                        put(ml - h * rp, nl + r, quad[r])
                                elif i == j and nl == (ml & ~3):
                                    for r in range(4):
                                        if nl + r <= ml:
                                            put(ml - h * rp, nl + r, quad[r])
                                        if nl + r < ml:
                                            put(nl + r - h * rp, ml, quad[r])
        # upper 4 x 4 blocks of a diagonal wavefront block
        if sym:
            for wave in (0, 3):
                mw = (wave // 2) * tm
                if mw // rp != h:
                    continue
                nb4 = tm // 4
                assert nb4 * nb4 % 16 == 0
                rowbase, colbase = mw - h * rp, mw
                for it in range(nb4 * nb4 // 16):
                    addr = []
                    for lane in range(64):
                        ids = it * 16 + 4 * (lane // 16) + (lane % 4)
                        brs, bcs, e = ids // nb4, ids % nb4, (lane % 16) // 4
                        addr.append(((rowbase + 4 * brs + e) * ldt + colbase + 4 * bcs) * 2)
                    got = tr_read(lds, addr)
                    for lane in range(64):
                        idr = it * 16 + lane // 4
                        br, bc, r = idr // nb4, idr % nb4, lane % 4
                        if br > bc:
                            for t in range(4):
                                put(rowbase + 4 * bc + r, colbase + 4 * br + t, got[lane][t])
        # row-wise write-out
        cprw = tile // 8
        assert rp * cprw % 256 == 0
        for it in range(rp * cprw // 256):
            for tid in range(256):
                c = tid + it * 256
                row, c8 = c // cprw, c % cprw
                ml = h * rp + row
                if diag and c8 * 8 >= (ml // tm + 1) * tm:
                    continue
                store(m0 + ml, n0 + c8 * 8, [lds[(row * ldt + c8 * 8 + t) * 2] for t in range(8)])
        # transposed write-out
        if mirror:
            if sym:
                lo, hi = max(tm, h * rp), min(tile, (h + 1) * rp)
                r_lo, rows, ccols = lo - h * rp, max(hi - lo, 0), tm
            else:
                r_lo, rows, ccols = 0, rp, tile
            assert rows % 32 == 0
            nb = rows // 32
            units = (ccols // 4) * nb
            for it in range((units + 15) // 16):
                for wave in range(4):
                    addr0, meta = [], []
                    for lane in range(64):
                        unit = it * 16 + wave * 4 + lane // 16
                        on = unit < units
                        u = min(unit, max(units - 1, 0))
                        cq, rb = (u // nb, u % nb) if nb else (0, 0)
                        L = lane % 16
                        addr0.append(((r_lo + 32 * rb + 8 * (L % 4) + L // 4) * ldt + 4 * cq) * 2)
                        meta.append((on, cq, rb, L // 4, L % 4))
                    if units == 0:
                        continue
                    t0 = tr_read(lds, addr0)
                    t1 = tr_read(lds, [a + 4 * ldt * 2 for a in addr0])
                    for lane in range(64):
                        on, cq, rb, q, r = meta[lane]
                        if on:
                            store(n0 + 4 * cq + r, m0 + h * rp + r_lo + 32 * rb + 8 * q, t0[lane] + t1[lane])
    return out, (m0, n0)


@pytest.mark.parametrize("tile,mi,npass", [(192, 16, 1), (256, 16, 1), (128, 16, 1)])
@pytest.mark.parametrize("diag", [False, True])
def test_syrk_epilogue_writes_the_tile_and_its_mirror_image(tile, mi, npass, diag):
    out, (m0, n0) = syrk_epilogue_model(tile, mi, npass, diag)
    expect = {}
    for a in range(tile):
        for b in range(tile):
            if diag:
                expect[(m0 + a, n0 + b)] = ("v", max(a, b), min(a, b))
            else:
                expect[(m0 + a, n0 + b)] = ("v", a, b)
                expect[(n0 + b, m0 + a)] = ("v", a, b)
    assert out == expect


@pytest.mark.parametrize("tile,npass", [(192, 1), (256, 1)])
def test_syrk_epilogue_lower_only(tile, npass):
    out, (m0, n0) = syrk_epilogue_model(tile, 16, npass, diag=False, skip_upper=True)
    assert out == {(m0 + a, n0 + b): ("v", a, b) for a in range(tile) for b in range(tile)}


@pytest.mark.parametrize("tile,npass", [(192, 1), (256, 1), (128, 1)])
def test_syrk_epilogue_lower_only_on_a_diagonal_tile(tile, npass):
    """With the upper triangle skipped, a diagonal tile stores its two diagonal blocks whole and the block below them;
    the block above the diagonal (whose wavefront computes nothing) must stay unwritten."""
    out, (m0, n0) = syrk_epilogue_model(tile, 16, npass, diag=True, skip_upper=True)
    tm = tile // 2
    assert out == {(m0 + a, n0 + b): ("v", a, b) for a in range(tile) for b in range(tile) if b < (a // tm + 1) * tm}


# ---- per-head product kernel (inst_head_apply.hip): a 128 x 128 slab of X in the K-strided tile layout ----
#
# The slab is parked by `park_slab` (row k = thread / 16 + 16 u, chunk = thread % 16, rotated by ks_rot), read as the
# Q operand of S X with `fast_frag16_ks<128>` for four k-steps (128 k-rows instead of the 64 of a ring slot), read and
# overwritten in place by the epilogue (row m, four columns), written out row-wise, and read as both operands of
# X' X'^T with plain 16-byte reads.  This restates each of them and checks them against each other.
HA_M, HA_W = 128, 128
HA_ROWB, HA_CH = HA_W * 2, HA_W // 8


def ha_chunk(k, c8):
    return k * HA_ROWB + ((c8 + ks_rot(16, k)) & (HA_CH - 1)) * 16


def test_head_apply_slab_layout():
    # park: every 16-byte chunk of the slab once, at an address of its own (512 threads, four chunks each)
    lds = {}
    for tid in range(512):
        for u in range(4):
            k, c8 = (tid >> 4) + 32 * u, tid & 15
            at = ha_chunk(k, c8)
            assert 0 <= at < HA_M * HA_ROWB and at % 16 == 0 and at // 16 not in lds
            lds[at // 16] = (k, c8)
    assert len(lds) == HA_M * HA_CH
    elem = {}  # byte address of a bf16 -> (k, column)
    for pos, (k, c8) in lds.items():
        for e in range(8):
            elem[pos * 16 + 2 * e] = (k, 8 * c8 + e)
    # Q fragments of S X: fragment (j, q), lane l must end up with X[32 q + 8 (l / 16) + 0 .. 7][16 j + l % 16]
    for j in range(HA_W // 16):
        for q in range(HA_M // 32):
            a_lo, a_hi = [], []
            for lane in range(64):
                g, i16 = lane >> 4, lane & 15
                kk, cq = i16 >> 2, i16 & 3
                s = ((cq >> 1) + 2 * kk + 8 * g) * 16 + (cq & 1) * 8  # ks16_consts with wave_row_base = 0
                r0 = (8 * g + kk) * HA_ROWB
                a_lo.append((((s + 2 * j * 16) & (HA_ROWB - 1)) | r0) + 32 * q * HA_ROWB)
                a_hi.append((((s + (2 * j + 8) * 16) & (HA_ROWB - 1)) | r0) + (32 * q + 4) * HA_ROWB)
            lo, hi = tr_read(elem, a_lo), tr_read(elem, a_hi)
            for lane in range(64):
                want = [(32 * q + 8 * (lane >> 4) + e, 16 * j + (lane & 15)) for e in range(8)]
                assert lo[lane] + hi[lane] == want
            for addrs in (a_lo, a_hi):  # one pass = 32 lanes of an 8-byte read: every bank at most once
                for p0 in (0, 32):
                    banks = [((addrs[lane] + 4 * w) // 4) % 64 for lane in range(p0, p0 + 32) for w in range(2)]
                    assert max(banks.count(x) for x in set(banks)) == 1
    # epilogue (8 wavefronts of 16 rows): a lane's four columns of row m are 8 contiguous bytes inside one chunk, each
    # element owned by one lane; the slab of X' uses the same addresses
    owners = {}
    for wave in range(8):
        for lane in range(64):
            for j in range(8):
                m, n = 16 * wave + (lane & 15), 16 * j + 4 * (lane >> 4)
                at = ha_chunk(m, n >> 3) + (n & 7) * 2
                assert at % 8 == 0
                for r in range(4):
                    assert elem[at + 2 * r] == (m, n + r)
                    assert (m, n + r) not in owners
                    owners[(m, n + r)] = (wave, lane)
    assert len(owners) == HA_M * HA_W
    # operands of X' X'^T: fragment rows 16 w + l % 16, k-step q: columns 32 q + 8 (l / 16) .. + 7 in one chunk
    for w in range(8):
        for q in range(4):
            for lane in range(64):
                row = 16 * w + (lane & 15)
                at = ha_chunk(row, 4 * q + (lane >> 4))
                assert [elem[at + 2 * e] for e in range(8)] == [(row, 32 * q + 8 * (lane >> 4) + e) for e in range(8)]
    # the partial Gram matrix: wavefront w writes rows 16 w .. + 15, column blocks 0 .. w: the lower triangle, each
    # element once
    seen = set()
    for wave in range(8):
        for lane in range(64):
            for j in range(wave + 1):
                m, n = 16 * wave + (lane & 15), 16 * j + 4 * (lane >> 4)
                for r in range(4):
                    assert (m, n + r) not in seen and m * HA_M + n + r < HA_M * HA_M
                    seen.add((m, n + r))
    assert all((m, n) in seen for m in range(HA_M) for n in range(m + 1))
    # and every float4 the chain kernel adds (groups of four columns starting at j <= i) lies inside what is written
    assert all((i, j + e) in seen for i in range(HA_M) for j in range(0, HA_M, 4) if j <= i for e in range(4))


# ---- chain kernel of the 128-row matrices (small_chain_kernel in mi_ns.hip): lower triangle stored, then mirrored ----
CH_M = 128


def ch_elem(row, col):
    return row * (CH_M * 2) + ((((col >> 3) ^ row) & 15) << 4) + (col & 7) * 2


def chain_mirror_model(lds):
    """`chain_mirror`: the 36 blocks of 16 x 16 on and below the diagonal, dealt out to 16 wavefronts; transpose read
    of 4 rows x 16 columns per 16-lane group, 8-byte store of the transposed piece (element-wise right of the diagonal
    inside a diagonal block).  Returns the set of (row, column) written."""
    written = []
    for wave in range(16):
        for sb in range(wave, 36, 16):
            bi = 0
            while (bi + 1) * (bi + 2) // 2 <= sb:
                bi += 1
            bj = sb - bi * (bi + 1) // 2
            assert 0 <= bj <= bi < 8
            addr = []
            for lane in range(64):
                patch, i16 = lane >> 4, lane & 15
                addr.append(ch_elem(16 * bi + 4 * patch + (i16 >> 2), 16 * bj + 4 * (i16 & 3)))
            got = tr_read(lds, addr)
            for lane in range(64):
                patch, i16 = lane >> 4, lane & 15
                dst_row, dst_col = 16 * bj + i16, 16 * bi + 4 * patch
                for r in range(4):
                    if bi != bj or dst_col + r > dst_row:
                        # the lane must hold source row 16 bi + 4 patch + r at source column 16 bj + i16 (what a
                        # diagonal block reads from above the diagonal is not there yet and is not used)
                        assert got[lane][r] == (16 * bi + 4 * patch + r, 16 * bj + i16)
                        written.append((dst_row, dst_col + r, got[lane][r]))
    return written


def test_chain_kernel_lower_triangle_then_mirror():
    # direct phase of a product: wavefront (ti, tj), tj <= ti, lane: row m = 32 ti + lane % 32, four columns from
    # n = 32 tj + 8 g + 4 (lane / 32); only what lies on or below the diagonal
    lds, count = {}, {}
    for wave in range(16):
        ti, tj = wave >> 2, wave & 3
        if tj > ti:
            continue
        for lane in range(64):
            for g in range(4):
                m, n = ti * 32 + (lane & 31), tj * 32 + 8 * g + 4 * (lane >> 5)
                for r in range(4):
                    if n + r <= m:
                        lds[ch_elem(m, n + r)] = (m, n + r)
                        count[(m, n + r)] = count.get((m, n + r), 0) + 1
                assert ch_elem(m, n) % 8 == 0 and [ch_elem(m, n + r) for r in range(4)] == [ch_elem(m, n) + 2 * r for r in range(4)]
    assert count == {(m, n): 1 for m in range(CH_M) for n in range(m + 1)}
    # the same for the build of D from the partial sums: the groups of four columns that start on or left of the
    # diagonal are numbered 33 per pair of rows (p, 127 - p); two per thread and 64 left over
    groups = []
    for g in range(64 * 33):
        pair, r = divmod(g, 33)
        n_lo = pair // 4 + 1
        groups.append((pair, 4 * r) if r < n_lo else (CH_M - 1 - pair, 4 * (r - n_lo)))
    assert len(groups) == 2 * 1024 + 64
    assert sorted(groups) == sorted((i, j) for i in range(CH_M) for j in range(0, CH_M, 4) if j <= i)
    built = set()
    for i, j in groups:
        built.update((i, j + e) for e in range(4) if j + e <= i)
    assert built == set(count)
    # mirror phase: everything right of the diagonal, once, and as the transpose of what is stored below it
    written = chain_mirror_model(lds)
    assert sorted((r, c) for r, c, _ in written) == [(r, c) for r in range(CH_M) for c in range(r + 1, CH_M)]
    assert all(src == (c, r) for r, c, src in written)
    # one pass of the transpose read (32 lanes x 8 bytes) touches every LDS bank at most once
    for bi in range(8):
        for bj in range(bi + 1):
            for half in (0, 32):
                banks = []
                for lane in range(half, half + 32):
                    patch, i16 = lane >> 4, lane & 15
                    a = ch_elem(16 * bi + 4 * patch + (i16 >> 2), 16 * bj + 4 * (i16 & 3))
                    banks += [(a // 4) % 64, (a // 4 + 1) % 64]
                assert max(banks.count(x) for x in set(banks)) <= 2


@pytest.mark.parametrize("tn", [64, 128])
def test_transposed_reads_of_the_gemm_staging_rows_are_conflict_free(tn):
    """Transposed float32 output of the staged GEMM epilogue: a 16-row block of a wavefront sits in LDS as float32 rows
    of tn values padded by 16 bytes; lane l reads rows 4 (l / 16) + e, e = 0 .. 3, of column 16 t + l % 16, four bytes
    at a time.  For every (t, e) the 64 lanes hit 64 different banks (4-byte banks, 64 of them), and together the reads
    cover every element of the block once."""
    rowb = tn * 4 + 16
    seen = [[0] * tn for _ in range(16)]
    for t in range(tn // 16):
        for e in range(4):
            banks = set()
            for lane in range(64):
                row, col = 4 * (lane >> 4) + e, 16 * t + (lane & 15)
                banks.add(((row * rowb + col * 4) // 4) % 64)
                seen[row][col] += 1
            assert len(banks) == 64
    assert all(v == 1 for r in seen for v in r)


@pytest.mark.parametrize("ns,lpt,nquad", [(3, 12, 36), (3, 8, 16), (2, 8, 16)])
@pytest.mark.parametrize("nk", [1, 2, 3, 5, 6, 7, 8, 9, 12, 13, 64])
@pytest.mark.parametrize("addend", [False, True])
def test_vmcnt_waits_of_the_k_loop(ns, lpt, nquad, nk, addend):
    """The K loop of the fast kernel tracks its direct-to-LDS loads with s_waitcnt vmcnt(N): vector memory loads come
    back in the order they were issued, so "at most N outstanding" means "everything but the N youngest has landed".
    This replays, per wavefront, the order in which the kernel issues the loads of its K tiles (cut into parts) and the
    register loads of the first addend of a lower-triangle product (nquad loads, issued between the prologue and
    tile 0), and every wait with its count, and asserts that at the wait that ends tile kt all loads of tile kt + 1
    have landed -- and that the wait of tile 0 does not sit out the addend (the reason for its larger count), while
    the addend has landed at the wait of tile 1."""
    nq = 2                                             # k-steps per tile (BK / 32)
    parts = nq if ns >= 3 and lpt % nq == 0 else 1
    pl = lpt // parts
    issued = []                                        # tags in issue order
    landed = 0                                         # loads [0, landed) have come back

    def issue(tag, count):
        issued.extend([tag] * count)

    def wait(n):
        nonlocal landed
        landed = max(landed, len(issued) - n)

    def tile_landed(t):
        return all(i < landed for i, tag in enumerate(issued) if tag == t)

    for t in range(ns - 1):
        if t < nk:
            issue(t, lpt)
    if ns - 1 < nk:
        issue(ns - 1, pl)
    wait((ns - 2) * lpt + pl if nk >= ns else 0)
    assert tile_landed(0)
    if addend:
        issue("addend", nquad)
    kt = 0
    while kt + 2 * ns - 1 < nk:                        # steady rounds
        for u in range(ns):
            t = kt + u
            for q in range(nq - 1):
                if parts > 1:
                    issue(t - 1 + ns, pl)              # part q + 1 of tile t - 1 + NS
            extra = nquad if (addend and t == 0) else 0
            assert (ns - 2) * lpt + extra < 64         # 6-bit counter
            wait((ns - 2) * lpt + extra)
            assert tile_landed(t + 1)
            if addend and t == 0:
                assert not all(i < landed for i, tag in enumerate(issued) if tag == "addend")
            if addend and t == 1:
                assert tile_landed("addend")
            issue(t + ns, pl)                          # part 0 of tile t + NS into the slot just vacated
        kt += ns
    while kt < nk:                                     # the rounds that are not all steady
        for u in range(ns):
            t = kt + u
            if t >= nk:
                break
            if parts > 1 and t + ns - 1 < nk:
                issue(t - 1 + ns, (parts - 1) * pl)
            wait(0)
            assert t + 1 >= nk or tile_landed(t + 1)
            if t + ns < nk:
                issue(t + ns, pl)
        kt += ns
    assert landed == len(issued)
    assert all(issued.count(t) == lpt for t in range(nk))  # every tile loaded once, completely
