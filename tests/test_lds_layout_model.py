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
    for mi, bk, nw, ks, rows in itertools.product((32, 16), (64, 32), (8, 4), (False, True), (256, 128, 192))
    if not (ks and rows == 192) and rows * bk * 2 % (1024 * nw) == 0 and not (mi == 16 and bk == 32)
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
