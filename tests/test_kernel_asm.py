"""Static check of the compiled gfx950 kernels: no accumulator-register traffic next to the MFMA instructions.

The fast kernels issue their MFMAs as inline assembly with the accumulators tied in place (AGPRs), so the compiler
neither sees an MFMA nor inserts the wait states an MFMA result needs before a VALU or memory instruction may read
it.  That is safe only while the register allocator keeps every accumulator where it is for the whole K loop and
the first read of an accumulator follows the drain (three ``s_nop 7``) after the loop.  A change elsewhere in a
kernel (register pressure in the epilogue, for instance) can make the allocator swap or spill accumulator registers
inside the loop; the result is then wrong in a few elements only.  This test compiles every translation unit of the library to assembly and
rejects, for every fast kernel,
  * any ``v_accvgpr_*`` move or AGPR spill inside an innermost loop that contains MFMAs,
  * any such instruction between an MFMA and the drain that follows it.
A second check counts loads.  The lower-triangle kernels of 128- and 192-row tiles request their first addend with
ordinary loads between the prologue and the K loop, and the wait at the end of K tile 0 leaves exactly that many more
loads in flight; were the compiler to merge, drop or move some of them, that wait would let a load of K tile 1 slip.
The test reads the number of those loads and the wait's immediate off the compiled code of every such kernel.
No GPU is involved.
"""
import os
import re
import shutil
import subprocess

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "emerging-optimizers_amd", "csrc")

ACC_TRAFFIC = re.compile(r"^\s*(v_accvgpr_\w+|scratch_(store|load)\w*\s+(off,\s*)?a\[|scratch_load\w*\s+a\[)")


def instructions(lines):
    """(index, text) of the lines that are instructions or labels (comments, directives and asm markers dropped)."""
    out = []
    for i, raw in enumerate(lines):
        t = raw.split(";")[0].strip()
        if not t or t.startswith(".") and not t.endswith(":") or t.startswith(";;"):
            continue
        out.append((i, t))
    return out


def agprs_of(text):
    """AGPR numbers an instruction names (a12, a[8:11])."""
    out = set()
    for m in re.finditer(r"\ba\[(\d+):(\d+)\]|\ba(\d+)\b", text):
        if m.group(3) is not None:
            out.add(int(m.group(3)))
        else:
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    return out


def accumulator_hazards(lines):
    ins = instructions(lines)
    text = [t for _, t in ins]
    # the accumulators are the AGPRs some MFMA writes; the compiler also parks ordinary values in free AGPRs, and
    # moving those around next to an MFMA is harmless
    accumulators = set()
    for t in text:
        if t.startswith("v_mfma"):
            accumulators |= agprs_of(t.split(",")[0])
    touches = lambda x: ACC_TRAFFIC.match(x) and (agprs_of(x) & accumulators)
    label_at = {t[:-1]: k for k, t in enumerate(text) if t.endswith(":")}
    bad = []
    # innermost loops (a branch back to an earlier label with no other loop inside)
    loops = []
    for k, t in enumerate(text):
        m = re.match(r"s_cbranch_\w+\s+(\S+)|s_branch\s+(\S+)", t)
        if m:
            target = label_at.get(m.group(1) or m.group(2))
            if target is not None and target <= k:
                loops.append((target, k))
    for lo, hi in loops:
        if any((a, b) != (lo, hi) and lo <= a and b <= hi for a, b in loops):
            continue
        body = text[lo:hi]
        if any(x.startswith("v_mfma") for x in body):
            bad += [f"in MFMA loop: {x}" for x in body if touches(x)]
    # between an MFMA and the drain (or the next MFMA)
    for k, t in enumerate(text):
        if not t.startswith("v_mfma"):
            continue
        for x in text[k + 1:k + 13]:
            # (what follows an unconditional branch in the text does not follow it at run time)
            if x.startswith("v_mfma") or x.startswith("s_nop 7") or x.startswith("s_branch") or x.startswith("s_endpgm"):
                break
            if touches(x):
                bad.append(f"after MFMA, before the drain: {x}")
    return bad


def test_detector_flags_swaps_and_spills():
    swap = """
.LBB0_1:
	v_accvgpr_read_b32 v66, a220
	v_accvgpr_mov_b32 a220, a0
	;;#ASMSTART
	v_mfma_f32_16x16x32_bf16 a[0:3], v[14:17], v[46:49], a[0:3]
	;;#ASMEND
	;;#ASMSTART
	v_mfma_f32_16x16x32_bf16 a[220:223], v[14:17], v[50:53], a[220:223]
	;;#ASMEND
	s_cbranch_scc1 .LBB0_1
""".splitlines()
    assert len(accumulator_hazards(swap)) == 2
    spill = """
	v_mfma_f32_16x16x32_bf16 a[232:235], v[14:17], v[46:49], a[232:235]
	scratch_store_dwordx4 off, a[232:235], off offset:100 ; 16-byte Folded Spill
	s_nop 7
	v_accvgpr_read_b32 v1, a0
""".splitlines()
    assert accumulator_hazards(spill) == ["after MFMA, before the drain: scratch_store_dwordx4 off, a[232:235], off offset:100"]
    other_path = """
	v_mfma_f32_16x16x32_bf16 a[48:51], v[14:17], v[46:49], a[48:51]
	s_cbranch_scc1 .LBB0_9
	s_branch .LBB0_1
.LBB0_8:
	v_accvgpr_write_b32 a48, 0
""".splitlines()
    assert accumulator_hazards(other_path) == []  # the block after the unconditional branch is entered from elsewhere
    clean = """
.LBB0_1:
	v_mfma_f32_16x16x32_bf16 a[0:3], v[14:17], v[46:49], a[0:3]
	ds_read_b64_tr_b16 v[118:119], v66
	s_cbranch_scc1 .LBB0_1
	v_accvgpr_read_b32 v191, a151
	s_nop 7
	v_accvgpr_read_b32 v1, a0
""".splitlines()
    assert accumulator_hazards(clean) == []  # a151 is no accumulator here: a value the compiler parked in a free AGPR


@pytest.fixture(scope="module")
def compiled_kernels(tmp_path_factory):
    """name -> assembly lines of every kernel of the library, compiled with the Makefile's own flags."""
    if shutil.which("hipcc") is None:
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("asm")
    subprocess.run(["make", "-j8", "-C", CSRC, "asm", f"ASMDIR={out}"], check=True, capture_output=True, timeout=900)
    kernels, name = {}, None
    for asm in sorted(out.glob("*.s")):
        for line in asm.read_text().splitlines():
            m = re.match(r"^(_ZN2mi\S+):\s", line)
            if m:
                name = m.group(1)
                kernels[name] = []
            elif name:
                kernels[name].append(line)
                if line.startswith(".Lfunc_end"):  # (not the first s_endpgm: a kernel may return early)
                    name = None
    return kernels


def test_no_accumulator_traffic_next_to_mfma(compiled_kernels):
    fast = {n: ls for n, ls in compiled_kernels.items() if "gemm_fast_kernel" in n or "small_chain_kernel" in n}
    # (the finishing kernel of a split-tail launch, split-tail role 2, has an epilogue and no K loop)
    no_mfma = [n for n, ls in fast.items() if not any("v_mfma" in x for x in ls)]
    assert len(fast) >= 20 and all(n.endswith("ELi2ELb0EEEvNS_10GemmParamsE") for n in no_mfma) and len(no_mfma) <= 1, no_mfma
    report = {n: accumulator_hazards(ls) for n, ls in fast.items()}
    report = {n: b for n, b in report.items() if b}
    assert not report, "\n".join(f"{n}: {len(b)} hazards, e.g. {b[0]}" for n, b in report.items())


# gemm_fast_kernel<FastCfg<TILE_M, WGM, WGN, BK, NS, TILE_N>, P_KS, Q_KS, MODE, OUT_F32, EDGE, STREAMK, RMW>
FAST_NAME = re.compile(r"gemm_fast_kernelINS_7FastCfgILi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)EEE"
                       r"Lb([01])ELb([01])ELi(\d)ELb([01])ELb([01])ELi(\d)ELb([01])E")


def early_addend_loads(lines):
    """(8-byte global loads in front of the first MFMA, immediates of the vmcnt waits of the kernel)."""
    text = [t for _, t in instructions(lines)]
    first_mfma = next(k for k, t in enumerate(text) if t.startswith("v_mfma"))
    loads = sum(1 for t in text[:first_mfma] if re.match(r"global_load_dwordx2\s", t))
    wider = sum(1 for t in text[:first_mfma] if re.match(r"global_load_dwordx[34]\s", t))
    waits = {int(m.group(1)) for t in text for m in [re.match(r"s_waitcnt vmcnt\((\d+)\)", t)] if m}
    return loads, wider, waits


def test_first_addend_is_requested_with_the_counted_number_of_loads(compiled_kernels):
    """SyrkStage::NQUAD loads of 8 bytes per lane, none merged into wider ones, and the wait at the end of K tile 0 that
    leaves (NS - 2) * LOADS_PER_TILE + NQUAD loads in flight (k_tile's EXTRA in gemm_fast.hpp)."""
    seen = 0
    for name, lines in compiled_kernels.items():
        m = FAST_NAME.search(name)
        if not m:
            continue
        tile_m, wgm, wgn, bk, ns, tile_n, p_ks, q_ks, mode, out_f32, edge, streamk, rmw = map(int, m.groups())
        nquad = (tile_m // wgm // 16) * (tile_n // wgn // 16)
        # the variants that hold the first addend in registers across the K loop (SyrkStage::CIN_EARLY), K loop included
        if mode != 0 or out_f32 or wgm * wgn != 4 or 2 * nquad > 80 or streamk == 2:
            continue
        loads_per_tile = (tile_m + tile_n) * bk * 2 // 1024 // (wgm * wgn)
        loads, wider, waits = early_addend_loads(lines)
        assert (loads, wider) == (nquad, 0), (name, loads, wider, nquad)
        assert (ns - 2) * loads_per_tile + nquad in waits, (name, sorted(waits))
        seen += 1
    assert seen >= 6  # 128 x 128 (two ring depths) and 192 x 192 tiles, whole and edge variants, both operand layouts


def test_device_scope_stores_carry_their_wait_states(compiled_kernels):
    """The lower-triangle epilogue stores its result with an inline-assembly `global_store_dwordx4 ... sc1` (written
    through the L2).  The compiler does not know that this is a store of more than 8 bytes, after which the data
    registers must not be rewritten for two wait states, so the statement carries an `s_nop 1` of its own: every such
    store in the compiled kernels must be followed by it, and there must be some (the staged epilogue of every
    lower-triangle kernel has two store loops)."""
    found = 0
    for name, lines in compiled_kernels.items():
        text = [t for _, t in instructions(lines)]
        for k, t in enumerate(text):
            if t.startswith("global_store_dwordx4") and t.endswith("sc1"):
                found += 1
                assert text[k + 1] == "s_nop 1", (name, t, text[k + 1])
    assert found >= 20
