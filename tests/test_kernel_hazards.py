"""The 16x16x128 GEMM kernel issues its MFMAs as hand-written instructions, which the compiler takes for ordinary
ones: it neither knows that their results arrive passes later nor inserts the wait states an accumulator read
needs.  The kernel keeps that distance by construction (hand-placed v_accvgpr_read_b32 between later MFMAs, wait
states before the last reads).  This test compiles the kernel's translation units to assembly (no GPU needed) and
checks the distance on what the compiler actually emitted, for every instantiation.
"""
import os
import re
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from float8_experimental_amd import _build

UNITS = ["f8mi_gemm_dma16.hip", "f8mi_gemm_dma16_nt.hip", "f8mi_gemm_dma16_tt.hip"]
MIN_MFMAS = 8        # MFMAs issued after the producing one (each occupies the matrix core for 8 passes of 4 cycles) ...
MIN_WAIT_STATES = 18  # ... or this many wait states of s_nop between the two


def _asm(unit, out_dir):
    out = os.path.join(out_dir, unit[:-4] + ".s")
    subprocess.run([_build.HIPCC, *_build.FLAGS, "--cuda-device-only", "-S", os.path.join(_build.CSRC, unit), "-o", out],
                   check=True, stderr=subprocess.DEVNULL)
    with open(out) as f:
        return f.read().split("\n")


@pytest.fixture(scope="module")
def listings(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("asm"))
    with ThreadPoolExecutor(max_workers=3) as ex:
        return dict(zip(UNITS, ex.map(lambda u: _asm(u, d), UNITS)))


@pytest.mark.parametrize("unit", UNITS)
def test_accumulator_reads_keep_their_distance_from_the_mfma_that_writes_them(listings, unit):
    lines = listings[unit]
    ends = [i for i, l in enumerate(lines) if re.match(r"\.Lfunc_end\d+:", l)]  # one per kernel (a kernel may hold several s_endpgm)
    assert len(ends) >= 12, "expected one kernel per operand format pair, output type and parity of the step count"
    start = 0
    for end in ends:
        written = {}  # accumulator register -> (MFMAs issued so far, line)
        n_mfma = n_reads = 0
        for i in range(start, end):
            line = lines[i]
            m = re.search(r"v_mfma_\S+ a\[(\d+):(\d+)\]", line)
            if m:
                n_mfma += 1
                for r in range(int(m.group(1)), int(m.group(2)) + 1):
                    written[r] = (n_mfma, i)
                continue
            assert "v_accvgpr_write" not in line, f"{unit}:{i + 1}: accumulators are only ever written by MFMAs"
            m = re.search(r"v_accvgpr_read_b32 v\d+, a(\d+)", line)
            if m:
                n_reads += 1
                at_mfma, at_line = written[int(m.group(1))]
                nops = sum(int(n) + 1 for n in re.findall(r"s_nop (\d+)", "\n".join(lines[at_line + 1:i])))
                assert n_mfma - at_mfma >= MIN_MFMAS or nops >= MIN_WAIT_STATES, (
                    f"{unit}:{i + 1}: {line.strip()} only {n_mfma - at_mfma} MFMAs and {nops} wait states after its MFMA")
        assert n_mfma > 0 and n_reads == 256, (unit, n_mfma, n_reads)  # 64 accumulator tiles of 4 registers, each read once
        start = end + 1


@pytest.mark.parametrize("unit", UNITS)
def test_every_lds_dma_sets_m0_itself_with_the_wait_state_it_needs(listings, unit):
    """A global load into the LDS takes its LDS address from M0.  The scalar write of M0 needs one wait state before
    the vector memory instruction that reads it, and nothing may change M0 in between: every such load must come
    straight after `s_mov_b32 m0, ...` and `s_nop`, as the kernel's hand-written sequence has it."""
    lines = [l.strip() for l in listings[unit]]
    code = [l for l in lines if l and not l.startswith((";", ".", "//")) and not l.endswith(":")]
    n = 0
    for i, l in enumerate(code):
        if l.startswith("global_load_lds_"):
            n += 1
            assert code[i - 1].startswith("s_nop"), f"{unit}: `{l}` follows `{code[i - 1]}`"
            assert code[i - 2].startswith("s_mov_b32 m0,"), f"{unit}: `{l}`: M0 written by `{code[i - 2]}`"
    assert n >= 12 * 16 * 3  # every instantiation has the prologue's 32 and at least two steps with 16


@pytest.mark.parametrize("unit", UNITS)
def test_no_spills_and_accumulators_stay_in_place(listings, unit):
    """The kernel's register budget is exact (256 accumulator registers + the fragments of two steps): a build that
    spills or moves accumulators through vector registers is a build that lost its schedule."""
    text = "\n".join(listings[unit])
    assert "scratch_store" not in text and "scratch_load" not in text
    assert "v_accvgpr_mov" not in text
    sizes = [int(x) for x in re.findall(r"; ScratchSize: (\d+)", text)]
    assert sizes and not any(sizes)
