"""The generated assembly of the four-wave Matmul tile (morello_amd/csrc/gen_gemm_wide.py), checked
as text: what the assembler and the hardware do not check for hand-written code.

An accumulating Spec adds C's old values into the accumulators in the middle of the k loop
(semantics: morello/src/spec.rs:480-485, MatmulAccum; morello/src/codegen/cpu.rs:2114-2124).  The
hardware does not interlock an accumulator moved by a vector instruction against the matrix
instructions around it, so the distances are the generator's to keep."""
import os
import re
import sys

import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "morello_amd", "csrc"))
import gen_gemm_wide as G  # noqa: E402


def blocks_and_moves(lines):
    """-> (number of MFMAs, accumulator reads too close behind the block's MFMA, accumulator writes
    too close before it, reads, writes) over the k loop of one variant."""
    mfmas, last_mfma, pending, early, late, reads, writes = 0, {}, {}, 0, 0, 0, 0
    loop_end = max(i for i, l in enumerate(lines) if l == "2:")
    for l in lines[:loop_end]:
        m = re.match(r"v_mfma\S+ a\[(\d+):", l)
        if m:
            blk = int(m.group(1)) // 4
            if blk in pending and mfmas - pending.pop(blk) < 2:
                late += 1
            last_mfma[blk] = mfmas
            mfmas += 1
            continue
        m = re.match(r"v_accvgpr_read_b32 v\d+, a(\d+)", l)
        if m:
            reads += 1
            blk = int(m.group(1)) // 4
            if blk in last_mfma and mfmas - 1 - last_mfma[blk] < 4:
                early += 1
        m = re.match(r"v_accvgpr_write_b32 a(\d+)", l)
        if m:
            writes += 1
            pending[int(m.group(1)) // 4] = mfmas
    return mfmas, early, late, reads, writes


@pytest.mark.parametrize("kind", ["u8", "i8", "bf16"])
def test_old_values_join_the_accumulators_clear_of_the_blocks_mfmas(kind):
    lines = G.gen(kind, True)
    mfmas, early, late, reads, writes = blocks_and_moves(lines)
    assert reads == writes == 256            # every accumulator register once
    assert early == 0 and late == 0
    # unrolled steps + the loop of six, 128 MFMAs a step
    assert mfmas == (G.C_STEPS + 2 + 6) * G.GAPS


@pytest.mark.parametrize("kind", ["u8", "i8", "bf16"])
def test_the_additions_temporaries_are_not_shared_by_two_additions_in_flight(kind):
    """An addition is three instructions that may sit behind three different MFMAs; a temporary
    holds one accumulator's value from the read to the write back, and nothing else writes it."""
    holds = {}
    for l in G.gen(kind, True):
        m = re.match(r"v_accvgpr_read_b32 (v\d+), a(\d+)", l)
        if m and int(m.group(1)[1:]) in G.C_TMP:
            assert m.group(1) not in holds, l
            holds[m.group(1)] = m.group(2)
            continue
        m = re.match(r"v_accvgpr_write_b32 a(\d+), (v\d+)", l)
        if m and m.group(2) in holds:
            assert holds.pop(m.group(2)) == m.group(1), l
            continue
        m = re.match(r"v_add_(u32|f32) (v\d+), (v\d+), v\d+", l)
        if m and m.group(2) in holds:
            assert m.group(3) == m.group(2), l
            continue
        for t in holds:      # no other instruction writes a temporary that is in use
            assert not re.match(r"\S+ " + t + r"\b", l), l
    assert not holds


@pytest.mark.parametrize("kind", ["u8", "i8", "bf16"])
@pytest.mark.parametrize("accum", [False, True])
def test_every_step_issues_the_same_work(kind, accum):
    """Each of the steps moves one A tile and one B tile and reads 48 operands, wherever the
    placement put them."""
    lines = G.gen(kind, accum)
    loop_end = max(i for i, l in enumerate(lines) if l == "2:")
    first = lines.index("s_barrier")           # the prologue's
    body = lines[first + 1:loop_end]
    steps = (G.C_STEPS + 2 if accum else 2) + 6
    count = lambda pat: sum(1 for l in body if re.match(pat, l))
    assert count(r"v_mfma") == steps * G.GAPS
    assert count(r"global_load_lds_dwordx4") == steps * 8
    assert count(r"ds_write_b128") == steps * 8
    assert count(r"s_barrier") == steps
    # 16 A operands and 32 transposing reads of B a step; every step reads the next one's first 23
    # behind its barrier, as the prologue does for the first
    assert count(r"ds_read_b128") + count(r"ds_read_b64_tr") == steps * 48 + 23
    if accum:
        assert count(r"global_load_dword v") == 256


def test_min_steps_matches_the_unrolled_part():
    assert G.MIN_STEPS == G.C_STEPS + 4
