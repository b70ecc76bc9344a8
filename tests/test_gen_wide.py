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


def in_running_order(lines, gap):
    """The instructions of a variant's first steps in the order they run.  With gap = 0 that is
    the text; otherwise a step that carries C's old values (text up to its branch into the loop)
    is followed by `gap` steps of the loop, entered at the branch's label."""
    if gap == 0:
        return lines[:max(i for i, l in enumerate(lines) if l == "2:")]
    label = {l[:-1]: i for i, l in enumerate(lines) if re.fullmatch(r"\d+:", l)}
    out, i = [], 0
    while not lines[i].startswith("s_mov_b32 s75, 0"):      # the last of those steps ends here
        l = lines[i]
        m = re.fullmatch(r"s_branch 1(\d)f", l)
        if m:                                                # run `gap` loop steps from position m
            ret = i + 1
            pos = int(m.group(1))
            for _ in range(gap):
                k = label[f"1{pos}"] + 1
                while not lines[k].startswith("s_sub_u32 s64, s64, 1"):
                    out.append(lines[k])
                    k += 1
                pos = (pos + 1) % 6
            i = ret
            continue
        out.append(l)
        i += 1
    return out


def blocks_and_moves(lines, gap=0):
    """-> (number of MFMAs, accumulator reads too close behind the block's MFMA, accumulator writes
    too close before it, reads, writes) over the steps of one variant that move accumulators."""
    mfmas, last_mfma, pending, early, late, reads, writes = 0, {}, {}, 0, 0, 0, 0
    for l in in_running_order(lines, gap):
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
@pytest.mark.parametrize("gap", [0, *G.SPACED_GAPS])
def test_old_values_join_the_accumulators_clear_of_the_blocks_mfmas(kind, gap):
    lines = G.gen(kind, True, None, gap)
    mfmas, early, late, reads, writes = blocks_and_moves(lines, gap)
    assert reads == writes == 256            # every accumulator register once
    assert early == 0 and late == 0
    if gap == 0:   # unrolled steps + the loop of six, 128 MFMAs a step
        assert mfmas == (G.C_STEPS + 2 + 6) * G.GAPS
    else:          # nine steps with `gap` loop steps behind each but the last
        assert mfmas == (G.C_STEPS + 1 + G.C_STEPS * gap) * G.GAPS


@pytest.mark.parametrize("kind", ["u8", "i8", "bf16"])
@pytest.mark.parametrize("gap", [0, *G.SPACED_GAPS])
def test_the_additions_temporaries_are_not_shared_by_two_additions_in_flight(kind, gap):
    """An addition is three instructions that may sit behind three different MFMAs; a temporary
    holds one accumulator's value from the read to the write back, and nothing else writes it."""
    holds = {}
    for l in G.gen(kind, True, None, gap):
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


@pytest.mark.parametrize("kind", ["u8", "i8", "bf16"])
@pytest.mark.parametrize("gap", G.SPACED_GAPS)
def test_spaced_steps_land_on_their_positions(kind, gap):
    """Step j of the nine runs as k step j (gap + 1): its LDS stage, B slot and the loop label it
    branches to follow from that, and the loop returns to every one of them."""
    lines = G.gen(kind, True, None, gap)
    branches = [l for l in lines if re.fullmatch(r"s_branch 1\df", l)]
    assert branches == [f"s_branch 1{(j * (gap + 1) + 1) % 6}f" for j in range(G.C_STEPS + 1)]
    for j in range(1, G.C_STEPS + 1):
        assert f"4{j}:" in lines and f"s_cbranch_scc1 4{j}b" in lines
    assert lines.index("20:") < lines.index("2:")
    assert G.spaced_min_steps(gap) == G.C_STEPS * (gap + 1) + 2


def test_min_steps_matches_the_unrolled_part():
    assert G.MIN_STEPS == G.C_STEPS + 4
