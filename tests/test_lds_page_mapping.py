"""The lane-to-LDS mapping of the prompt attention kernel's direct loads, simulated on the host.

``csrc/attention_mfma.hip: page_sources()`` tells each lane of each load instruction which 16-byte chunk of a
page of K it must fetch so that, with an instruction filling 1 KB of LDS in lane order, chunk ``c`` of key row
``k`` ends at ``k * K_STRIDE + (c ^ k_swizzle(k)) * 8``, where ``read_key_fragments`` looks for it.  The formula
holds only if an instruction's 64 chunks are whole key rows; the kernel's ``PF_DMA`` gate must refuse the head
sizes for which they are not.  This test repeats both formulas and counts misplaced chunks.
"""
import re
from pathlib import Path

import pytest

SRC = (Path(__file__).resolve().parent.parent / "palm-infra_amd" / "csrc" / "attention_mfma.hip").read_text()
WAVE, PF_WAVES, PAGE_TOKENS = 64, 4, 64


def k_swizzle(row):
    return (row & 3) | (((row >> 3) & 1) << 2)


def gate(hd):
    """PF_DMA as the source states it (the expression is read from the source, so a change there is seen here)."""
    m = re.search(r"constexpr bool PF_DMA = (.*?);", SRC)
    expr = m.group(1)
    chunks = hd // 8
    k_stride = (chunks + 7) // 8 * 8 * 8
    env = {"CHUNKS": chunks, "WAVE": WAVE, "PAGE_TOKENS": PAGE_TOKENS, "K_STRIDE": k_stride, "HD": hd}
    return bool(eval(expr.replace("&&", " and "), {}, env))


def misplaced(hd):
    chunks = hd // 8
    page_chunks = PAGE_TOKENS * hd // 8
    loads = (page_chunks + PF_WAVES * WAVE - 1) // (PF_WAVES * WAVE)
    k_rows = WAVE // chunks
    lds = {}
    for i in range(loads):
        for wave in range(PF_WAVES):
            inst = i * PF_WAVES + wave
            for lane in range(WAVE):
                k_row = inst * k_rows + lane // chunks
                src_chunk = (lane % chunks) ^ k_swizzle(k_row)
                lds[inst * 64 + lane] = (k_row, src_chunk)            # what lands at this 16-byte place of LDS
    wrong = 0
    for row in range(PAGE_TOKENS):
        for c in range(chunks):
            place = row * chunks + (c ^ k_swizzle(row))                # K_STRIDE == HD where the gate holds
            wrong += lds.get(place) != (row, c)
    return wrong


@pytest.mark.parametrize("hd", range(16, 257, 16))
def test_direct_loads_are_used_only_where_their_mapping_is_right(hd):
    if gate(hd):
        assert misplaced(hd) == 0
    if hd in (64, 128):
        assert gate(hd)                       # the sizes the fast path was made for keep it
    if hd == 192:
        assert not gate(hd) and misplaced(hd) > 0      # rows of 24 chunks straddle two instructions
