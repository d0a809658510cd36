"""CPU model of the kernel template's LDS layouts: the formulas of csrc/gemm_f32_mfma.hip restated
in Python and checked for what the kernel relies on -- every element of a tile is deposited once
and read from where it was deposited, and the 16 lanes that the LDS serves per cycle on a 128-bit
read fall into 16 different bank groups (64 banks of 4 bytes on gfx950)."""

import itertools
import re
from pathlib import Path

import pytest

TEMPLATE = (Path(__file__).resolve().parent.parent / "mlir-roller_amd" / "csrc" / "gemm_f32_mfma.hip").read_text()


def swizzle_params(bk):
    cpr = bk // 4                                   # 16-byte chunks per LDS row
    rpl = 1 if cpr >= 16 else 16 // cpr             # rows per 256 bytes
    swz_n = 16 if cpr >= 16 else cpr                # swizzle period
    return cpr, rpl, swz_n


def test_model_constants_are_the_templates():
    # the three macros this model restates, as written in the template
    assert re.search(r"#define CPR \(BK / 4\)", TEMPLATE)
    assert re.search(r"#define RPL \(CPR >= 16 \? 1 : 16 / CPR\)", TEMPLATE)
    assert re.search(r"#define SWZ_N \(CPR >= 16 \? 16 : CPR\)", TEMPLATE)
    assert "(u % CPR) ^ ((row / RPL) % SWZ_N)" in TEMPLATE                       # writer side
    assert "((r * (KSUPER / 4) + lg) ^ ((lr / RPL) % SWZ_N)) * 4" in TEMPLATE      # reader side
    assert "return w * WN + b0 * MI + sw * lane + (bj - b0);" in TEMPLATE          # Bt row -> column
    assert "#define NSEG4 (TN / 4)" in TEMPLATE and "#define HAS_SEG2 ((TN % 4) / 2)" in TEMPLATE and "#define HAS_SEG1 (TN % 2)" in TEMPLATE


def segments(tn):
    """(first block, width) of the B-read segments of a wave with ``tn`` column blocks: as many of
    four blocks as fit, then one of two and one of one (``seg_first`` / ``seg_width`` of the template)."""
    out = [(4 * s, 4) for s in range(tn // 4)]
    if (tn % 4) // 2:
        out.append((4 * (tn // 4), 2))
    if tn % 2:
        out.append((tn - 1, 1))
    return out


def test_segments_cover_the_column_blocks():
    assert segments(8) == [(0, 4), (4, 4)] and segments(5) == [(0, 4), (4, 1)] and segments(6) == [(0, 4), (4, 2)]
    assert segments(3) == [(0, 2), (2, 1)] and segments(7) == [(0, 4), (4, 2), (6, 1)] and segments(1) == [(0, 1)] and segments(2) == [(0, 2)]
    for tn in range(1, 33):
        blocks = [b0 + e for b0, w in segments(tn) for e in range(w)]
        assert blocks == list(range(tn))


@pytest.mark.parametrize("bk,mi,rows", [(8, 32, 128), (16, 32, 128), (32, 32, 256), (64, 32, 128), (128, 32, 64),
                                        (16, 16, 64), (32, 16, 128), (64, 16, 128), (256, 16, 32)])
def test_direct_tile_is_a_bijection_and_reads_find_their_data(bk, mi, rows):
    cpr, rpl, swz_n = swizzle_params(bk)
    kg = 64 // mi
    ksuper = 4 * kg
    # writer: LDS unit u holds global chunk (row, c)
    holds = {}
    for u in range(rows * cpr):
        row, c = u // cpr, (u % cpr) ^ ((u // cpr // rpl) % swz_n)
        assert 0 <= c < cpr
        holds[u] = (row, c)
    assert len(set(holds.values())) == rows * cpr                   # every chunk of the tile exactly once
    # reader: lane (lr, lg) of row block bi wants k = kk + 4*lg .. +3 of row bi*mi + lr in round kk/ksuper
    for bi, r, lr, lg in itertools.product(range(rows // mi), range(bk // ksuper), range(mi), range(kg)):
        row = bi * mi + lr
        slot = (r * (ksuper // 4) + lg) ^ ((lr // rpl) % swz_n)
        assert holds[row * cpr + slot] == (row, r * (ksuper // 4) + lg)


@pytest.mark.parametrize("bk,mi", [(8, 32), (16, 32), (32, 32), (64, 32), (128, 32), (16, 16), (32, 16), (64, 16), (128, 16)])
def test_swizzled_fragment_reads_are_free_of_bank_conflicts(bk, mi):
    cpr, rpl, swz_n = swizzle_params(bk)
    kg = 64 // mi
    ksuper = 4 * kg
    for r in range(bk // ksuper):
        for first in range(0, 64, 16):                              # the LDS serves 16 lanes of a b128 read per cycle
            groups = set()
            for lane in range(first, first + 16):
                lr, lg = lane % mi, lane // mi
                byte = (lr * cpr + ((r * (ksuper // 4) + lg) ^ ((lr // rpl) % swz_n))) * 16
                groups.add((byte // 16) % 16)                       # 64 banks * 4 B = 16 groups of 16 bytes
            assert len(groups) == 16, (bk, mi, r, first)


@pytest.mark.parametrize("bk,pad,mi", [(8, 4, 32), (16, 4, 32), (24, 4, 32), (32, 4, 32), (40, 4, 32), (64, 4, 32), (16, 4, 16), (32, 4, 16), (48, 4, 16)])
def test_padded_rows_of_the_staged_path_are_free_of_bank_conflicts(bk, pad, mi):
    # the K step is a multiple of 8, so the host pads every row by one 16-byte unit: (BK + PAD)/4 is odd and
    # consecutive rows start in different 16-byte bank groups (mod 16)
    row_floats = bk + pad
    assert (row_floats // 4) % 2 == 1
    for first in range(0, 64, 16):
        groups = {(((lane % mi) * row_floats + 4 * (lane // mi)) * 4 // 16) % 16 for lane in range(first, first + 16)}
        assert len(groups) == 16


WAVE_WIDTHS = [(32, 32), (64, 32), (128, 32), (256, 32), (16, 16), (32, 16), (64, 16), (128, 16),
               (96, 32), (160, 32), (48, 16), (80, 16), (96, 16), (112, 16), (160, 16)]      # 3, 5, 6, 7, 10 column blocks too


def epilogue_column(bj, lane, mi, tn):
    """Column (inside the wave tile) to which the epilogue stores block bj's accumulator of ``lane``."""
    b0, w = next(sg for sg in segments(tn) if sg[0] <= bj < sg[0] + sg[1])
    return b0 * mi + w * lane + (bj - b0)


@pytest.mark.parametrize("wn,mi,waves_n", [(wn, mi, 2) for wn, mi in WAVE_WIDTHS])
def test_transposed_operand_rows_are_a_permutation_that_matches_the_epilogue(wn, mi, waves_n):
    tn = wn // mi
    bn = wn * waves_n

    def col_of_row(row):                             # bt_col_of_row of the template
        w, q = divmod(row, wn)
        bj, lane = divmod(q, mi)
        b0 = (bj & ~3) if bj < 4 * (tn // 4) else (4 * (tn // 4) if (tn % 4) // 2 and bj < 4 * (tn // 4) + 2 else tn - 1)
        sw = 4 if bj < 4 * (tn // 4) else (2 if (tn % 4) // 2 and bj < 4 * (tn // 4) + 2 else 1)
        return w * wn + b0 * mi + sw * lane + (bj - b0)

    assert sorted(col_of_row(r) for r in range(bn)) == list(range(bn))
    # block bj of wave w reads LDS row w*wn + bj*mi + lane; the epilogue stores that accumulator to
    # the column its segment assigns
    for w, bj, lane in itertools.product(range(waves_n), range(tn), range(mi)):
        assert col_of_row(w * wn + bj * mi + lane) == w * wn + epilogue_column(bj, lane, mi, tn)


@pytest.mark.parametrize("wn,mi", WAVE_WIDTHS)
def test_column_interleave_covers_every_column_once_and_matches_the_epilogue(wn, mi):
    """B[K, N] operand: for a segment (b0, w) a lane reads w consecutive columns at wn0 + b0*MI + w*lane and
    element e of that read feeds block b0 + e; the epilogue stores that block's accumulator to the same column."""
    assert "f.b4[t][v] = *(const v4f*)&row[4 * v * MI + 4 * lr];" in TEMPLATE
    assert "f.b2[t] = *(const v2f*)&row[4 * NSEG4 * MI + 2 * lr];" in TEMPLATE and "f.b1[t] = row[(TN - 1) * MI + lr];" in TEMPLATE
    assert "const int col = wn0 + b0 * MI + sw * lr;" in TEMPLATE
    tn = wn // mi
    fed = {}                                        # (block, lane) -> column whose B values the block's MFMA receives
    for (b0, w), lane in itertools.product(segments(tn), range(mi)):
        for e in range(w):
            fed[(b0 + e, lane)] = b0 * mi + w * lane + e
    assert sorted(fed.values()) == list(range(wn))                  # the wave tile's columns, each exactly once
    for (bj, lane), col in fed.items():
        assert col == epilogue_column(bj, lane, mi, tn)             # where the epilogue writes that accumulator
    # a lane's w stores are adjacent and aligned to w, so they leave as one vector store
    for (b0, w), lane in itertools.product(segments(tn), range(mi)):
        cols = [fed[(b0 + e, lane)] for e in range(w)]
        assert cols == list(range(cols[0], cols[0] + w)) and cols[0] % w == 0


@pytest.mark.parametrize("mi", [32, 16])
def test_k_permutation_pairs_the_same_k_on_both_operands(mi):
    """MFMA t of a round contracts k = kk + 4*g + t for lane group g: A takes element t of the 128-bit read at
    k offset 4*g, B is read from row kk + 4*g + t; over the 4 MFMAs and 64/mi groups every k of the round once."""
    assert "const int b_frag = (4 * lg) * LDB_S + wn0;" in TEMPLATE and "const float* row = &Bs[b_frag + (kk + t) * LDB_S];" in TEMPLATE
    kg = 64 // mi
    ksuper = 4 * kg
    seen = []
    for t, g in itertools.product(range(4), range(kg)):
        a_k = 4 * g + t                  # element t of the A read that starts at k offset 4*g
        b_row = 4 * g + t                # b_frag's row offset 4*g plus (kk + t)
        assert a_k == b_row
        seen.append(a_k)
    assert sorted(seen) == list(range(ksuper))
