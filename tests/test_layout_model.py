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
    assert "w * WN + v * MI * VN + VN * (rem % MI) + rem / MI" in TEMPLATE         # Bt row -> column


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


@pytest.mark.parametrize("wn,mi,waves_n", [(32, 32, 4), (64, 32, 2), (128, 32, 2), (256, 32, 1), (16, 16, 4), (32, 16, 2), (64, 16, 2), (128, 16, 1)])
def test_transposed_operand_rows_are_a_permutation_that_matches_the_epilogue(wn, mi, waves_n):
    tn = wn // mi
    vn = 4 if tn >= 4 else tn
    bn = wn * waves_n

    def col_of_row(row):
        w, q = divmod(row, wn)
        v, rem = divmod(q, mi * vn)
        return w * wn + v * mi * vn + vn * (rem % mi) + rem // mi

    assert sorted(col_of_row(r) for r in range(bn)) == list(range(bn))
    # block bj of wave w reads LDS row w*wn + bj*mi + lane; the epilogue stores that accumulator to
    # column w*wn + (bj // vn)*mi*vn + vn*lane + bj % vn
    for w, bj, lane in itertools.product(range(waves_n), range(tn), range(mi)):
        assert col_of_row(w * wn + bj * mi + lane) == w * wn + (bj // vn) * mi * vn + vn * lane + bj % vn


@pytest.mark.parametrize("wn,mi", [(32, 32), (64, 32), (128, 32), (256, 32), (16, 16), (32, 16), (64, 16), (128, 16)])
def test_column_interleave_covers_every_column_once_and_matches_the_epilogue(wn, mi):
    """B[K, N] operand: a lane reads VN consecutive columns at wn0 + v*MI*VN + VN*lane and element e of that
    read feeds block v*VN + e; the epilogue stores block bj's accumulator to column (bj//VN)*MI*VN + VN*lane + bj%VN."""
    assert "wn0 + VN * lr;  // + (kk+t)*LDB_S + v*MI*VN" in TEMPLATE and "const int col = wn0 + v * MI * VN + VN * lr;" in TEMPLATE
    tn = wn // mi
    vn = 4 if tn >= 4 else tn
    nvb = tn // vn
    fed = {}                                        # (block, lane) -> column whose B values the block's MFMA receives
    for v, lane, e in itertools.product(range(nvb), range(mi), range(vn)):
        fed[(v * vn + e, lane)] = v * mi * vn + vn * lane + e
    assert sorted(fed.values()) == list(range(wn))                  # the wave tile's columns, each exactly once
    for (bj, lane), col in fed.items():
        assert col == (bj // vn) * mi * vn + vn * lane + bj % vn    # where the epilogue writes that accumulator
    # a lane's VN stores are adjacent, so they leave as one vector store
    for v, lane in itertools.product(range(nvb), range(mi)):
        cols = [fed[(v * vn + e, lane)] for e in range(vn)]
        assert cols == list(range(cols[0], cols[0] + vn)) and cols[0] % vn == 0


@pytest.mark.parametrize("mi", [32, 16])
def test_k_permutation_pairs_the_same_k_on_both_operands(mi):
    """MFMA t of a round contracts k = kk + 4*g + t for lane group g: A takes element t of the 128-bit read at
    k offset 4*g, B is read from row kk + 4*g + t; over the 4 MFMAs and 64/mi groups every k of the round once."""
    assert "const int b_frag = (4 * lg) * LDB_S + wn0 + VN * lr;" in TEMPLATE and "f.b[t][v] = *(const bvec_t*)&Bs[b_frag + (kk + t) * LDB_S" in TEMPLATE
    kg = 64 // mi
    ksuper = 4 * kg
    seen = []
    for t, g in itertools.product(range(4), range(kg)):
        a_k = 4 * g + t                  # element t of the A read that starts at k offset 4*g
        b_row = 4 * g + t                # b_frag's row offset 4*g plus (kk + t)
        assert a_k == b_row
        seen.append(a_k)
    assert sorted(seen) == list(range(ksuper))
