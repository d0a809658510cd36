"""CPU model of the kernel template's LDS layouts: the formulas of csrc/gemm_f32_mfma.hip restated
in Python and checked for what the kernel relies on -- every element of a tile is deposited once
and read from where it was deposited, and the lanes that the LDS serves in one cycle touch every bank
at most once (the cycle order of gfx950 was measured, see ``lds_cycles``)."""

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


@pytest.mark.parametrize("bk,pad,mi", [(8, 4, 32), (16, 4, 32), (24, 4, 32), (32, 4, 32), (40, 4, 32), (64, 4, 32), (16, 8, 16), (32, 8, 16),
                                       (48, 8, 16), (64, 8, 16)])
def test_padded_rows_of_the_staged_path_are_free_of_bank_conflicts(bk, pad, mi):
    # 32x32x2: the host pads every row by one 16-byte unit, (BK + PAD)/4 odd, and consecutive rows start in
    # different 16-byte bank groups.  16x16x4: the LDS pairs quarter-waves of two lane groups in one cycle, and
    # their reads are one 16-byte unit apart; rows padded by two units, (BK + PAD)/4 = 2 mod 4, keep them clear
    # (one unit does not: the last assert).  Checked against the measured cycle order, ``lds_cycles`` below.
    from mlir_roller_amd.roller import lds_row_pad
    assert lds_row_pad(bk, mi) == pad
    row_floats = bk + pad
    assert (row_floats // 4) % 4 == 2 if mi == 16 else (row_floats // 4) % 2 == 1
    for kk in range(0, bk, 4 * (64 // mi)):
        addr = [(lane % mi) * row_floats + 4 * (lane // mi) + kk for lane in range(64)]
        assert extra_cycles(addr, 4) == 0, (bk, pad, mi, kk)
    if mi == 16:
        assert extra_cycles([(lane % mi) * (bk + 4) + 4 * (lane // mi) for lane in range(64)], 4) > 0


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
    assert "f.b2[t] = *(const v2f*)&row[4 * NSEG4 * MI + 2 * lr];" in TEMPLATE
    assert "f.b1[t] = Bs[b_frag_lone + (kk + t) * LDB_S];" in TEMPLATE
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



# ---- B[K, N] tile: where its columns sit in LDS, and the banks the fragment reads touch --------------------
#
# How the LDS of gfx950 serves a wave's read was measured with single-wave probes under rocprofv3
# (SQ_LDS_BANK_CONFLICT per instruction, two groups of lanes switched on at a time):
#   32-bit   32 lanes a cycle (0-31, 32-63), 32 banks of 4 bytes
#   64-bit   32 lanes a cycle (0-31, 32-63), 64 banks
#   128-bit  16 lanes a cycle, 64 banks; the cycles of lanes 0-31 are the quarter-waves (4 lanes) {0, 3, 5, 6}
#            and {1, 2, 4, 7} (even and odd number of set bits), likewise for lanes 32-63
#   2 x 64-bit from one address register (ds_read2_b64, what two 64-bit reads of adjacent rows become)
#            16 consecutive lanes a cycle, 64 banks, one row per cycle

def lds_cycles(width):
    """Lanes that the LDS serves together, per read width in floats (4 = ds_read_b128, 2 = ds_read2_b64 as the
    kernel's 64-bit segment reads are emitted, 1 = ds_read_b32 / ds_read2_b32) and the number of banks."""
    if width == 4:
        quarters = lambda half, odd: [q for q in range(8) if bin(q).count("1") % 2 == odd]
        return [[32 * half + 4 * q + j for q in quarters(half, odd) for j in range(4)] for half in (0, 1) for odd in (0, 1)], 64
    if width == 2:
        return [list(range(16 * g, 16 * g + 16)) for g in range(4)], 64
    return [list(range(0, 32)), list(range(32, 64))], 32


def extra_cycles(addresses, width):
    """Bank-conflict cycles of one read: ``addresses[lane]`` is the lane's first float."""
    cycles, banks = lds_cycles(width)
    extra = 0
    for lanes in cycles:
        hit = {}
        for lane in lanes:
            for e in range(width):
                hit.setdefault((addresses[lane] + e) % banks, set()).add(addresses[lane] + e)
        extra += max(len(v) for v in hit.values()) - 1
    return extra


def test_the_lds_model_reproduces_the_probe():
    mi = 16
    grp = lambda f: [f(lane % mi, lane // mi) for lane in range(64)]
    assert extra_cycles(list(range(64)), 1) == 0
    assert extra_cycles(grp(lambda lr, lg: 640 * lg + lr), 1) == 2                      # lane groups on the same 16 banks
    assert extra_cycles(grp(lambda lr, lg: 640 * lg + 32 * (lg & 1) + lr), 1) == 2      # 32 floats apart: the same banks
    assert extra_cycles(grp(lambda lr, lg: 640 * lg + 16 * (lg & 1) + lr), 1) == 0
    assert extra_cycles(grp(lambda lr, lg: 640 * lg + 16 * (lg >> 1) + lr), 1) == 2
    assert extra_cycles([2 * lane for lane in range(64)], 1) == 2
    assert extra_cycles([4 * lane for lane in range(64)], 4) == 0
    assert extra_cycles(grp(lambda lr, lg: 640 * lg + 4 * lr), 4) == 0                  # every lane group on the same 64 banks
    assert extra_cycles(grp(lambda lr, lg: 640 * lg + 32 * (lg & 1) + 4 * lr), 4) == 4  # windows of odd groups moved by 32 banks
    assert extra_cycles(grp(lambda lr, lg: 640 * lg + 16 * (lg & 1) + 4 * lr), 4) == 4
    assert extra_cycles(grp(lambda lr, lg: 32 * lr + 4 * lg), 4) == 12                  # A rows of 32 floats, not swizzled
    assert extra_cycles(grp(lambda lr, lg: 32 * lr + 4 * (lg ^ ((lr // 2) % 8))), 4) == 0
    assert extra_cycles([8 * lane for lane in range(64)], 4) == 4 and extra_cycles([16 * lane for lane in range(64)], 4) == 12


@pytest.mark.parametrize("bk,mi", [(8, 32), (16, 32), (32, 32), (64, 32), (128, 32), (16, 16), (32, 16), (64, 16), (128, 16)])
def test_swizzled_a_reads_under_the_measured_cycle_order(bk, mi):
    """The A-side swizzle again, with the quarter-wave pairing that the hardware actually uses."""
    cpr, rpl, swz_n = swizzle_params(bk)
    kg = 64 // mi
    # rows of 16 floats with the 16-wide instruction: four rows fill the 64 banks, and the quarter-waves that the
    # LDS pairs up end on the same chunk -- the one combination with a conflict; the policy never picks a K step
    # below 32
    expected = 4 if (bk, mi) == (16, 16) else 0
    for r in range(bk // (4 * kg)):
        addr = [(lane % mi) * bk + 4 * ((r * kg + lane // mi) ^ (((lane % mi) // rpl) % swz_n)) for lane in range(64)]
        assert extra_cycles(addr, 4) == expected, (bk, mi, r)


def lone_swap(mi, tn, waves_n, trans_b=False):
    return (not trans_b) and mi == 16 and tn % 2 == 1 and waves_n % 2 == 0


def b_tile_col(krow, col, wn, mi, tn, waves_n):
    """b_tile_col of the template: the tile column found at float column ``col`` of LDS row ``krow``."""
    if lone_swap(mi, tn, waves_n) and (krow >> 2) & 1 and col % wn >= (tn - 1) * mi:
        return ((col // wn) ^ 1) * wn + col % wn
    return col


def test_lone_swap_is_the_templates():
    assert "#define LONE_SWAP (!TRANS_B && MI == 16 && (TN % 2) == 1 && (NWN % 2) == 0)" in TEMPLATE
    assert "if (((krow >> 2) & 1) && col % WN >= (TN - 1) * MI) return ((col / WN) ^ 1) * WN + col % WN;" in TEMPLATE
    assert "c = b_tile_col(krow, slot * 4) / 4;" in TEMPLATE and "b_soff[i] = krow * LDB_S + slot * 4;" in TEMPLATE
    assert ("const int b_frag_lone = (4 * lg) * LDB_S + ((LONE_SWAP && (lg & 1)) ? (((wave % NWN) ^ 1) * WN) : wn0) + (TN - 1) * MI + lr;"
            in TEMPLATE)


def b_read_addresses(bn, wn, mi, wave_n, t, kk=0):
    """Per segment of wave ``wave_n``: (width, [first float of every lane's read]) for MFMA ``t`` of a round."""
    tn, waves_n = wn // mi, bn // wn
    out = []
    for b0, w in segments(tn):
        addr = []
        for lane in range(64):
            lr, lg = lane % mi, lane // mi
            row = kk + 4 * lg + t
            if w == 1:
                base = ((wave_n ^ 1) * wn) if (lone_swap(mi, tn, waves_n) and lg & 1) else wave_n * wn
                addr.append(row * bn + base + (tn - 1) * mi + lr)
            else:
                addr.append(row * bn + wave_n * wn + b0 * mi + w * lr)
        out.append((b0, w, addr))
    return out


@pytest.mark.parametrize("wn,mi", WAVE_WIDTHS)
@pytest.mark.parametrize("waves_n", [1, 2, 4])
def test_b_reads_find_the_columns_the_loader_deposited(wn, mi, waves_n):
    bn, tn, bk = wn * waves_n, wn // mi, 32
    holds = {}                                                       # (LDS row, float column) -> tile column
    for krow, col in itertools.product(range(bk), range(bn)):
        holds[(krow, col)] = b_tile_col(krow, col - col % 4, wn, mi, tn, waves_n) + col % 4
    for krow in range(bk):
        assert sorted(holds[(krow, c)] for c in range(bn)) == list(range(bn))   # a permutation of the row
    for wave_n, t, kk in itertools.product(range(waves_n), range(4), range(0, bk, 4 * (64 // mi))):
        for b0, w, addr in b_read_addresses(bn, wn, mi, wave_n, t, kk):
            for lane in range(64):
                lr, lg = lane % mi, lane // mi
                krow, col = divmod(addr[lane], bn)
                assert krow == kk + 4 * lg + t                        # the k that element t of the A read carries
                for e in range(w):                                    # the columns the epilogue stores block b0+e to
                    assert holds[(krow, col + e)] == wave_n * wn + b0 * mi + w * lr + e


@pytest.mark.parametrize("wn,mi", WAVE_WIDTHS)
@pytest.mark.parametrize("waves_n", [2, 4])
def test_b_fragment_reads_are_free_of_bank_conflicts(wn, mi, waves_n):
    bn = wn * waves_n
    for wave_n, t in itertools.product(range(waves_n), range(4)):
        for b0, w, addr in b_read_addresses(bn, wn, mi, wave_n, t):
            assert extra_cycles(addr, w) == 0, (bn, wn, mi, wave_n, t, b0, w)


def test_a_lone_column_block_without_a_partner_wave_keeps_its_conflict():
    """One wave along N (or an odd number) leaves the lone block of a 16-wide instruction nowhere to swap to;
    the model must show the two cycles that costs, or it proves nothing about the cases above."""
    for b0, w, addr in b_read_addresses(80, 80, 16, 0, 0):
        assert extra_cycles(addr, w) == (2 if w == 1 else 0)
    # ... and what the template did before the swap, on the 96x160 tile of the ragged benchmark shape
    unswapped = [(4 * (lane // 16)) * 160 + 64 + lane % 16 for lane in range(64)]
    assert extra_cycles(unswapped, 1) == 2
