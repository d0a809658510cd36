// fp32 GEMM kernel template for gfx950 (MI355X, CDNA4):  C[M,N] = A[M,K] * B[K,N]
// (or, with TRANS_B, C[M,N] = A[M,K] * Bt[N,K]^T)
//
// Row-major operands, fp32 MFMA with fp32 accumulators.  The file is a template in the
// preprocessor sense: every rTile parameter arrives as a -D define from the JIT (hiprtc) or from
// an ahead-of-time hipcc line, and one translation unit yields exactly one kernel, "gemm_kernel"
// (the symbol name the reference loads, /root/reference/src/roller.py:499).
//
// It stands in for the kernel that the reference derives from its transform-dialect schedule
// (/root/reference/src/roller.py:93-342): one workgroup per BM x BN tile of C, a serial K loop of
// step BK (the policy's rstep), both operand tiles staged through workgroup memory with STAGES
// buffers (the reference's pipeline_depth), accumulators held in registers across the K loop and
// written once, and a workgroup-id remap for cache reuse (the reference swizzles in panels of 8,
// roller.py:334-339).  What differs is everything below that level: the per-thread outer product
// becomes a per-wave grid of MFMA blocks, and cp.async becomes buffer loads that write LDS directly
// (DIRECT) or a register-staged prefetch.
//
// Parameters (all compile-time):
//   BM, BN      block tile (rows, columns of C per workgroup)
//   BK          K step per main-loop iteration; multiple of 4*(64/MI)
//   WM, WN      wave tile; (BM/WM)*(BN/WN) waves of 64 lanes form the workgroup
//   MI          32 -> v_mfma_f32_32x32x2_f32, 16 -> v_mfma_f32_16x16x4_f32
//   STAGES      pipeline depth: 1 = one LDS buffer, nothing overlapped; 2 = two LDS buffers, the
//               global loads of step k+1 staged through registers during the MFMAs of step k and
//               written to LDS after them; 3 = two LDS buffers and the fully pipelined loop: the
//               loads of a tile are issued a whole K step ahead (DIRECT: straight into the other
//               LDS buffer; staged: into registers, two steps ahead of their use), the LDS
//               fragments of the next MFMA group are read while the current group executes, also
//               across the barrier that ends a K step; 4 and 5 (DIRECT only) = the same with
//               three and four LDS buffers, so that loads run two and three K steps ahead of the
//               MFMAs -- for short K steps whose MFMA time does not cover a trip to HBM
//   PAD_A,PAD_B extra floats per LDS row of the A tile ([BM][BK+PAD_A]) and B tile ([BK][BN+PAD_B]);
//               LDS holds the A tiles of all buffers first, then the B tiles, so that both tiles of
//               either buffer are within the 64 KB immediate offset of an LDS read
//   VEC         4 = 16-byte aligned 128-bit global accesses (needs K%4==0, N%4==0, lda/ldb/ldc%4==0
//               and 16-byte aligned base pointers), 1 = any K, N, leading dimension and 4-byte
//               aligned pointers: 128-bit loads at dword alignment with per-element zeroing of
//               what lies past a row's end, dword stores
//   EDGE        1 = predicate ragged tiles (any M, N, K), 2 = M and N may be ragged but the host
//               guarantees BK|K (no per-step K predicates), 0 = host guarantees BM|M, BN|N, BK|K
//   SWZ         workgroup-id remap: bit0 = give every XCD a contiguous run of tiles,
//               bit1 = walk the tile grid in panels of GROUP tile rows
//   GROUP, NXCD panel height in tiles; number of XCDs the dispatcher round-robins over
//   ACCUM       1 = C += A*B (what linalg.matmul means, roller.py:62), 0 = C = A*B
//   DIRECT      1 = global loads write LDS directly (buffer_load_dwordx4 ... lds), no staging
//               registers and no LDS write instructions; needs STAGES>=3, PAD_A=PAD_B=0
//               and BK a power of two.  With VEC=1 (dword-aligned rows; STAGES=3 and EDGE=1
//               then) full K steps are loaded the same way, at dword alignment, and the step
//               that K ends in with buffer_load_dword ... lds, one float per lane and four
//               instructions per 16-byte unit: every float is then inside its matrix or not on
//               its own, where a 16-byte unit across the end of a row of A would bring the next
//               row's first floats with it.
//               A wave's load lands as 64 consecutive 16-byte units, so rows cannot be padded;
//               instead the 16-byte chunks of every A row are XOR-swizzled with the row number
//               (on the load side by choosing which global chunk a lane fetches, on the read
//               side in the fragment address), which keeps the 128-bit A reads conflict-free.
//   STREAMK     0 = one workgroup per tile of C.  n > 0 = a fixed grid of n workgroups per CU, each of
//               which works through an equal share of all (tile, K step) units, contiguous in K
//               (gemm_sk_decode.inc).  A tile whose K range is split over workgroups is summed through
//               a workspace: every piece is stored there, an arrival counter per tile tells the last
//               piece in, and that workgroup adds the pieces in K order and writes C -- the same
//               order whoever arrives last, so results are bit-identical from run to run.  Needs
//               STAGES == 3.
//   TRANS_B     1 = the second operand is given transposed, Bt[N][ldb >= K] (K contiguous, the
//               layout in which the policy models both inputs, /root/reference/src/analyze.py:33-41).
//               Its tile then sits in LDS like the A tile ([BN][BK+PAD_B], swizzled under DIRECT)
//               and a lane reads four consecutive k of one column with one ds_read_b128.  LDS row
//               r of the tile holds the column that block r/MI hands to lane r%MI (see below), so
//               consecutive lanes read consecutive rows and C leaves in the same vector stores.
//
// Layout trick that removes every LDS bank conflict and every register shuffle on the read side:
// an MFMA sums over its k slots, and a GEMM does not care which MFMA block owns which column, so
// both index sets may be permuted as long as A and B agree.
//   * A stays K-contiguous in LDS.  A lane reads four consecutive k of its row with one
//     ds_read_b128; the four values feed four consecutive MFMAs.  MFMA t therefore contracts over
//     k = kk + 4*g + t for lane group g (g = lane / MI), and the B operand of that MFMA is read
//     from row kk + 4*g + t.
//   * B stays N-contiguous in LDS.  A lane reads w consecutive columns with one ds_read and the
//     w values feed w different column blocks.  The TN column blocks of a wave are cut into
//     segments of w = 4 blocks, then one of 2 and one of 1 for what is left (TN = 8: 4+4; 5: 4+1;
//     6: 4+2; 3: 2+1); a segment that starts at block b0 covers the MI*w columns from
//     wn0 + b0*MI, and block b0+e owns the columns wn0 + b0*MI + w*(lane%MI) + e.  In the
//     epilogue the same w accumulators are adjacent in memory again and leave as one vector store.
// Rows of LDS-A are padded so that (BK+PAD_A)/4 is odd: the 16-byte reads of lanes in consecutive
// rows then fall into distinct bank groups.
//
// The K loop is written for the instruction issue of one wave per SIMD: an LDS read or a global
// load issues beside the MFMAs for free, an instruction of the vector ALU (an address add, a
// compare, a select) takes MFMA issue time, and the loop of the aligned 128-bit kernels has none.
//
// Summation order is fixed by (BK, MI) alone (with STREAMK: and by the split, a function of the
// problem size and the grid), never by timing, so results are bit-identical from run to run.

#ifndef __HIPCC_RTC__  // hiprtc pre-includes the device runtime declarations
#include <hip/hip_runtime.h>
#endif

#ifndef BM
#define BM 128
#endif
#ifndef BN
#define BN 128
#endif
#ifndef BK
#define BK 16
#endif
#ifndef WM
#define WM 64
#endif
#ifndef WN
#define WN 64
#endif
#ifndef MI
#define MI 32
#endif
#ifndef STAGES
#define STAGES 2
#endif
#ifndef PAD_A
#define PAD_A 4
#endif
#ifndef PAD_B
#define PAD_B 0
#endif
#ifndef VEC
#define VEC 4
#endif
#ifndef EDGE
#define EDGE 1
#endif
#ifndef SWZ
#define SWZ 3
#endif
#ifndef GROUP
#define GROUP 8
#endif
#ifndef NXCD
#define NXCD 8
#endif
#ifndef ACCUM
#define ACCUM 0
#endif
#ifndef SCHED
#define SCHED 1
#endif
#ifndef DIRECT
#define DIRECT 0
#endif
#ifndef TRANS_B
#define TRANS_B 0
#endif
#ifndef STREAMK
#define STREAMK 0
#endif

#define EDGE_K (EDGE == 1) /* the K extent may be ragged as well */
#define NWM (BM / WM)
#define NWN (BN / WN)
#define NWAVES (NWM * NWN)
#define NT (64 * NWAVES)
#define TM (WM / MI)
#define TN (WN / MI)
#define KG (64 / MI)       /* lane groups along k inside one MFMA (= its k extent) */
#define KSUPER (4 * KG)    /* k covered by the four MFMAs fed from one 128-bit A read */
/* segments of column blocks that one B read feeds: TN / 4 of four blocks (128-bit reads), then
 * one of two (64-bit) and one of one (32-bit) for the remainder */
#define NSEG4 (TN / 4)
#define HAS_SEG2 ((TN % 4) / 2)
#define HAS_SEG1 (TN % 2)
#define NSEG (NSEG4 + HAS_SEG2 + HAS_SEG1)
#define LDA_S (BK + PAD_A)
#if TRANS_B
#define LDB_S (BK + PAD_B)
#define B_STAGE (BN * LDB_S)
#else
#define LDB_S (BN + PAD_B)
#define B_STAGE (BK * LDB_S)
#endif
#define A_STAGE (BM * LDA_S)
#define STAGE_FLOATS (A_STAGE + B_STAGE)
#define LDS_BUFS (STAGES >= 3 ? STAGES - 1 : STAGES)
#define SUPERS (BK / KSUPER) /* MFMA groups per K step, each fed by one round of fragment reads */
#define A_UNITS (BM * BK / 4)
#define B_UNITS (BK * BN / 4)
#define A_PER_T ((A_UNITS + NT - 1) / NT)
#define B_PER_T ((B_UNITS + NT - 1) / NT)
#define OOB_OFFSET 0x80000000u
/* cache policy operand of a buffer access: sc0 (bit 0) and sc1 (bit 4) together = coherent across the whole system */
#define SK_COHERENT 0x11
// Cache policy of the stores of C: non-temporal (aux bit 1).  C is written once and never read by the
// kernel, so its lines should not displace operand panels from the L2 nor wait there, dirty, for the
// write-back at the end of the kernel (measured: 0.3 % on 2048^3, 1 % on 1024^3 and 1536^3, nothing
// on the largest shapes; write-through forms, sc1 / sc0 sc1, gave the same on small shapes and cost
// 0.3 % on 3000x5000x1536).
#define C_STORE_AUX 2
/* DIRECT: 16-byte chunks per A row; A rows per 256 bytes of LDS (the 64 banks that a 128-bit read
 * of 16 lanes must cover without collision); the swizzle period.  Rows that start at the same
 * offset within a 256-byte window get their chunks XOR-ed with distinct values, so the 16 lanes
 * of one read cycle, which sit in 16 consecutive rows at the same chunk, hit 16 distinct bank
 * groups. */
#define CPR (BK / 4)
#define RPL (CPR >= 16 ? 1 : 16 / CPR)
#define SWZ_N (CPR >= 16 ? 16 : CPR)
/* The LDS serves a 32-bit read 32 lanes a cycle (lanes 0-31, then 32-63) out of 32 banks.  With the
 * 16x16x4 instruction the two lane groups of a cycle read rows 4 apart, and a row is a multiple of 32
 * floats from the next one that matters, so the lone column block of a wave (TN odd: 16 consecutive
 * floats per lane group) would come from the same 16 banks for both groups.  On rows whose k group
 * (k / 4) is odd, the waves 2j and 2j+1 along N therefore swap their lone blocks' columns in LDS: the
 * two are WN = 16 * odd floats apart, i.e. 16 banks, so the groups of a cycle read disjoint banks.
 * The 128-bit reads keep their columns: the LDS pairs quarter-waves of different lane groups in one
 * cycle and needs all lane groups on the same bank alignment there.  Needs an even number of waves
 * along N; the loader fetches the global columns that belong in its LDS slot. */
#define LONE_SWAP (!TRANS_B && MI == 16 && (TN % 2) == 1 && (NWN % 2) == 0)

static_assert(MI == 32 || MI == 16, "MI selects v_mfma_f32_32x32x2_f32 or v_mfma_f32_16x16x4_f32");
static_assert(BM % WM == 0 && BN % WN == 0, "wave tile must divide block tile");
static_assert(WM % MI == 0 && WN % MI == 0, "MFMA block must divide wave tile");
static_assert(TM * TN <= 32, "at most 32 MFMA blocks per wave: beyond that the accumulator array is no longer kept in registers");
static_assert(BK % KSUPER == 0, "BK must be a multiple of 4*(64/MI)");
static_assert(PAD_A % 4 == 0 && PAD_B % 4 == 0, "LDS rows stay 16-byte aligned");
static_assert(TRANS_B == 0 || TRANS_B == 1, "TRANS_B is a flag");
static_assert(EDGE >= 0 && EDGE <= 2, "EDGE: 0 none, 1 all three extents, 2 M and N only");
static_assert(NT <= 1024, "at most 16 waves per workgroup");
static_assert(STAGES >= 1 && STAGES <= 5, "pipeline depth 1 to 5");
static_assert(STAGES <= 3 || DIRECT, "more than two LDS buffers only with direct-to-LDS loads");
static_assert(VEC == 4 || VEC == 1, "global access width");
static_assert(STREAMK >= 0 && (!STREAMK || STAGES == 3), "the stream-K variant is built on the pipelined loop with two LDS buffers");
static_assert(!DIRECT || (STAGES >= 3 && PAD_A == 0 && PAD_B == 0), "DIRECT needs STAGES>=3 and no padding");
/* Waiting for "all but the newest n tiles" counts this wave's outstanding loads, which is exact
 * only if every wave issues the same number of loads per tile. */
// With dword-aligned rows (VEC == 1) the direct-to-LDS loads of a full K step are the same 16-byte
// units per lane (the memory pipeline accepts dword alignment for them), but a unit that straddles
// the end of K would bring the next row's first floats with it: the steps that may hold the end of K
// load one float per lane instead, four instructions for every one, each float tested by itself.
#define DW_DIRECT (DIRECT && VEC == 1)
#define LOADS_PER_TILE (A_PER_T + B_PER_T)
#define A_DW_LOADS ((4 * A_UNITS + NT - 1) / NT)
#define B_DW_LOADS ((4 * B_UNITS + NT - 1) / NT)
#define EXACT_LOADS (A_UNITS % NT == 0 && B_UNITS % NT == 0)
static_assert(!DW_DIRECT || (LDS_BUFS == 2 && EDGE == 1), "direct-to-LDS loads of dword-aligned rows: two LDS buffers, all three extents tested");
static_assert(LDS_BUFS <= 2 || EXACT_LOADS, "three or more LDS buffers need operand tiles that divide evenly over the threads");
static_assert(LDS_BUFS <= 2 || (LDS_BUFS - 2) * LOADS_PER_TILE <= 63, "too many loads in flight for the 6-bit vmcnt");
/* the prologue may start on tile 0 while the other requested tiles are still in flight, if that
 * count can be waited for exactly; otherwise it waits for everything */
#define PROLOGUE_IN_FLIGHT ((EXACT_LOADS && (LDS_BUFS - 1) * LOADS_PER_TILE <= 63) ? (LDS_BUFS - 1) * LOADS_PER_TILE : 0)
/* s_waitcnt that waits until at most n vector-memory operations of this wave are outstanding
 * (vmcnt is split over bits 3:0 and 15:14; expcnt and lgkmcnt are left at "do not wait") */
#define WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0f70 | ((n) & 0xf) | ((((n) >> 4) & 0x3) << 14))
static_assert(!DIRECT || (A_UNITS % 64 == 0 && B_UNITS % 64 == 0), "DIRECT moves whole waves of 16-byte units");
static_assert(!DIRECT || (BK & (BK - 1)) == 0, "DIRECT swizzles A rows with XOR: BK must be a power of two");
static_assert(LDS_BUFS * STAGE_FLOATS * 4 <= 160 * 1024, "tile does not fit the 160 KB LDS of a CU");

typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

#if MI == 32
typedef v16f acc_t;
#define ACC_REGS 16
#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x2f32((a), (b), (c), 0, 0, 0)
// accumulator register r of lane group g holds row 8*(r/4) + 4*g + r%4 of the 32x32 block
#define ACC_ROW(r, g) (8 * ((r) / 4) + 4 * (g) + (r) % 4)
#else
typedef v4f acc_t;
#define ACC_REGS 4
#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32((a), (b), (c), 0, 0, 0)
// accumulator register r of lane group g holds row 4*g + r of the 16x16 block
#define ACC_ROW(r, g) (4 * (g) + (r))
#endif

#define DEV static __device__ __forceinline__

#if STREAMK
#ifndef SK_DECODE_INCLUDED   /* the JIT path of the library puts the text in front of this file */
#include "gemm_sk_decode.inc"
#endif
#endif

// first block and width of B-read segment s
DEV constexpr int seg_first(int s) { return s < NSEG4 ? 4 * s : (s == NSEG4 && HAS_SEG2 ? 4 * NSEG4 : TN - 1); }
DEV constexpr int seg_width(int s) { return s < NSEG4 ? 4 : (s == NSEG4 && HAS_SEG2 ? 2 : 1); }

template <int V>
struct int_c {
  static constexpr int value = V;
};

// Instruction-scheduler directive: in the enclosing scheduling region, order the next NM MFMAs
// and the next NO instructions of class MASK (0x100 LDS read, 0x200 LDS write, 0x020 global
// read) so that the others are spread over the MFMAs as evenly as possible, earliest first:
// each memory instruction is issued in the shadow of an MFMA instead of in a burst that leaves
// the matrix pipe idle.
template <int NM, int NO, int MASK>
DEV void interleave_with_mfma() {
  if constexpr (NM > 0) {
    constexpr int q = NO / NM, rem = NO % NM;
#pragma unroll
    for (int i = 0; i < NM; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (i < rem) {
        __builtin_amdgcn_sched_group_barrier(MASK, q + 1, 0);
      } else if (q > 0) {
        __builtin_amdgcn_sched_group_barrier(MASK, q > 0 ? q : 1, 0);
      }
    }
  } else if constexpr (NO > 0) {
    __builtin_amdgcn_sched_group_barrier(MASK, NO > 0 ? NO : 1, 0);
  }
}

// Raw buffer resource over [base, base+bytes): loads beyond it return 0, stores beyond it are
// dropped.  Word 3 = 0x00020000 is the 32-bit raw data format on gfx9-family targets.
DEV __amdgpu_buffer_rsrc_t make_rsrc(const void* base, long bytes) {
  int n = bytes <= 0 ? 0 : (bytes > 0x7fffffffL ? 0x7fffffff : (int)bytes);
  return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, n, 0x00020000);
}

// Resource of an operand tile for K step kt.  With 128-bit accesses every 16-byte unit is inside the
// matrix or outside it as a whole and the predicates of the loads decide (an excluded unit gets
// OOB_OFFSET, which is beyond any range), so the range only has to tell a live tile (everything
// passes) from one past the end of K (nothing passes): scalar selects, where the exact remainder
// costs 64-bit compares on the vector unit in every K step.  With dword-aligned rows (VEC == 1) a
// 128-bit load can straddle the end of the matrix, and the exact range is what zeroes its tail.
DEV __amdgpu_buffer_rsrc_t tile_rsrc(const void* base, bool live, long bytes) {
#if VEC == 4
  (void)bytes;
  return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, live ? 0x7fffffff : 0, 0x00020000);
#else
  // a live tile has a positive remainder; "above 2^31-1" as a test for set upper bits stays on
  // the scalar unit, where an ordered 64-bit compare would go to the vector unit
  unsigned hi = (unsigned)((unsigned long)bytes >> 32);
  const unsigned lo = (unsigned)bytes;
  asm("" : "+s"(hi));   // (keeps the halves apart: put back together, the test is a 64-bit compare)
  const int n = (hi | (lo >> 31)) != 0 ? 0x7fffffff : (int)lo;
  return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, live ? n : 0, 0x00020000);
#endif
}

template <bool SAME = false>
DEV v4f load_unit(__amdgpu_buffer_rsrc_t r, unsigned off, bool p0, bool p1, bool p2, bool p3) {
#if VEC == 4
  (void)p1; (void)p2; (void)p3;
  return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, p0 ? off : OOB_OFFSET, 0, 0));
#else
  // Rows that are not multiples of four floats long start at dword-aligned addresses only.  The
  // four elements still come with one 128-bit load (the memory pipeline accepts dword alignment
  // for multi-dword buffer loads); elements past the end of a row or column range would carry the
  // neighbouring row's data and are zeroed here.  The predicates are monotone (p0 >= p1 >= p2 >= p3);
  // SAME says that the caller passes four equal ones (the unit is in or out as a whole).
  v4f v = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, p0 ? off : OOB_OFFSET, 0, 0));
  if constexpr (!SAME) {
    v.y = p1 ? v.y : 0.0f;
    v.z = p2 ? v.z : 0.0f;
    v.w = p3 ? v.w : 0.0f;
  }
  return v;
#endif
}

#if TRANS_B
// Column of the block tile that LDS row `row` of the Bt tile holds.  Block bj = b0 + e of a wave,
// in a segment of width sw that starts at block b0, owns the columns b0*MI + sw*lane + e of its
// wave tile; row bj*MI + lane holds that column.
DEV int bt_col_of_row(int row) {
  const int w = row / WN, q = row % WN, bj = q / MI, lane = q % MI;
  const int b0 = bj < 4 * NSEG4 ? (bj & ~3) : (HAS_SEG2 && bj < 4 * NSEG4 + 2 ? 4 * NSEG4 : TN - 1);
  const int sw = bj < 4 * NSEG4 ? 4 : (HAS_SEG2 && bj < 4 * NSEG4 + 2 ? 2 : 1);
  return w * WN + b0 * MI + sw * lane + (bj - b0);
}
#endif

// Tile column that sits at float column `col` of LDS row `krow` of the B[K,N] tile (an involution).
DEV constexpr int b_tile_col(int krow, int col) {
#if LONE_SWAP
  if (((krow >> 2) & 1) && col % WN >= (TN - 1) * MI) return ((col / WN) ^ 1) * WN + col % WN;
#endif
  (void)krow;
  return col;
}

// The same with STRIDE MFMAs ahead of each of the NO other instructions (needs NO * STRIDE <= NM).
template <int NM, int NO, int MASK, int STRIDE>
DEV void stride_with_mfma() {
  static_assert(NO * STRIDE <= NM, "not enough MFMAs for this spacing");
#pragma unroll
  for (int i = 0; i < NO; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, STRIDE, 0);
    __builtin_amdgcn_sched_group_barrier(MASK, 1, 0);
  }
  if constexpr (NM - NO * STRIDE > 0) __builtin_amdgcn_sched_group_barrier(0x008, NM - NO * STRIDE, 0);
}

// Maps the hardware workgroup id to a tile of C.
DEV bool tile_of_workgroup(int nbm, int nbn, int& tile_m, int& tile_n) {
  int pid = blockIdx.y * gridDim.x + blockIdx.x;
  const int npid = nbm * nbn;
  if (pid >= npid) return false;  // launch wider than the tile grid
#if SWZ & 1
  // Workgroups are dealt to the XCDs round-robin; undo that so that XCD x works on one
  // contiguous run of the tile order and its L2 sees neighbouring tiles.
  {
    const int per = (npid + NXCD - 1) / NXCD;
    int tall = npid % NXCD;
    if (tall == 0) tall = NXCD;
    const int xcd = pid % NXCD, loc = pid / NXCD;
    pid = xcd < tall ? xcd * per + loc : tall * per + (xcd - tall) * (per - 1) + loc;
  }
#endif
#if SWZ & 2
  {
    const int width = GROUP * nbn;
    const int first_m = (pid / width) * GROUP;
    const int rows = nbm - first_m < GROUP ? nbm - first_m : GROUP;
    tile_m = first_m + (pid % width) % rows;
    tile_n = (pid % width) / rows;
  }
#else
  tile_m = pid / nbn;
  tile_n = pid % nbn;
#endif
  return true;
}

extern "C" __global__ __launch_bounds__(NT) void gemm_kernel(
    const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C,
    int M, int N, int K, int lda, int ldb, int ldc
#if STREAMK
    // workspace: one slot of BM*BN floats per piece of a split tile (two per workgroup); one arrival
    // counter per tile, zero before the launch and zero again when it ends; the split
    , float* __restrict__ sk_slots, unsigned* __restrict__ sk_arrivals, const sk_params sk
#endif
) {
  extern __shared__ __attribute__((aligned(16))) float lds[];

  const int tid = threadIdx.y * blockDim.x + threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / NWN) * WM;
  const int wn0 = (wave % NWN) * WN;
  const int lr = lane % MI;  // row of A / column slot of B inside an MFMA block
  const int lg = lane / MI;  // k group inside an MFMA

#if STREAMK
  // This workgroup's work, one segment (a run of K steps of one tile) at a time: first its share of
  // the (tile, K step) units of the tiles that are shared out, then its whole tiles, one per round of
  // the grid.  All of it is wave-uniform scalar arithmetic.
  unsigned wg = blockIdx.x;
  if (wg >= sk.grid) return;
#if SWZ & 1
  {
    // workgroups are dealt to the XCDs round-robin: give every XCD one contiguous stretch of the units
    // (and of the tiles of every round)
    const unsigned per = (sk.grid + NXCD - 1) / NXCD;
    unsigned tall = sk.grid % NXCD;
    if (tall == 0) tall = NXCD;
    const unsigned xcd = wg % NXCD, loc = wg / NXCD;
    wg = xcd < tall ? xcd * per + loc : tall * per + (xcd - tall) * (per - 1) + loc;
  }
#endif
  unsigned sk_unit = sk_first_unit(sk, wg);
  const unsigned sk_end = sk_first_unit(sk, wg + 1);
  unsigned sk_tile = wg;                             // the next whole tile: wg, wg + grid, ... below dp_tiles
  for (bool again = false; sk_unit < sk_end || sk_tile < sk.dp_tiles; again = true) {
  sk_segment seg;
  if (sk_unit < sk_end) {
    seg = sk_segment_at(sk, sk_unit, sk_end);
    sk_unit += seg.ke - seg.kb;
  } else {
    seg = sk_whole_tile(sk, sk_tile);
    sk_tile += sk.grid;
  }
  const int tile_m = (int)seg.tile_m, tile_n = (int)seg.tile_n;
  const int kb = (int)seg.kb;                       // first K step of the segment
  if (again) __syncthreads();                       // every wave is done with the LDS tiles of the previous segment
#else
  const int nbm = (M + BM - 1) / BM, nbn = (N + BN - 1) / BN;
  int tile_m, tile_n;
  if (!tile_of_workgroup(nbm, nbn, tile_m, tile_n)) return;
  constexpr int kb = 0;
  {
#endif
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // ---- global -> register staging: per-thread loop-invariant offsets ----
  unsigned a_goff[A_PER_T], b_goff[B_PER_T];
  int a_soff[A_PER_T], b_soff[B_PER_T];
  int a_kcol[A_PER_T], b_krow[B_PER_T];
  bool a_ok[A_PER_T], b_ok[B_PER_T][4];
#pragma unroll
  for (int i = 0; i < A_PER_T; ++i) {
    const int u = tid + i * NT;
#if DIRECT
    // LDS unit u of the tile is (row, slot u % CPR); it holds chunk slot ^ swizzle(row) of that row
    const int row = u / CPR, c = (u % CPR) ^ ((row / RPL) % SWZ_N);
#else
    const int row = u / (BK / 4), c = u % (BK / 4);
#endif
    a_goff[i] = (unsigned)(row * lda + c * 4) * 4u;
    a_soff[i] = row * LDA_S + c * 4;
    a_kcol[i] = c * 4;
    a_ok[i] = (A_UNITS % NT == 0 || u < A_UNITS) && (!EDGE || m0 + row < M);
  }
#pragma unroll
  for (int i = 0; i < B_PER_T; ++i) {
    const int u = tid + i * NT;
    const bool in = (B_UNITS % NT == 0 || u < B_UNITS);
#if TRANS_B
    // as for A, with the row of the tile standing for a (permuted) column of C; b_krow holds the
    // k offset of the unit inside the K step
#if DIRECT
    const int row = u / CPR, c = (u % CPR) ^ ((row / RPL) % SWZ_N);
#else
    const int row = u / (BK / 4), c = u % (BK / 4);
#endif
    const int col = bt_col_of_row(row);
    b_goff[i] = (unsigned)(col * ldb + c * 4) * 4u;
    b_soff[i] = row * LDB_S + c * 4;
    b_krow[i] = c * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) b_ok[i][e] = in && (!EDGE || n0 + col < N);
#else
    // LDS unit u sits in row krow of the tile at float column 4 * slot and holds tile column 4 * c
    const int krow = u / (BN / 4), slot = u % (BN / 4), c = b_tile_col(krow, slot * 4) / 4;
    b_goff[i] = (unsigned)(krow * ldb + c * 4) * 4u;
    b_soff[i] = krow * LDB_S + slot * 4;
    b_krow[i] = krow;
#pragma unroll
    for (int e = 0; e < 4; ++e) b_ok[i][e] = in && (!EDGE || n0 + c * 4 + e < N);
#endif
  }

  // The K loop below counts its steps from the segment's first one: operand bases start there and
  // Kl is what is left of K from there on (all of K, from the start, unless STREAMK).
  const int Kl = K - kb * BK;
#if TRANS_B
#define B_STEP(k0) (long)(k0)                             /* floats from Bg to K step k0 */
#else
#define B_STEP(k0) ((long)(k0) * ldb)
#endif
  const float* Ag = A + (long)m0 * lda + kb * BK;
  long a_rem = ((long)(M - m0 - 1) * lda + Kl) * 4;       // valid bytes from Ag to the end of A
#if TRANS_B
  const float* Bg = B + (long)n0 * ldb + B_STEP(kb * BK);
  long b_rem = ((long)(N - n0 - 1) * ldb + Kl) * 4;       // valid bytes from Bg to the end of Bt
#else
  const float* Bg = B + n0 + B_STEP(kb * BK);
  long b_rem = ((long)(Kl - 1) * ldb + (N - n0)) * 4;     // valid bytes from Bg to the end of B
#endif

#if !DIRECT
  v4f ra[A_PER_T], rb[B_PER_T];
#endif

#if STREAMK
  const int KT = (int)(seg.ke - seg.kb);                  // K steps of this segment
#else
  const int KT = (K + BK - 1) / BK;
#endif

#if DIRECT
  // Issues the loads of K step kt straight into LDS buffer `stage`.  Instruction i of a wave
  // fills the 64 consecutive 16-byte units that start at unit i*NT + wave*64 of the operand tile.
  // KTAIL (a compile-time 0/1) says whether tile kt may be the one that K ends in: only then are
  // the units tested against K (with dword-aligned rows: is the tile loaded float by float).
  auto fetch_direct = [&](auto ktail, int kt, int stage) __attribute__((always_inline)) {
    constexpr bool KTEST = EDGE_K && decltype(ktail)::value;
    typedef __attribute__((address_space(3))) void* lds_ptr_t;
    const int k0 = kt * BK;
    const bool live = kt < KT;
    const __amdgpu_buffer_rsrc_t ar = tile_rsrc(Ag + k0, live, a_rem - (long)k0 * 4);
    const __amdgpu_buffer_rsrc_t br = tile_rsrc(Bg + B_STEP(k0), live, b_rem - B_STEP(k0) * 4);
    float* As = lds + stage * A_STAGE;
    float* Bs = lds + LDS_BUFS * A_STAGE + stage * B_STAGE;
    if constexpr (DW_DIRECT && KTEST) {
      // Dword-aligned rows.  A tile past the end needs no request (no wait of this variant counts
      // loads: two LDS buffers), a full tile takes the 16-byte loads below, and the tile that K ends
      // in is loaded one float per lane: instruction j of a wave fills the 64 consecutive floats that
      // start at float j*NT + wave*64 of the operand tile's LDS image; float d of the image is
      // element d % 4 of 16-byte unit d / 4.  That is once per tile, so the offsets are worked out
      // from the thread number here (behind an opaque copy: otherwise they would be hoisted and
      // kept in registers across the loop) rather than carried.
      if (!live) return;
    }
    if (DW_DIRECT && KTEST && k0 + BK > Kl) {
      int t = tid;
      asm volatile("" : "+v"(t));
#pragma unroll
      for (int j = 0; j < A_DW_LOADS; ++j) {
        const int first = j * NT + wave * 64;
        if ((4 * A_UNITS) % NT == 0 || first < 4 * A_UNITS) {
          const int d = t + j * NT, u = d / 4, row = u / CPR, k = ((u % CPR) ^ ((row / RPL) % SWZ_N)) * 4 + d % 4;
          const bool ok = m0 + row < M && k0 + k < Kl;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(ar, (lds_ptr_t)(As + first), 4, ok ? (unsigned)(row * lda + k) * 4u : OOB_OFFSET, 0, 0, 0);
        }
      }
#pragma unroll
      for (int j = 0; j < B_DW_LOADS; ++j) {
        const int first = j * NT + wave * 64;
        if ((4 * B_UNITS) % NT == 0 || first < 4 * B_UNITS) {
          const int d = t + j * NT, u = d / 4;
#if TRANS_B
          const int row = u / CPR, k = ((u % CPR) ^ ((row / RPL) % SWZ_N)) * 4 + d % 4, col = bt_col_of_row(row);
          const bool ok = n0 + col < N && k0 + k < Kl;
          const unsigned off = (unsigned)(col * ldb + k) * 4u;
#else
          const int krow = u / (BN / 4), col = b_tile_col(krow, u % (BN / 4) * 4) + d % 4;
          const bool ok = n0 + col < N && k0 + krow < Kl;
          const unsigned off = (unsigned)(krow * ldb + col) * 4u;
#endif
          __builtin_amdgcn_raw_ptr_buffer_load_lds(br, (lds_ptr_t)(Bs + first), 4, ok ? off : OOB_OFFSET, 0, 0, 0);
        }
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < A_PER_T; ++i) {
      const int first = i * NT + wave * 64;
      if (A_UNITS % NT == 0 || first < A_UNITS) {
        const bool ok = a_ok[i] && (!KTEST || DW_DIRECT || k0 + a_kcol[i] < Kl);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ar, (lds_ptr_t)(As + first * 4), 16, ok ? a_goff[i] : OOB_OFFSET, 0, 0, 0);
      }
    }
    // (B[K,N] with dword-aligned rows: a unit that straddles N is loaded if its first column is inside;
    // what it brings beyond N only ever meets columns of C that are not stored)
#pragma unroll
    for (int i = 0; i < B_PER_T; ++i) {
      const int first = i * NT + wave * 64;
      if (B_UNITS % NT == 0 || first < B_UNITS) {
        const bool ok = b_ok[i][0] && (!KTEST || DW_DIRECT || k0 + b_krow[i] < Kl);  // K % 4 == 0: a chunk is in or out as a whole
        __builtin_amdgcn_raw_ptr_buffer_load_lds(br, (lds_ptr_t)(Bs + first * 4), 16, ok ? b_goff[i] : OOB_OFFSET, 0, 0, 0);
      }
    }
  };
#else

  // Issues the global loads of K step kt into the staging registers.  A step at or beyond KT
  // (the pipelined loop asks for up to two steps ahead) gets an empty resource: every load
  // returns 0 and touches no memory.  KTAIL (a compile-time 0/1) says whether tile kt may be the
  // one that K ends in: only then are the elements tested against K.
  auto fetch = [&](auto ktail, int kt) __attribute__((always_inline)) {
    constexpr bool KTEST = EDGE_K && decltype(ktail)::value;
    const int k0 = kt * BK;
    const bool live = kt < KT;
    const __amdgpu_buffer_rsrc_t ar = tile_rsrc(Ag + k0, live, a_rem - (long)k0 * 4);
    const __amdgpu_buffer_rsrc_t br = tile_rsrc(Bg + B_STEP(k0), live, b_rem - B_STEP(k0) * 4);
#pragma unroll
    for (int i = 0; i < A_PER_T; ++i) {
      const int k = k0 + a_kcol[i];
      ra[i] = load_unit<!KTEST>(ar, a_goff[i],
                                a_ok[i] && (!KTEST || k + 0 < Kl), a_ok[i] && (!KTEST || k + 1 < Kl),
                                a_ok[i] && (!KTEST || k + 2 < Kl), a_ok[i] && (!KTEST || k + 3 < Kl));
    }
#pragma unroll
    for (int i = 0; i < B_PER_T; ++i) {
#if TRANS_B
      const int k = k0 + b_krow[i];
      rb[i] = load_unit<!KTEST>(br, b_goff[i],
                                b_ok[i][0] && (!KTEST || k + 0 < Kl), b_ok[i][1] && (!KTEST || k + 1 < Kl),
                                b_ok[i][2] && (!KTEST || k + 2 < Kl), b_ok[i][3] && (!KTEST || k + 3 < Kl));
#else
      // Columns at or beyond N only ever meet columns of C that are not stored, so a unit that
      // straddles N needs no zeroing: it is loaded if its first column is inside (what lies
      // past the end of the last row of B is beyond the range and comes back as zero).
      const bool kin = !KTEST || k0 + b_krow[i] < Kl;
      rb[i] = load_unit<true>(br, b_goff[i], b_ok[i][0] && kin, false, false, false);
#endif
    }
  };

  auto stash = [&](int stage) __attribute__((always_inline)) {
    float* As = lds + stage * A_STAGE;
    float* Bs = lds + LDS_BUFS * A_STAGE + stage * B_STAGE;
#pragma unroll
    for (int i = 0; i < A_PER_T; ++i)
      if (A_UNITS % NT == 0 || tid + i * NT < A_UNITS) *(v4f*)&As[a_soff[i]] = ra[i];
#pragma unroll
    for (int i = 0; i < B_PER_T; ++i)
      if (B_UNITS % NT == 0 || tid + i * NT < B_UNITS) *(v4f*)&Bs[b_soff[i]] = rb[i];
  };
#endif

  acc_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < ACC_REGS; ++r) acc[i][j][r] = 0.0f;

#if DIRECT
  const int a_frag = (wm0 + lr) * LDA_S;            // + bi*MI*LDA_S + swizzled chunk of the round
  int a_round[SUPERS];
#pragma unroll
  for (int r = 0; r < SUPERS; ++r) a_round[r] = ((r * (KSUPER / 4) + lg) ^ ((lr / RPL) % SWZ_N)) * 4;
#else
  const int a_frag = (wm0 + lr) * LDA_S + 4 * lg;   // + bi*MI*LDA_S + kk
#endif
#if TRANS_B && DIRECT
  const int b_frag = (wn0 + lr) * LDB_S;                // + bj*MI*LDB_S + swizzled chunk of the round
#elif TRANS_B
  const int b_frag = (wn0 + lr) * LDB_S + 4 * lg;       // + bj*MI*LDB_S + kk
#else
  const int b_frag = (4 * lg) * LDB_S + wn0;            // + (kk+t)*LDB_S + b0*MI + w*lr per segment
  // LONE_SWAP: lanes of an odd k group find their wave's lone column block where the partner wave's is
  const int b_frag_lone = (4 * lg) * LDB_S + ((LONE_SWAP && (lg & 1)) ? (((wave % NWN) ^ 1) * WN) : wn0) + (TN - 1) * MI + lr;
#endif

  // One round of LDS fragment reads: TM 128-bit reads of A (four consecutive k each) and, for each
  // of the four k slots, one vector read of B per segment (TRANS_B: TN 128-bit reads, four
  // consecutive k of one column each).  Feeds 4*TM*TN MFMAs.
  struct frag_t {
    v4f a[TM];
#if TRANS_B
    v4f b[TN];
#else
    v4f b4[4][NSEG4 > 0 ? NSEG4 : 1];
    v2f b2[4];
    float b1[4];
#endif
  };
  auto read_frags = [&](frag_t& f, int stage, int kk) __attribute__((always_inline)) {
    const float* As = lds + stage * A_STAGE;
    const float* Bs = lds + LDS_BUFS * A_STAGE + stage * B_STAGE;
#pragma unroll
#if DIRECT
    for (int bi = 0; bi < TM; ++bi) f.a[bi] = *(const v4f*)&As[a_frag + bi * MI * LDA_S + a_round[kk / KSUPER]];
#else
    for (int bi = 0; bi < TM; ++bi) f.a[bi] = *(const v4f*)&As[a_frag + bi * MI * LDA_S + kk];
#endif
#if TRANS_B && DIRECT
#pragma unroll
    for (int bj = 0; bj < TN; ++bj) f.b[bj] = *(const v4f*)&Bs[b_frag + bj * MI * LDB_S + a_round[kk / KSUPER]];
#elif TRANS_B
#pragma unroll
    for (int bj = 0; bj < TN; ++bj) f.b[bj] = *(const v4f*)&Bs[b_frag + bj * MI * LDB_S + kk];
#else
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float* row = &Bs[b_frag + (kk + t) * LDB_S];
#pragma unroll
      for (int v = 0; v < NSEG4; ++v) f.b4[t][v] = *(const v4f*)&row[4 * v * MI + 4 * lr];
      if constexpr (HAS_SEG2) f.b2[t] = *(const v2f*)&row[4 * NSEG4 * MI + 2 * lr];
      if constexpr (HAS_SEG1) f.b1[t] = Bs[b_frag_lone + (kk + t) * LDB_S];
    }
#endif
  };
  auto mfma_frags = [&](const frag_t& f, int t0 = 0, int t1 = 4) __attribute__((always_inline)) {
#pragma unroll
    for (int t = t0; t < t1; ++t)
#pragma unroll
      for (int bi = 0; bi < TM; ++bi)
#pragma unroll
        for (int bj = 0; bj < TN; ++bj) {
#if TRANS_B
          const float bval = f.b[bj][t];
#else
          const float bval = bj < 4 * NSEG4 ? f.b4[t][bj / 4][bj % 4] : (HAS_SEG2 && bj < 4 * NSEG4 + 2 ? f.b2[t][bj - 4 * NSEG4] : f.b1[t]);
#endif
          acc[bi][bj] = MFMA(f.a[bi][t], bval, acc[bi][bj]);
        }
  };

  // ---- main loop ----
#if STAGES >= 3
  if (KT > 0) {
    // Software pipeline.  At the top of step kt: tile kt is in its LDS buffer, its first fragment
    // round is already in registers, and the staging registers hold tile kt+1 (loaded during step
    // kt-1).  Within the step each fragment round is read while the previous one is in the MFMA
    // pipe; before the last round is multiplied, tile kt+1 goes to the other LDS buffer, the
    // loads of tile kt+2 are issued, the workgroup meets at the barrier, and the first fragment
    // round of tile kt+1 is read -- so that the last MFMA group covers that read's latency.
    //
    // Instructions of the vector ALU take issue slots from the MFMAs (LDS reads and global loads
    // do not), so the loop carries none: with two LDS buffers the steps run two per loop trip, the
    // first of a pair on buffer 0 and the second on buffer 1, both compile-time constants (as is
    // the fragment set, which alternates too when a step has an odd number of rounds), and every
    // LDS address is a loop-invariant register plus an immediate offset.  The last step is always
    // on buffer 0; an odd number of pipelined steps therefore starts with a single step on buffer
    // 1, and tile 0 goes to buffer `first` = parity of the number of pipelined steps.
    frag_t fr[2];
    constexpr int ODD = SUPERS % 2;
    const int pipelined = KT - 1;
    const int first = pipelined & 1;
#if DIRECT
    // (dword-aligned rows: the number of loads per tile is known only if K cannot end in these tiles)
    if (!DW_DIRECT || KT > LDS_BUFS) {
#pragma unroll
      for (int i = 0; i < LDS_BUFS; ++i) fetch_direct(int_c<!DW_DIRECT>{}, i, LDS_BUFS == 2 ? (i ^ first) : i);
      // this wave's part of tile 0 is in LDS (of every requested tile when the loads per wave differ)
      WAIT_VMCNT(PROLOGUE_IN_FLIGHT);
    } else {
#pragma unroll
      for (int i = 0; i < LDS_BUFS; ++i) fetch_direct(int_c<1>{}, i, LDS_BUFS == 2 ? (i ^ first) : i);
      WAIT_VMCNT(0);
    }
#else
    fetch(int_c<1>{}, 0);
    stash(first);
    fetch(int_c<1>{}, 1);
#endif
    __syncthreads();
    if (first) {
      read_frags(fr[ODD], LDS_BUFS == 2 ? 1 : 0, 0);
    } else {
      read_frags(fr[0], 0, 0);
    }

    // P = which of the two fragment sets holds round 0 of this step (compile-time, so that the
    // sets stay in fixed registers); the set alternates every round.
    // MFMAs and fragment reads per round; LDS writes and global loads per K step
    constexpr int G = 4 * TM * TN, R = TM + (TRANS_B ? TN : 4 * NSEG), W = A_PER_T + B_PER_T, L = DIRECT ? LOADS_PER_TILE : W * (VEC == 4 ? 1 : 4);

    // `buffer`: the LDS buffer of this step's tile when there are two (with more, kt % LDS_BUFS).
    auto step = [&](auto parity, auto ktail, auto buffer, int kt) __attribute__((always_inline)) {
      constexpr int P = decltype(parity)::value;
      const int cur = LDS_BUFS == 2 ? decltype(buffer)::value : (unsigned)kt % LDS_BUFS;
      const int nxt = LDS_BUFS == 2 ? 1 - decltype(buffer)::value : (unsigned)(kt + 1) % LDS_BUFS;
#pragma unroll
      for (int r = 0; r + 1 < SUPERS; ++r) {
        read_frags(fr[(P + r + 1) & 1], cur, (r + 1) * KSUPER);
        mfma_frags(fr[(P + r) & 1]);
      }
      // the last round is split around the barrier: its first half covers the LDS writes of
      // tile kt+1 and the global loads of tile kt+2, its second half the first reads of tile kt+1
      // (DIRECT: one quarter before the barrier, three after it, which leaves room to issue the
      // loads of tile kt+2 behind every second MFMA instead of every one: measured 0.3-0.8 % faster)
#if DIRECT
      mfma_frags(fr[(P + SUPERS - 1) & 1], 0, 1);
      // Tile kt+1 was requested LDS_BUFS-1 steps ago, straight into the next buffer; once every
      // wave's part has landed (the requests for later tiles may still be in flight) and all have
      // met, buffer `cur` is free again and takes tile kt+LDS_BUFS.
#if SCHED
#pragma unroll
      for (int r = 0; r + 1 < SUPERS; ++r) interleave_with_mfma<G, R, 0x100>();
      // the barrier (and the wait for the LDS reads that comes with it) stays behind the MFMAs above:
      // left to float, it lands right behind the last read and the wave sits out that read's latency
      interleave_with_mfma<G / 4, 0, 0x100>();
      __builtin_amdgcn_sched_barrier(0);
#endif
      WAIT_VMCNT((LDS_BUFS - 2) * LOADS_PER_TILE);
      __syncthreads();
      read_frags(fr[(P + SUPERS) & 1], nxt, 0);
      fetch_direct(ktail, kt + LDS_BUFS, cur);
      mfma_frags(fr[(P + SUPERS - 1) & 1], 1, 4);
#if SCHED
      {
        constexpr int REST = 3 * G / 4, PAIRED = R < REST ? R : REST, LEFT = REST - PAIRED;
        interleave_with_mfma<PAIRED, R, 0x100>();
        if constexpr (LEFT >= 2 * L) {
          stride_with_mfma<LEFT, L, 0x020, 2>();
        } else {
          interleave_with_mfma<LEFT, L, 0x020>();
        }
      }
#endif
#else
      mfma_frags(fr[(P + SUPERS - 1) & 1], 0, 2);
      stash(nxt);
      fetch(ktail, kt + 2);
#if SCHED
#pragma unroll
      for (int r = 0; r + 1 < SUPERS; ++r) interleave_with_mfma<G, R, 0x100>();
      interleave_with_mfma<G / 4, W, 0x200>();
      interleave_with_mfma<G / 2 - G / 4, L, 0x020>();
#endif
      __syncthreads();
      read_frags(fr[(P + SUPERS) & 1], nxt, 0);
      mfma_frags(fr[(P + SUPERS - 1) & 1], 2, 4);
#if SCHED
      interleave_with_mfma<G / 2, R, 0x100>();
#endif
#endif
    };
    auto last_step = [&](auto parity, auto buffer, int kt) __attribute__((always_inline)) {
      constexpr int P = decltype(parity)::value;
      const int cur = LDS_BUFS == 2 ? decltype(buffer)::value : (unsigned)kt % LDS_BUFS;
#pragma unroll
      for (int r = 0; r + 1 < SUPERS; ++r) {
        read_frags(fr[(P + r + 1) & 1], cur, (r + 1) * KSUPER);
        mfma_frags(fr[(P + r) & 1]);
      }
      mfma_frags(fr[(P + SUPERS - 1) & 1]);
#if SCHED
#pragma unroll
      for (int r = 0; r + 1 < SUPERS; ++r) interleave_with_mfma<G, R, 0x100>();
#endif
#if DIRECT
      WAIT_VMCNT(0);  // the (empty) requests for the tiles past the end have drained
#endif
    };

    // One pair of steps: buffers 0 then 1.
    // (the scheduling fences keep the interleave directives of one step from picking up the
    // instructions of the other)
    auto pair = [&](auto ktail, int kt) __attribute__((always_inline)) {
      step(int_c<0>{}, ktail, int_c<0>{}, kt);
      __builtin_amdgcn_sched_barrier(0);
      step(int_c<ODD>{}, ktail, int_c<1>{}, kt + 1);
      __builtin_amdgcn_sched_barrier(0);
    };
    int kt = 0;
    if (first) {
      // (with a K edge this step may be the one that requests the last tile)
      step(int_c<ODD>{}, int_c<1>{}, int_c<1>{}, kt);
      ++kt;
    }
#if EDGE_K
    // Step kt requests tile kt + LDS_BUFS.  Only tile KT-1 can be cut short by K, so only the pair
    // with the step that requests it, and the pairs behind it (they request tiles past the end:
    // empty range, zeros whatever the test says), test their units against K.
    const int plain = pipelined - LDS_BUFS;     // steps before the one that requests tile KT-1
    for (; kt + 1 < plain; kt += 2) pair(int_c<0>{}, kt);
    for (; kt + 1 < pipelined; kt += 2) pair(int_c<1>{}, kt);
#else
    for (; kt + 1 < pipelined; kt += 2) pair(int_c<0>{}, kt);
#endif
    last_step(int_c<0>{}, int_c<0>{}, pipelined);
  }
#else
  static_assert(!DIRECT, "DIRECT belongs to the pipelined loop");
  auto multiply = [&](int stage) __attribute__((always_inline)) {
#pragma unroll
    for (int kk = 0; kk < BK; kk += KSUPER) {
      frag_t f;
      read_frags(f, stage, kk);
      mfma_frags(f);
    }
  };
  if (KT > 0) {
    fetch(int_c<1>{}, 0);
    stash(0);
  }
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const bool more = kt + 1 < KT;
#if STAGES == 2
    const int cur = kt & 1;
    if (more) fetch(int_c<1>{}, kt + 1);
    multiply(cur);
    if (more) stash(cur ^ 1);
    __syncthreads();
#else
    if (more) fetch(int_c<1>{}, kt + 1);
    multiply(0);
    __syncthreads();
    if (more) stash(0);
    __syncthreads();
#endif
  }
#endif

  // ---- epilogue: every accumulator leaves once ----
#if STREAMK
  // A segment that covers its tile's whole K range stores C like the plain kernel.  Any other is a
  // piece: it goes to this workgroup's slot in the workspace (slot 1 for a piece that starts the
  // tile, which can only be the workgroup's last segment; slot 0 for one that starts inside the
  // tile, which can only be its first), in the order the threads hold it.  The pieces of a tile
  // belong to consecutive workgroups, first_wg .. first_wg + pieces - 1 in K order.  Whoever finds
  // the tile's counter at pieces - 1 was last: it adds all pieces up in K order, its own included
  // (read back, so the sum is formed the same way whoever comes last), stores C and clears the
  // counter for the next launch.
  //
  // Pieces are written and read with the sc0 sc1 cache policy: stores go through the caches to
  // memory and loads come from there, past whatever this XCD's L2 holds, so a piece needs no
  // cache-wide write-back on the writer's side and no invalidate on the reader's (either of which would
  // empty the L2 that the other workgroups of the XCD share their operand panels through -- measured:
  // with fences the split cost more than it saved).  A writer waits until its stores have been
  // acknowledged (vmcnt 0) before its workgroup is counted in; the reader only reads once it has
  // seen the count.
  //
  // Everything below that depends on the thread number alone is the same for every segment, and
  // the compiler would work it out once, ahead of the segment loop, and keep it in registers through
  // every K loop (40 to 90 of them: the difference between one and two workgroups per CU for the
  // larger tiles).  The epilogue therefore derives its lane coordinates from an opaque copy.
  int tid_here = threadIdx.y * blockDim.x + threadIdx.x;
  asm volatile("" : "+v"(tid_here));
  const int tid = tid_here, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / NWN) * WM, wn0 = (wave % NWN) * WN, lr = lane % MI, lg = lane / MI;
  bool store_c = true;
  if (seg.kb != 0 || seg.ke != sk.kt) {
    constexpr int CHUNKS = ACC_REGS / 4;            // 16-byte chunks per MFMA block and lane
    const unsigned tile_unit = sk_tile_unit(sk, seg.tile);   // (shared) unit number of the tile's first K step
    const unsigned first_wg = sk_owner(sk, tile_unit);
    const unsigned pieces = sk_owner(sk, tile_unit + sk.kt - 1) - first_wg + 1;
    const unsigned my_slot = 2 * wg + (seg.kb == 0 ? 1 : 0);
    {
      const __amdgpu_buffer_rsrc_t wr = make_rsrc(sk_slots + (long)my_slot * (BM * BN), (long)BM * BN * 4);
#pragma unroll
      for (int bi = 0; bi < TM; ++bi) {
#pragma unroll
        for (int bj = 0; bj < TN; ++bj)
#pragma unroll
          for (int c = 0; c < CHUNKS; ++c) {
            const v4f v = {acc[bi][bj][4 * c], acc[bi][bj][4 * c + 1], acc[bi][bj][4 * c + 2], acc[bi][bj][4 * c + 3]};
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v), wr, (unsigned)((((bi * TN + bj) * CHUNKS + c) * NT + tid) * 16), 0, SK_COHERENT);
          }
        __builtin_amdgcn_sched_barrier(0);   // (a row of blocks at a time, see the reading side)
      }
    }
    // the piece has arrived in memory; then count this workgroup in
    WAIT_VMCNT(0);
    __syncthreads();
    if (tid == 0)
      lds[0] = __builtin_bit_cast(float, __hip_atomic_fetch_add(&sk_arrivals[seg.tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    __syncthreads();
    const unsigned before = __builtin_amdgcn_readfirstlane(__builtin_bit_cast(unsigned, lds[0]));
    store_c = before == pieces - 1;
    if (store_c) {
      // One row of MFMA blocks at a time, the pieces of that row in K order.  The loads of up to
      // AHEAD pieces are in flight together (every one is a round trip past the L2, and one after the
      // other they made a tile of many pieces wait for each in turn); AHEAD keeps them within 32
      // registers, and a row at a time keeps the kernel at two waves per SIMD (left alone, the
      // scheduler issues every load of a piece first and needs a second set of accumulators).
      constexpr int ROW_CHUNKS = TN * CHUNKS;
      constexpr int AHEAD = ROW_CHUNKS <= 2 ? 4 : ROW_CHUNKS <= 4 ? 2 : 1;
#pragma unroll
      for (int bi = 0; bi < TM; ++bi) {
        for (unsigned p0 = 0; p0 < pieces; p0 += AHEAD) {
          v4f v[AHEAD][ROW_CHUNKS];
#pragma unroll
          for (int a = 0; a < AHEAD; ++a) {
            // past the last piece: the last one again (loaded, not added)
            const unsigned piece = p0 + a < pieces ? p0 + a : pieces - 1;
            const unsigned slot = piece == 0 ? 2 * first_wg + 1 : 2 * (first_wg + piece);
            const __amdgpu_buffer_rsrc_t rr = make_rsrc(sk_slots + (long)slot * (BM * BN), (long)BM * BN * 4);
#pragma unroll
            for (int bj = 0; bj < TN; ++bj)
#pragma unroll
              for (int c = 0; c < CHUNKS; ++c)
                v[a][bj * CHUNKS + c] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rr, (unsigned)((((bi * TN + bj) * CHUNKS + c) * NT + tid) * 16), 0, SK_COHERENT));
          }
#pragma unroll
          for (int a = 0; a < AHEAD; ++a) {
            if (p0 + a < pieces) {               // the same for every lane
#pragma unroll
              for (int bj = 0; bj < TN; ++bj)
#pragma unroll
                for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
                  for (int e = 0; e < 4; ++e)
                    acc[bi][bj][4 * c + e] = p0 + a == 0 ? v[a][bj * CHUNKS + c][e] : acc[bi][bj][4 * c + e] + v[a][bj * CHUNKS + c][e];
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (tid == 0) __hip_atomic_store(&sk_arrivals[seg.tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (store_c) {
#else
  {
#endif
  float* Cg = C + (long)m0 * ldc + n0;
  const __amdgpu_buffer_rsrc_t cr = make_rsrc(Cg, ((long)(M - m0 - 1) * ldc + (N - n0)) * 4);
#pragma unroll
  for (int bi = 0; bi < TM; ++bi)
#pragma unroll
    for (int r = 0; r < ACC_REGS; ++r) {
      const int row = wm0 + bi * MI + ACC_ROW(r, lg);
      const bool rok = !EDGE || m0 + row < M;
#pragma unroll
      for (int sg = 0; sg < NSEG; ++sg) {
        const int b0 = seg_first(sg), sw = seg_width(sg);
        const int col = wn0 + b0 * MI + sw * lr;
        const unsigned off = (unsigned)(row * ldc + col) * 4u;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = e < sw ? acc[bi][b0 + (e < sw ? e : 0)][r] : 0.0f;
        if (VEC == 4 && sw == 4) {
          const unsigned po = rok && (!EDGE || n0 + col < N) ? off : OOB_OFFSET;
          v4f out = {o[0], o[1], o[2], o[3]};
#if ACCUM
          out += __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(cr, po, 0, 0));
#endif
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, out), cr, po, 0, C_STORE_AUX);
        } else if (VEC == 4 && sw == 2) {
          const unsigned po = rok && (!EDGE || n0 + col < N) ? off : OOB_OFFSET;
          v2f out = {o[0], o[1]};
#if ACCUM
          out += __builtin_bit_cast(v2f, __builtin_amdgcn_raw_buffer_load_b64(cr, po, 0, 0));
#endif
          __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u, out), cr, po, 0, C_STORE_AUX);
        } else {
#pragma unroll
          for (int e = 0; e < sw; ++e) {
            const unsigned po = rok && (!EDGE || n0 + col + e < N) ? off + 4u * e : OOB_OFFSET;
            float out = o[e];
#if ACCUM
            out += __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(cr, po, 0, 0));
#endif
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, out), cr, po, 0, C_STORE_AUX);
          }
        }
      }
    }
  }   // store_c
  }   // segment
}
