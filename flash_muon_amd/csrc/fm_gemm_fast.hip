// Fast path of the bf16 (or fp16) NT contraction for gfx950: 256x256 output tiles, 4 waves (one per SIMD) of
// 128x128 each, 64-wide k stages copied global -> LDS by the DMA form of global_load (no VGPR
// staging) into a ring of three stages of operand A and two of operand B.
//
// Schedule.  One workgroup per CU.  Tiles are taken in rounds of `grid` whole tiles: all workgroups
// start a tile together and walk k in step, so the workgroups of one XCD, which hold a compact
// block of tiles, find each other's operand panels in their shared L2.  What is left after the
// last full round (fewer tiles than workgroups) is cut so that the last round is as short as its
// share of the work: in space, into 64x64 sub-tiles over the whole k, when at most a sixteenth as
// many tiles as workgroups are left (nothing is added up afterwards; of a symmetric product the
// tiles left are diagonal ones); otherwise along k into `split` parts per tile, one part per
// workgroup, which go to memory as fp32 and are added in part order by a second, small kernel that
// also runs the epilogue.  A product whose 128x256 half tiles fit into one round runs on those, and
// one of at most 16 tiles may run on sub-tiles altogether.
#include "fm_internal.h"

#include <type_traits>
#include <cstdlib>
#include <atomic>
#include <chrono>

namespace fm {

namespace {

constexpr int BM = 256, BN = 256, BKF = 64;
constexpr int ROWB = BKF * 2;               // bytes per LDS row
constexpr int OPER_BYTES = BM * ROWB;       // one operand stage: 32 KiB
constexpr int PART_FLOATS = BM * BN;        // one fp32 partial tile
constexpr int kMaxParts = 64;               // parts one tile can be cut into
constexpr int kMaxSlots = 768;              // partial-tile slots a schedule may use (192 MiB)
constexpr int kMaxGrid = 256;               // workgroups per launch: the XCD remap and the slot count assume no more
constexpr int kMaxKsplit = 16;              // base parts per tile

#define FM_LDS_ADDR(p) ((uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)(p)))

// One wave-wide global -> LDS copy of 16 bytes per lane: lane l lands at lds_base + 16*l.
// The compiler does not see the LDS write, so every use is ordered by hand with
// s_waitcnt vmcnt + s_barrier before the data is read.
__device__ __forceinline__ void dma16(uint32_t voff, const void* sbase, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(sbase), "s"(lds_base) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}

// LDS during the main loop: three stages of operand A and two of operand B, 32 KiB each, in the
// order A0 A1 B0 B1 A2.  Stage s of A sits in A slot s % 3, stage s of B in B slot s % 2.  A
// ds_read takes a 16-bit immediate offset, so one address register reaches two neighbouring slots:
// the fragment addresses are kept for the windows at 0 (A0, A1), 64 KiB (B0, B1) and 128 KiB (A2)
// and no address arithmetic is left in the loop (every VALU instruction between two MFMAs delays
// the second one by its own issue time).
__host__ __device__ constexpr int a_slot_off(int slot) { return slot == 2 ? 4 * OPER_BYTES : slot * OPER_BYTES; }
__host__ __device__ constexpr int b_slot_off(int slot) { return (2 + slot) * OPER_BYTES; }

// one global -> LDS copy with the destination given as an offset from the wave's copy base.
// (s_add_i32 writes SCC: without the clobber the compiler keeps the carry of a 64-bit pointer
// addition alive across the statement, and a panel that crosses a 4 GiB boundary is then read
// 4 GiB too low.)
__device__ __forceinline__ void dma16o(uint32_t voff, const void* sbase, uint32_t lds_base, int off) {
  asm volatile("s_add_i32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(sbase), "s"(lds_base), "n"(off) : "memory", "scc", "m0");
}

// The same copy in two statements with other instructions between them: the destination goes to M0
// first (the instruction between is the wait state the copy needs after a write of M0), the copy
// itself follows.  Nothing between the two may write M0; tests/test_generated_code.py looks for that
// in the generated code.
__device__ __forceinline__ void dma16_m0(uint32_t lds_base, int off) {
  asm volatile("s_add_i32 m0, %0, %1" :: "s"(lds_base), "n"(off) : "scc", "m0");
}
__device__ __forceinline__ void dma16_go(uint32_t voff, const void* sbase) {
  asm volatile("global_load_lds_dwordx4 %0, %1" :: "v"(voff), "s"(sbase) : "memory");
}

// ---- whole tiles on 16x16x32 MFMAs --------------------------------------------------------------
// A whole 256x256 tile runs on the 16x16x32 form of the instruction: on N(0,1) operands a loop of
// nothing but MFMAs sustains 2.03 PFLOP/s with it and 1.78 with the 32x32x16 form, the power cap
// allowing a clock of 2.0 against 1.77 GHz.  A wave's 128x128 block is 8 x 8 accumulator tiles of four
// registers; a 64-wide k stage is two k32 substeps of 64 MFMAs and 16 fragment reads each.
//
// Layout.  A lane of a 16x16 accumulator tile holds four consecutive rows (4 (lane / 16) + r) of one
// column (lane % 16) of the rows and columns its fragments were loaded with, and those are chosen so
// that the write-out needs no exchange between lanes: LDS row l of an operand stage holds row
// perm_a(l) of operand A's panel and row perm_b(l) of operand B's (permutations inside groups of 32
// rows, applied where the copies fetch from global memory, so that a fragment is 16 consecutive LDS
// rows).  Fragment i of A is then rows 32 (i / 2) + 8 g + 4 (i % 2) + r of the block for the lanes of
// group g = lane / 16, and fragment j of B columns 32 (j / 2) + 2 n + j % 2 for lane n = lane % 16:
// per 32x32 sub-block a lane holds 8 consecutive rows of 2 adjacent columns, i.e. after rounding a
// 32-bit word of every one of 8 rows of C (two columns) and 16 bytes of two rows of C2 (eight rows).
//
// 16-byte chunk c of LDS row r sits at position c ^ swz16(r); the 16 rows of a fragment then cover
// all 64 banks once per chunk column, and a fragment 16 rows further down is the same per-lane
// address plus 2048 bytes: six address registers in all, the rest is immediate offsets.
__device__ __forceinline__ int swz16(int row) { return (row >> 1) & 7; }
__host__ __device__ constexpr int perm_a(int l) { return (l & ~31) + 8 * ((l >> 2) & 3) + 4 * ((l >> 4) & 1) + (l & 3); }
__host__ __device__ constexpr int perm_b(int l) { return (l & ~31) + 2 * (l & 15) + ((l >> 4) & 1); }

template <bool F16>
__device__ __forceinline__ f32x4_t mfma_16x16x32(bf16x8_t a, bf16x8_t b, f32x4_t c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// NA: 16-row fragments of operand A per wave: 8 for a whole tile (128 rows), 4 for a 128x256 half tile (64 rows)
template <int NA> struct Frag16 { bf16x8_t a[NA], b[8]; };
// per-lane LDS byte addresses of fragment 0 for k32 substep kk: operand A in A slots 0 and 1
// (a_lo, + OPER_BYTES) and in A slot 2 (a_hi), operand B in B slots 0 and 1
struct FragAddr16 { uint32_t a_lo[2], a_hi[2], b[2]; };

template <int ASLOT>
__device__ __forceinline__ bf16x8_t read_a16(const unsigned char* smem, const FragAddr16& fa, int i, int kk) {
  if constexpr (ASLOT == 2) return *reinterpret_cast<const bf16x8_t*>(smem + fa.a_hi[kk] + i * 2048);
  else return *reinterpret_cast<const bf16x8_t*>(smem + fa.a_lo[kk] + ASLOT * OPER_BYTES + i * 2048);
}
template <int BSLOT>
__device__ __forceinline__ bf16x8_t read_b16(const unsigned char* smem, const FragAddr16& fa, int j, int kk) {
  return *reinterpret_cast<const bf16x8_t*>(smem + fa.b[kk] + BSLOT * OPER_BYTES + j * 2048);
}

// The 8 NA MFMAs of k32 substep KK of the stage in (ASLOT, BSLOT).  The NA + 8 fragment reads of the
// next substep (the second half of this stage, or the first half of the next one) ride on the first
// 2 (NA + 8) of them, in the order the next substep needs them.  During substep 0 the NA copies of
// operand A of the stage two ahead go out, into the A slot the previous stage has left; during
// substep 1, behind the barrier of the stage, the 8 copies of operand B of that stage, into the B slot
// this stage has just read for the last time.  Both go out evenly over their substep, one copy every
// 8 MFMAs of a whole tile: the same copies bunched up behind the barrier, where they would have longer
// to land, measured 2 % slower.
template <bool F16, int NA, int ASLOT, int BSLOT, int KK, bool FIRST>
__device__ __forceinline__ void substep16(f32x4_t (&acc)[NA][8], const Frag16<NA>& cur, Frag16<NA>& nxt,
                                          const unsigned char* smem, const FragAddr16& fa,
                                          const uint32_t (&voA)[NA], const uint32_t (&voB)[8],
                                          const bf16_t* gA, const bf16_t* gB, uint32_t ldsw) {
  constexpr int AFREE = (ASLOT + 2) % 3, ANEXT = (ASLOT + 1) % 3, BNEXT = BSLOT ^ 1;
  // every fragment of this substep was asked for half a substep ago: one wait for all of them, said
  // in the form the compiler's bookkeeping of outstanding reads understands, instead of one in front
  // of the first use of each
  if constexpr (KK == 0) __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0)
#pragma unroll
  for (int q = 0; q < 8 * NA; ++q) {
    if ((q & 1) == 0 && q < 2 * (NA + 8)) {
      const int t = q >> 1;   // read t of the next substep: a0, b0 .. b7, a1 .. a(NA - 1)
      if constexpr (KK == 0) {
        if (t == 0) nxt.a[0] = read_a16<ASLOT>(smem, fa, 0, 1);
        else if (t <= 8) nxt.b[t - 1] = read_b16<BSLOT>(smem, fa, t - 1, 1);
        else nxt.a[t - 8] = read_a16<ASLOT>(smem, fa, t - 8, 1);
      } else {
        if (t == 0) nxt.a[0] = read_a16<ANEXT>(smem, fa, 0, 0);
        else if (t <= 8) nxt.b[t - 1] = read_b16<BNEXT>(smem, fa, t - 1, 0);
        else nxt.a[t - 8] = read_a16<ANEXT>(smem, fa, t - 8, 0);
      }
    }
    // (a copy is two statements, M0 and the copy, one MFMA apart, in the slots that carry no read)
    if constexpr (KK == 0) {
      if ((q & 7) == 5) dma16_m0(ldsw, a_slot_off(AFREE) + (q >> 3) * 4096);
      if ((q & 7) == 7) dma16_go(voA[q >> 3], gA);
    } else {
      if (q % NA == 1) dma16_m0(ldsw, b_slot_off(BSLOT) + (q / NA) * 4096);
      if (q % NA == 3) dma16_go(voB[q / NA], gB);
    }
    if constexpr (FIRST && KK == 0) {
      const f32x4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
      acc[q >> 3][q & 7] = mfma_16x16x32<F16>(cur.a[q >> 3], cur.b[q & 7], zero);
    } else {
      acc[q >> 3][q & 7] = mfma_16x16x32<F16>(cur.a[q >> 3], cur.b[q & 7], acc[q >> 3][q & 7]);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// One k stage.  At the barrier between its substeps every wave has waited for its copies of the
// next stage (all but the NA newest, operand A of the stage after), and every fragment read of this
// stage has returned, so that its B slot may be refilled.
template <bool F16, int NA, int ASLOT, int BSLOT, bool FIRST = false>
__device__ __forceinline__ void stage16(f32x4_t (&acc)[NA][8], Frag16<NA>& f0, Frag16<NA>& f1, const unsigned char* smem,
                                        const FragAddr16& fa, const uint32_t (&voA)[NA], const uint32_t (&voB)[8],
                                        const bf16_t* nA, const bf16_t* nB, uint32_t ldsw) {
  substep16<F16, NA, ASLOT, BSLOT, 0, FIRST>(acc, f0, f1, smem, fa, voA, voB, nA, nB, ldsw);
  __builtin_amdgcn_s_waitcnt(0x0070 | NA);   // vmcnt(NA) lgkmcnt(0)
  asm volatile("s_barrier" ::: "memory");
  substep16<F16, NA, ASLOT, BSLOT, 1, false>(acc, f1, f0, smem, fa, voA, voB, nA, nB, ldsw);
}

// ---- a diagonal tile of a symmetric product as one item of the half-tile schedule ---------------
// Of the 8 x 8 MFMA tiles of a diagonal 256x256 tile only those on or below the diagonal are
// distinct: 36, against the 32 of a half tile, 9 per wave.  Waves 0 and 1 take the lower triangles
// of the two 128x128 squares on the diagonal, without tile (1, 0) (4 fragments, 9 MFMAs per
// substep); waves 2 and 3 a 64x128 half each of the square above the diagonal, in the shape of any
// other wave of the half-tile kernel, and tile (1, 0) of the first and the second square (two more
// fragments, read once more rather than picked from the six at the cost of vector instructions
// among the MFMAs).  Both operands are the one 256-row panel, which goes round the three A slots
// (8 copies per wave and stage, issued two stages ahead); the B slots are idle.
struct DFrag { bf16x8_t f[8]; };   // triangle waves: rows 32q of their square; the others: 2 row, 4 column fragments and the ninth tile's two
struct DFragAddr { uint32_t lo[8][4], hi[8][4]; };   // A slots 0 and 1 / A slot 2

template <int ASLOT>
__device__ __forceinline__ bf16x8_t read_d(const unsigned char* smem, const DFragAddr& fa, int q, int ks) {
  if constexpr (ASLOT == 2) return *reinterpret_cast<const bf16x8_t*>(smem + fa.hi[q][ks]);
  else return *reinterpret_cast<const bf16x8_t*>(smem + fa.lo[q][ks] + ASLOT * OPER_BYTES);
}

// where a triangle wave keeps MFMA tile (i, j), j <= i, among its 3 x 4 accumulator tuples
__host__ __device__ constexpr int tri_r(int i, int j) { return i < 3 ? i : (j < 3 ? 0 : 1); }
__host__ __device__ constexpr int tri_c(int i, int j) { return i < 3 ? j : (j < 3 ? j + 1 : 2); }
// row and column fragment of MFMA q of a triangle wave: (0,0) (1,1) (2,0) (2,1) (2,2) (3,0) .. (3,3)
__host__ __device__ constexpr int tri_i(int q) { return q < 2 ? q : q < 5 ? 2 : 3; }
__host__ __device__ constexpr int tri_j(int q) { return q < 2 ? q : q < 5 ? q - 2 : q - 5; }

// the 9 MFMAs of one substep, with the fragment reads of `ks_next` of slot RSLOT riding on the
// first ones and copies Q0 .. Q1-1 of the panel two stages ahead on the later ones.
template <bool F16, bool TRI, int RSLOT, int Q0, int Q1, int CSLOT, bool FIRST>
__device__ __forceinline__ void dsubstep(f32x16_t (&acc)[3][4], const DFrag& cur, DFrag& nxt, const unsigned char* smem,
                                         const DFragAddr& fa, int ks_next, const uint32_t (&vo)[8], const bf16_t* gP,
                                         uint32_t ldsw) {
  constexpr int NM = 9, NRD = TRI ? 4 : 8;
  constexpr int C0 = 5, CSTEP = 1;   // copies after MFMA 5, 6, 7
#pragma unroll
  for (int q = 0; q < NM; ++q) {
    if (q < NRD) nxt.f[q] = read_d<RSLOT>(smem, fa, q, ks_next);
    if (q >= C0 && (q - C0) % CSTEP == 0 && Q0 + (q - C0) / CSTEP < Q1)
      dma16o(vo[Q0 + (q - C0) / CSTEP], gP, ldsw, a_slot_off(CSLOT) + (Q0 + (q - C0) / CSTEP) * 4096);
    const f32x16_t zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if constexpr (TRI) {
      f32x16_t& c = acc[tri_r(tri_i(q), tri_j(q))][tri_c(tri_i(q), tri_j(q))];
      c = mfma_32x32x16<F16>(cur.f[tri_i(q)], cur.f[tri_j(q)], FIRST ? zero : c);
    } else if (q < 8) {
      f32x16_t& c = acc[q >> 2][q & 3];
      c = mfma_32x32x16<F16>(cur.f[q >> 2], cur.f[2 + (q & 3)], FIRST ? zero : c);
    } else {   // tile (1, 0) of a diagonal square: rows 32 .. 63 times rows 0 .. 31 of it
      acc[2][0] = mfma_32x32x16<F16>(cur.f[6], cur.f[7], FIRST ? zero : acc[2][0]);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// one k stage of the panel in A slot ASLOT
template <bool F16, bool TRI, int ASLOT, bool FIRST>
__device__ __forceinline__ void dstage(f32x16_t (&acc)[3][4], DFrag& f0, DFrag& f1, const unsigned char* smem,
                                       const DFragAddr& fa, const uint32_t (&vo)[8], const bf16_t* nP, uint32_t ldsw) {
  constexpr int AFREE = (ASLOT + 2) % 3, ANEXT = (ASLOT + 1) % 3;
  dsubstep<F16, TRI, ASLOT, 0, 3, AFREE, FIRST>(acc, f0, f1, smem, fa, 1, vo, nP, ldsw);
  dsubstep<F16, TRI, ASLOT, 3, 6, AFREE, false>(acc, f1, f0, smem, fa, 2, vo, nP, ldsw);
  dsubstep<F16, TRI, ASLOT, 6, 8, AFREE, false>(acc, f0, f1, smem, fa, 3, vo, nP, ldsw);
  // everybody's copies of the next stage have landed (all but the 8 newest, of the stage after),
  // and nobody reads the slot that the next stage's copies go to
  asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  dsubstep<F16, TRI, ANEXT, 0, 0, AFREE, false>(acc, f1, f0, smem, fa, 0, vo, nP, ldsw);
}

// ---- the part of a tile after the main loop -----------------------------------------------------
// Each wave finishes its 128x128 block a quarter (32 rows x 128 columns, one row of MFMA tiles) at
// a time, in its own LDS region:
//   F  fp32 accumulators of the quarter, column-major (F[c][r], 4-row groups XOR-swizzled by c/8):
//      written 16 bytes per lane straight from the accumulator layout, read without serious bank
//      conflicts by both passes below;
//   E  the epilogue operand of the quarter (bf16, row-major), two buffers, brought in by the DMA
//      form of global_load while the previous quarter is being written out;
//   RA the per-row additions to alpha of the block's 128 rows.
// Nothing is loaded from global memory between the stores of a tile: a load issued after a store
// has to wait for that store as well (one counter tracks both), and a loop of load-compute-store
// then runs at one memory round trip per iteration.
constexpr int QF_PITCH = 36;                              // floats per column: 32 rows + 4 of padding
constexpr int QF_FLOATS = 128 * QF_PITCH;                 // 18432 bytes
constexpr int QE_BYTES = 32 * 256;                        // one E buffer: 32 rows of 128 bf16
constexpr int EPI_WAVE_BYTES = QF_FLOATS * 4 + 2 * QE_BYTES + 512;   // 35328
constexpr int QUARTER_FLOATS = 128 * 32;                  // fp32 values of a quarter (partial tiles)
constexpr int SMEM_BYTES = 5 * OPER_BYTES;                // 163840: the operand ring; the staging needs 4 * EPI_WAVE_BYTES = 141312

struct EpiLds {
  float* F;
  unsigned char* E[2];
  float* RA;
  uint32_t e_addr[2];   // LDS byte addresses of the E buffers, for the DMA
};
__device__ __forceinline__ EpiLds epi_lds(unsigned char* wave_base) {
  EpiLds l;
  l.F = reinterpret_cast<float*>(wave_base);
  l.E[0] = wave_base + QF_FLOATS * 4;
  l.E[1] = l.E[0] + QE_BYTES;
  l.RA = reinterpret_cast<float*>(l.E[1] + QE_BYTES);
  l.e_addr[0] = FM_LDS_ADDR(l.E[0]);
  l.e_addr[1] = FM_LDS_ADDR(l.E[1]);
  return l;
}

// float index of row r (0..31) of column c (0..127) in F
__device__ __forceinline__ int qf_idx(int c, int r) { return c * QF_PITCH + (r ^ (((c >> 3) & 7) << 2)); }

// One 32x32 MFMA tile of the accumulators -> columns 32 ct .. +31 of a staged quarter: register 4q+e of
// lane l is row 8q + 4(l/32) + e, column l%32 of the tile, four consecutive rows of one column.
__device__ __forceinline__ void stage_tile(const f32x16_t& a, float* F, int ct, int lane) {
  const int col = 32 * ct + (lane & 31), rg = 4 * (lane >> 5);
  float* const dst = F + col * QF_PITCH;
  const int x = ((col >> 3) & 7) << 2;
  *reinterpret_cast<f32x4_t*>(dst + ((0 + rg) ^ x)) = __builtin_shufflevector(a, a, 0, 1, 2, 3);
  *reinterpret_cast<f32x4_t*>(dst + ((8 + rg) ^ x)) = __builtin_shufflevector(a, a, 4, 5, 6, 7);
  *reinterpret_cast<f32x4_t*>(dst + ((16 + rg) ^ x)) = __builtin_shufflevector(a, a, 8, 9, 10, 11);
  *reinterpret_cast<f32x4_t*>(dst + ((24 + rg) ^ x)) = __builtin_shufflevector(a, a, 12, 13, 14, 15);
}

// the 128 x 32 floats of the staged quarter, in staging order, to a partial-tile slot (coalesced)
__device__ __forceinline__ void copy_stage_to_ws(const float* F, float* dst, int lane) {
#pragma unroll 8
  for (int it = 0; it < 16; ++it) {
    const int idx = it * 64 + lane;             // 16-byte unit: column idx/8, 4-row group idx%8
    const f32x4_t v = *reinterpret_cast<const f32x4_t*>(F + (idx >> 3) * QF_PITCH + (idx & 7) * 4);
    *reinterpret_cast<f32x4_t*>(dst + idx * 4) = v;
  }
}

// sum of the `nparts` parts of one quarter (slot numbers in `slots`, in k order) into F, added in that
// order; `parts` points at the quarter inside slot 0; this wave takes the 16-byte units
// it_begin*64 .. it_end*64.  Loads go out eight parts at a time.
__device__ __forceinline__ void sum_parts_to_stage(const float* parts, const int* slots, int nparts, float* F,
                                                   int lane, int it_begin, int it_end, int slot_floats = PART_FLOATS) {
  for (int it = it_begin; it < it_end; ++it) {
    const int idx = it * 64 + lane;
    f32x4_t v = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int t0 = 0; t0 < nparts; t0 += 8) {
      f32x4_t x[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int tt = (t0 + t < nparts) ? t0 + t : nparts - 1;   // clamped; the value is dropped below
        x[t] = *reinterpret_cast<const f32x4_t*>(parts + (size_t)slots[tt] * slot_floats + idx * 4);
      }
#pragma unroll
      for (int t = 0; t < 8; ++t) if (t0 + t < nparts) v += x[t];
    }
    *reinterpret_cast<f32x4_t*>(F + (idx >> 3) * QF_PITCH + (idx & 7) * 4) = v;
  }
}

// DMA of the epilogue operand of quarter q of the block (32 rows x 256 bytes) into an E buffer:
// copies n_begin .. n_end of the 8 (4 rows each) are issued by the calling wave
__device__ __forceinline__ void epi_dma_e(const GemmArgs& g, int row_base, int col_base, int lane,
                                          uint32_t lds_addr, int n_begin, int n_end) {
  const bf16_t* src = g.E + (int64_t)row_base * g.lde + col_base;
  for (int n = n_begin; n < n_end; ++n) {
    const uint32_t voff = (uint32_t)(((n * 4 + (lane >> 4)) * (int)g.lde + (lane & 15) * 8) * 2);
    dma16(voff, src, lds_addr + n * 1024);
  }
}

// Epilogue of the staged quarter: rows row_base .. +32, columns col_base .. +128, iterations
// it_begin .. it_end (of 8) of each pass.  The direct pass (passes & 1) writes C, 1 row x 8 columns
// per lane, and puts the rounded values back into F when an operand was added; the transposed pass
// (passes & 2) writes C2, 8 rows x 1 column per lane, from F.  Both store 16 bytes per lane, and
// both copies carry the same bits.
// HAS_E: v = (alpha + row_alpha) * E + beta * acc, else v = acc.
// DIAG: a diagonal tile of a symmetric product.  Its own mirror image lies inside the tile, and the
// accumulators at (i, j) and (j, i) already hold the same bits: both add the same exact products
// x_ik * x_jk in the same order, through the same dot-product datapath.  So such a tile is written
// once, whole, by the direct pass and has no transposed pass.  The fp32 diagonal, if asked for, is
// split off here.
// G iterations of the direct pass with an operand E, off the diagonal: every LDS read of the batch
// is issued before the first value is put back into F, so the batch pays one LDS round trip and
// not one per iteration (a read may not be moved above an earlier write to F by the compiler).
template <bool F16, int G>
__device__ __forceinline__ void direct_e_batch(const GemmArgs& g, float* F, const unsigned char* Eb, const float* RA,
                                               int ra_off, int row_base, int col_base, int lane, int it0) {
  const float alpha = g.alpha, beta = g.beta;
  unsigned short* C = reinterpret_cast<unsigned short*>(g.C);
  float v[G][8], al[G];
  union { uint4 v; unsigned short s[8]; } e[G];
#pragma unroll
  for (int n = 0; n < G; ++n) {
    const int idx = (it0 + n) * 64 + lane;
    const int r = idx >> 4, c0 = (idx & 15) * 8;
#pragma unroll
    for (int k = 0; k < 8; ++k) v[n][k] = F[qf_idx(c0 + k, r)];
    e[n].v = *reinterpret_cast<const uint4*>(Eb + r * 256 + c0 * 2);
    al[n] = alpha + RA[ra_off + r];
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int n = 0; n < G; ++n) {
    const int idx = (it0 + n) * 64 + lane;
    const int r = idx >> 4, c0 = (idx & 15) * 8;
    union { uint4 v; unsigned short s[8]; } o;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      o.s[k] = f32_to_elem<F16>(__builtin_fmaf(al[n], elem_to_f32<F16>(e[n].s[k]), beta * v[n][k]));
      F[qf_idx(c0 + k, r)] = elem_to_f32<F16>(o.s[k]);   // what the transposed pass stores
    }
    if (C) *reinterpret_cast<uint4*>(C + (int64_t)(row_base + r) * g.c_rs + col_base + c0) = o.v;
  }
}

template <bool F16, bool HAS_E, bool DIAG>
__device__ __forceinline__ void epilogue_quarter_t(const GemmArgs& g, float* F, const unsigned char* Eb,
                                                   const float* RA, int ra_off, int row_base, int col_base,
                                                   int lane, int it_begin, int it_end, int passes) {
  const float alpha = g.alpha, beta = g.beta;
  const bool dout = DIAG && g.diag_out != nullptr;
  if constexpr (HAS_E && !DIAG) {
    if (passes & 1) {
      int it = it_begin;
      for (; it + 4 <= it_end; it += 4) direct_e_batch<F16, 4>(g, F, Eb, RA, ra_off, row_base, col_base, lane, it);
      for (; it + 2 <= it_end; it += 2) direct_e_batch<F16, 2>(g, F, Eb, RA, ra_off, row_base, col_base, lane, it);
      if (it < it_end) direct_e_batch<F16, 1>(g, F, Eb, RA, ra_off, row_base, col_base, lane, it);
    }
  } else if ((passes & 1) && (g.C || HAS_E)) {
    unsigned short* C = reinterpret_cast<unsigned short*>(g.C);
#pragma unroll 4
    for (int it = it_begin; it < it_end; ++it) {
      const int idx = it * 64 + lane;
      const int r = idx >> 4, c0 = (idx & 15) * 8;     // row r, columns c0 .. c0+7 of the quarter
      const int row = row_base + r, col = col_base + c0;
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = F[qf_idx(c0 + k, r)];
      union { uint4 v; unsigned short s[8]; } e, o;
      if (HAS_E) {
        e.v = *reinterpret_cast<const uint4*>(Eb + r * 256 + c0 * 2);
        const float al = alpha + RA[ra_off + r];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = __builtin_fmaf(al, elem_to_f32<F16>(e.s[k]), beta * v[k]);
      }
      if (DIAG) {                                       // selects only: no branch per element
        const int kd = row - col;                       // the diagonal element of this row, if 0..7
        float dv = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const bool on = dout && kd == k;
          dv = on ? v[k] : dv;
          v[k] = on ? 0.0f : v[k];
        }
        if (dout && (unsigned)kd < 8u) g.diag_out[row] = dv;
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) o.s[k] = f32_to_elem<F16>(v[k]);
      if (g.C) *reinterpret_cast<uint4*>(C + (int64_t)row * g.c_rs + col) = o.v;
    }
  }
  if (!DIAG && (passes & 2) && g.C2) {
    unsigned short* C2 = reinterpret_cast<unsigned short*>(g.C2);
#pragma unroll 4
    for (int it = it_begin; it < it_end; ++it) {
      const int idx = it * 64 + lane;
      const int c = idx >> 2, r0 = (idx & 3) * 8;      // column c, rows r0 .. r0+7 of the quarter
      const int col = col_base + c, row = row_base + r0;
      const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(F + qf_idx(c, r0));
      const f32x4_t hi = *reinterpret_cast<const f32x4_t*>(F + qf_idx(c, r0 + 4));
      const float a[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      union { uint4 v; unsigned short s[8]; } o;
#pragma unroll
      for (int k = 0; k < 8; ++k) o.s[k] = f32_to_elem<F16>(a[k]);
      *reinterpret_cast<uint4*>(C2 + (int64_t)col * g.c2_rs + row) = o.v;
    }
  }
}

template <bool F16>
__device__ __forceinline__ void epilogue_quarter(const GemmArgs& g, bool diag, float* F, const unsigned char* Eb,
                                                 const float* RA, int ra_off, int row_base, int col_base,
                                                 int lane, int it_begin, int it_end, int passes) {
  if constexpr (!F16) {   // fp16 problems carry no operand E
    if (g.E) {
      if (diag) epilogue_quarter_t<false, true, true>(g, F, Eb, RA, ra_off, row_base, col_base, lane, it_begin, it_end, passes);
      else epilogue_quarter_t<false, true, false>(g, F, Eb, RA, ra_off, row_base, col_base, lane, it_begin, it_end, passes);
      return;
    }
  }
  if (diag) epilogue_quarter_t<F16, false, true>(g, F, Eb, RA, ra_off, row_base, col_base, lane, it_begin, it_end, passes);
  else epilogue_quarter_t<F16, false, false>(g, F, Eb, RA, ra_off, row_base, col_base, lane, it_begin, it_end, passes);
}

// ---- write-out of a whole tile from the accumulators --------------------------------------------
// An MFMA accumulator register pair of a lane holds two consecutive rows of one column, which is
// what the transposed output wants: after rounding, a lane has 8 bytes of a row of C2 per register
// quadruple.  They are collected column by column in LDS over two quarters (64 rows = 128 bytes per
// column) and leave as whole cache lines, 8 lanes per row of C2.  The direct output needs a real
// transposition, and it stages the same rounded 16-bit values: neighbouring lanes (columns c and
// c+1) exchange halves, so that every lane holds two consecutive columns of one row, and a quarter
// (32 rows x 128 columns) is staged row-major, 8 KiB instead of 16 KiB of fp32, and read back 16
// bytes per lane.  Both copies carry the same bits.
// The operand E is read transposed (ET) in the accumulators' own layout, 8 consecutive rows of one
// column per lane and load, so the arithmetic happens in registers before anything is staged.
constexpr int QT_PITCH = 320;             // bytes per staged row: 128 values + 64 bytes, so that rows r and r+1 use different banks
constexpr int QT_BYTES = 32 * QT_PITCH;   // one staged quarter of a wave
constexpr int QM_PITCH = 136;             // bytes per staged column of the mirrored copy: 64 rows + 8 bytes (2-way conflicts at most)
constexpr int QM_OFFSET = QT_BYTES + 512; // after the direct staging and the 128 row additions
constexpr int QM_BYTES = 128 * QM_PITCH;  // two quarters of the mirrored copy
static_assert(QM_OFFSET + QM_BYTES <= EPI_WAVE_BYTES, "the write-out stages inside the wave's region");

// 16 bytes per lane at base + voff + soff (bytes) through a buffer descriptor: the per-lane part of
// an address is one 32-bit register, the rest is scalar
typedef int v4i_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t block_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0xffffffff, 0x00020000);
}
__device__ __forceinline__ uint4 buf_load16(__amdgpu_buffer_rsrc_t b, uint32_t voff, int soff) {
  const v4i_t v = __builtin_amdgcn_raw_buffer_load_b128(b, (int)voff, soff, 0);
  return uint4{(uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w};
}
__device__ __forceinline__ void buf_store16(__amdgpu_buffer_rsrc_t b, uint32_t voff, int soff, const uint4& d) {
  const v4i_t v = {(int)d.x, (int)d.y, (int)d.z, (int)d.w};
  __builtin_amdgcn_raw_buffer_store_b128(v, b, (int)voff, soff, 0);
}

__device__ __forceinline__ void swap32(uint32_t& lo_half_keeps, uint32_t& hi_half_keeps) {
  // lanes 0..31 give `hi_half_keeps` to, and take `lo_half_keeps` of, the lane 32 above
  const auto r = __builtin_amdgcn_permlane32_swap(lo_half_keeps, hi_half_keeps, false, false);
  lo_half_keeps = r[0];
  hi_half_keeps = r[1];
}

// two values rounded to the element type, `lo` in the low half
template <bool F16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {lo, hi};
  if constexpr (F16) {
    typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, h2_t));
  } else {
    typedef __bf16 b2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, b2_t));
  }
}

// MODE: 0 without the operand E, 1 with it and beta == 1 (the product is added as it is), 2 with it
// and any beta.  A kernel holds one instance only: of identical element reads in several branches
// the optimizer makes one read of all 256 accumulators ahead of the branch, and they do not fit
// into the vector registers.
// The wave's block is 32 NI rows x 128 columns at (row0, col0).  `diag`: the block has no mirror
// image to write (it lies in a diagonal tile of a symmetric product, which holds both); `dshift`:
// MFMA tile (i, i + dshift) of the block lies on the diagonal of the output, or a value no tile has.
// KIND 1 and 2: the block is a 128x128 square on the diagonal of a symmetric product, of which the
// wave holds some MFMA tiles on or below the diagonal (1: all but (1, 0), at
// acc[tri_r(i, j)][tri_c(i, j)]; 2: (1, 0) alone, at acc[2][0]).  Those are written in place, and
// the ones below the diagonal also as their mirror images above it.
__host__ __device__ constexpr bool epi_has(int kind, int i, int j) {
  return kind == 0 ? true : kind == 1 ? (j <= i && !(i == 1 && j == 0)) : (i == 1 && j == 0);
}
__host__ __device__ constexpr bool epi_row_has(int kind, int i) {
  return i >= 0 && (epi_has(kind, i, 0) || epi_has(kind, i, 1) || epi_has(kind, i, 2) || epi_has(kind, i, 3));
}
__host__ __device__ constexpr bool epi_mirrors(int kind, int i, int j) {   // tile (i, j) has a mirror image to write
  return kind == 0 ? true : (i >= 0 && j < i && epi_has(kind, i, j));
}

template <bool F16, int MODE, int NI, int KIND, int NR>
__device__ __forceinline__ void epilogue_regs(const GemmArgs& g, bool diag, int dshift,
                                              const f32x16_t (&acc)[NR][4], unsigned char* T, int row0, int col0,
                                              int lane) {
  constexpr bool TRI = KIND != 0;
  constexpr int NQ = KIND == 0 ? NI : KIND == 1 ? 4 : 2;   // quarters: rows of MFMA tiles
  // what follows is derived from `lane` anew for every tile: kept in registers across the main
  // loop instead, the per-lane offsets of the write-out would crowd out the loop's own
  asm volatile("" : "+v"(lane));
  constexpr bool has_e = !F16 && MODE != 0;
  const int lc = lane & 31, lh = lane >> 5, par = lane & 1;
  const bool direct = g.C != nullptr;
  const bool mirror = g.C2 != nullptr && !diag;
  const bool dout = (KIND == 1 || (KIND == 0 && diag)) && g.diag_out != nullptr;
  const float alpha = g.alpha, beta = g.beta;
  const uint32_t sel = par ? 0x03020706u : 0x05040100u;   // odd lanes keep the high halves, even lanes the low ones
  float* const RA = reinterpret_cast<float*>(T + QT_BYTES);
  // staging: this lane writes row 8qq + 4lh + 2h + par, columns 32j + (lc & ~1) .. +1, and reads
  // row 4it + lane/16, columns 8(lane % 16) .. +7
  unsigned char* const tw = T + (4 * lh + par) * QT_PITCH + (lc & ~1) * 2;
  const unsigned char* const tr = T + (lane >> 4) * QT_PITCH + (lane & 15) * 16;
  // Global accesses go through buffer descriptors based at the wave's block, so that an address is
  // one of three per-lane byte offsets plus a scalar offset:
  // rows 32i + 16t + 8lh .. +7 of column 32j + lc are what a lane loads of ET and stores to C2,
  // row 4it + lane/16, columns 8(lane % 16) .. +7 what it stores to C.
  const uint32_t et_lane = (uint32_t)(lc * (int)g.ldet + 8 * lh) * 2u;
  // rows 64h + 8(lane % 8) .. +7 of column 8it + lane/8: the mirrored copy, a cache line per 8 lanes
  const uint32_t c2_lane = (uint32_t)((lane >> 3) * (int)g.c2_rs + (lane & 7) * 8) * 2u;
  unsigned char* const mw = T + QM_OFFSET + lc * QM_PITCH + 8 * lh;
  const unsigned char* const mr = T + QM_OFFSET + (lane >> 3) * QM_PITCH + (lane & 7) * 16;
  const uint32_t c_lane = (uint32_t)((lane >> 4) * (int)g.c_rs + (lane & 15) * 8) * 2u;
  const __amdgpu_buffer_rsrc_t et_buf = block_rsrc(g.ET + (int64_t)col0 * g.ldet + row0);
  const __amdgpu_buffer_rsrc_t c2_buf = block_rsrc(g.C2 + (int64_t)col0 * g.c2_rs + row0);
  const __amdgpu_buffer_rsrc_t c_buf = block_rsrc(g.C + (int64_t)row0 * g.c_rs + col0);
  const int et_col = 64 * (int)g.ldet, c2_col = 16 * (int)g.c2_rs, c_row = 8 * (int)g.c_rs;   // bytes: 32 columns, 8 columns, 4 rows
#define FM_ET(i, j, t) buf_load16(et_buf, et_lane, (j) * et_col + 64 * (i) + 32 * (t))

  uint4 ev[4][2];
  if constexpr (has_e) {
    // the block's 32 NI additions to alpha (zeros when there are none), before any store of this tile
    float2 ra = {0.0f, 0.0f};
    if (NQ == 4 || lane < 16 * NQ) {
      if (g.row_alpha) ra = *reinterpret_cast<const float2*>(g.row_alpha + row0 + lane * 2);
      *reinterpret_cast<float2*>(RA + lane * 2) = ra;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int t = 0; t < 2; ++t)
        if (epi_has(KIND, 0, j)) ev[j][t] = FM_ET(0, j, t);
  }

#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    f32x4_t al[4];
    if constexpr (has_e) {
#pragma unroll
      for (int qq = 0; qq < 4; ++qq) {
        al[qq] = *reinterpret_cast<const f32x4_t*>(RA + 32 * i + 8 * qq + 4 * lh);
#pragma unroll
        for (int e = 0; e < 4; ++e) al[qq][e] += alpha;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (!epi_has(KIND, i, j)) continue;
      // the scheduler works on one MFMA tile at a time: left alone with the whole unrolled
      // write-out, it moves every accumulator to a vector register first and runs out of them
      __builtin_amdgcn_sched_barrier(0);
      // DOUT: the fp32 diagonal is split off and stored as zero.  A variant of the whole body, not
      // a branch inside it, which would make the sixteen values a merge of two vectors.
      auto tile = [&](auto dout_tag) {
      constexpr bool DOUT = decltype(dout_tag)::value;
      float v[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) v[r] = acc[KIND == 0 ? i : KIND == 1 ? tri_r(i, j) : 2][KIND == 0 ? j : KIND == 1 ? tri_c(i, j) : 0][r];
      if constexpr (has_e) {
        uint32_t eb[4][2];   // [qq][h]: the operand in the accumulators' layout
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          uint32_t a0 = ev[j][t].x, a1 = ev[j][t].y, b0 = ev[j][t].z, b1 = ev[j][t].w;
          swap32(a0, b0);
          swap32(a1, b1);
          eb[2 * t][0] = a0; eb[2 * t][1] = a1; eb[2 * t + 1][0] = b0; eb[2 * t + 1][1] = b1;
          if (i < NQ - 1 && epi_has(KIND, i + 1, j)) ev[j][t] = FM_ET(i + 1, j, t);
        }
        if constexpr (MODE == 2) {
#pragma unroll
          for (int r = 0; r < 16; ++r) v[r] *= beta;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const uint32_t w = eb[r >> 2][(r >> 1) & 1];
          const float ef = elem_to_f32<F16>((unsigned short)((r & 1) ? (w >> 16) : (w & 0xffffu)));
          v[r] = __builtin_fmaf(al[r >> 2][r & 3], ef, v[r]);
        }
      }
      if constexpr (DOUT) {
        float dv = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const bool on = lc == 8 * (r >> 2) + 4 * lh + (r & 3);
          dv = on ? v[r] : dv;
          v[r] = on ? 0.0f : v[r];
        }
        if (lh == ((lc >> 2) & 1)) g.diag_out[row0 + 32 * i + lc] = dv;
      }
      uint32_t P[4][2];   // [qq][h]: rows 8qq + 4lh + 2h, +1 of column 32j + lc, rounded
#pragma unroll
      for (int qq = 0; qq < 4; ++qq)
#pragma unroll
        for (int h = 0; h < 2; ++h) P[qq][h] = pack2<F16>(v[4 * qq + 2 * h], v[4 * qq + 2 * h + 1]);
      if (direct) {   // stage the column of the quarter for the direct output
#pragma unroll
        for (int qq = 0; qq < 4; ++qq)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const uint32_t own = P[qq][h];
            const uint32_t nbr = __builtin_amdgcn_update_dpp(0u, own, 0xB1, 0xF, 0xF, true);   // lane ^ 1
            *reinterpret_cast<uint32_t*>(tw + (8 * qq + 2 * h) * QT_PITCH + 64 * j) = __builtin_amdgcn_perm(nbr, own, sel);
          }
      }
      if (mirror && epi_mirrors(KIND, i, j)) {   // rows 32(i % 2) + 8qq + 4lh .. +3 of column 32j + lc, for the pass after every second quarter
#pragma unroll
        for (int qq = 0; qq < 4; ++qq)
          *reinterpret_cast<uint2*>(mw + 32 * j * QM_PITCH + 64 * (i & 1) + 16 * qq) = uint2{P[qq][0], P[qq][1]};
      }
      };
      if (dout && j == i + dshift) tile(std::true_type{});
      else tile(std::false_type{});
    }
    __builtin_amdgcn_sched_barrier(0);
    // Every load of the tile has arrived long ago.  Said once in a form the compiler's bookkeeping
    // of outstanding loads understands: it does not see the waits written in assembly, takes some
    // load for pending when the next tile begins, and waits for everything in flight in the middle
    // of the main loop.
    if constexpr (has_e) {
      if (i == NQ - 1) __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
      if constexpr (TRI) {   // the tiles the next quarter has and this one had not
        if (i < NQ - 1) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int t = 0; t < 2; ++t)
              if (epi_has(KIND, i + 1, j) && !epi_has(KIND, i, j)) ev[j][t] = FM_ET(i + 1, j, t);
        }
      }
    }

    if (direct && epi_row_has(KIND, i)) {
      // the quarter's columns 32j .. +31 are there when the wave holds tile (i, j)
      const int cols_there = (epi_has(KIND, i, 0) ? 1 : 0) | (epi_has(KIND, i, 1) ? 2 : 0) |
                                 (epi_has(KIND, i, 2) ? 4 : 0) | (epi_has(KIND, i, 3) ? 8 : 0);
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        uint4 d[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) d[it] = *reinterpret_cast<const uint4*>(tr + 4 * (4 * half + it) * QT_PITCH);
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          if (!TRI || ((cols_there >> ((lane & 15) >> 2)) & 1)) buf_store16(c_buf, c_lane, (8 * i + 4 * half + it) * c_row, d[it]);
        }
      }
    }
    if (mirror && (i & 1)) {   // two quarters of the mirrored copy: 128 columns x 128 bytes
#pragma unroll
      for (int grp = 0; grp < 4; ++grp) {   // columns 32 grp .. +31: tiles (i - 1, grp) and (i, grp)
        if (!epi_mirrors(KIND, i - 1, grp) && !epi_mirrors(KIND, i, grp)) continue;
        uint2 d[4][2];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const unsigned char* src = mr + 8 * (4 * grp + it) * QM_PITCH;
          d[it][0] = *reinterpret_cast<const uint2*>(src);
          d[it][1] = *reinterpret_cast<const uint2*>(src + 8);
        }
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          // a lane's 8 rows lie in quarter i - 1 or i
          if (!TRI || ((lane & 7) < 4 ? epi_mirrors(KIND, i - 1, grp) : epi_mirrors(KIND, i, grp)))
            buf_store16(c2_buf, c2_lane, (4 * grp + it) * c2_col + 128 * (i >> 1),
                        uint4{d[it][0].x, d[it][0].y, d[it][1].x, d[it][1].y});
        }
      }
    }
  }
#undef FM_ET
}

// ---- write-out of a whole tile from the 16x16 accumulator tiles ---------------------------------
// The wave's block is 16 NA rows x 128 columns at (row0, col0); per 32x32 sub-block (I, J) a lane (n =
// lane % 16, g = lane / 16) holds rows 32 I + 8 g + 4 a + r of columns 32 J + 2 n + b in register r of
// tile (2 I + a, 2 J + b).  Rounded pairs (b = 0, 1) are 32-bit words of a row of C: they are staged
// row-major, a quarter (32 rows x 128 columns) at a time, and read back 16 bytes per lane.  Rounded
// pairs of rows are collected column by column over two quarters (64 rows = 128 bytes per column of
// the block) and leave as whole cache lines of C2, 8 lanes per row of it.  The operand E is read
// transposed (ET), 8 consecutive rows of one column per lane and load, which is exactly what the lane
// holds of that column, so the arithmetic happens in registers.  Both copies carry the same bits.
// MODE, diag, dshift: as for epilogue_regs (MFMA tile there = 32x32 sub-block here).
constexpr int QD_PITCH = 256;   // staged row of the direct copy: 128 values; 64-byte groups XOR-swizzled by row / 8
static_assert(32 * QD_PITCH <= QT_BYTES, "the direct staging of the 16x16 write-out fits the region of the other one");

template <bool F16, int MODE, int NA>
__device__ __forceinline__ void epilogue_regs16(const GemmArgs& g, bool diag, int dshift, const f32x4_t (&acc)[NA][8],
                                                unsigned char* T, int row0, int col0, int lane) {
  constexpr int NQ = NA / 2;   // quarters: groups of 32 rows
  // derived from `lane` anew for every tile (see epilogue_regs)
  asm volatile("" : "+v"(lane));
  constexpr bool has_e = !F16 && MODE != 0;
  const int n = lane & 15, grp = lane >> 4;
  const bool direct = g.C != nullptr;
  const bool mirror = g.C2 != nullptr && !diag;
  const bool dout = diag && g.diag_out != nullptr;
  const float alpha = g.alpha, beta = g.beta;
  float* const RA = reinterpret_cast<float*>(T + QT_BYTES);
  // direct staging: this lane writes rows 8 grp + 4 a + r, the 4 bytes of columns 32 J + 2 n .. + 1, at
  // 64-byte group J ^ grp of the row; it reads row 4 it + lane / 16, columns 8 (lane % 16) .. + 7
  unsigned char* const tw = T + (8 * grp) * QD_PITCH + 4 * n;
  const unsigned char* const tr = T + (lane >> 4) * QD_PITCH + (lane & 3) * 16;
  const int rgrp = (lane >> 2) & 3;   // 64-byte group of what it reads, before the swizzle
  // mirrored staging: rows 32 (I % 2) + 8 grp + 4 a .. + 3 of column 32 J + 2 n + b; read as in epilogue_regs
  unsigned char* const mw = T + QM_OFFSET + (2 * n) * QM_PITCH + 16 * grp;
  const unsigned char* const mr = T + QM_OFFSET + (lane >> 3) * QM_PITCH + (lane & 7) * 16;
  const uint32_t et_lane = (uint32_t)((2 * n) * (int)g.ldet + 8 * grp) * 2u;
  const uint32_t c2_lane = (uint32_t)((lane >> 3) * (int)g.c2_rs + (lane & 7) * 8) * 2u;
  const uint32_t c_lane = (uint32_t)((lane >> 4) * (int)g.c_rs + (lane & 15) * 8) * 2u;
  const __amdgpu_buffer_rsrc_t et_buf = block_rsrc(g.ET + (int64_t)col0 * g.ldet + row0);
  const __amdgpu_buffer_rsrc_t c2_buf = block_rsrc(g.C2 + (int64_t)col0 * g.c2_rs + row0);
  const __amdgpu_buffer_rsrc_t c_buf = block_rsrc(g.C + (int64_t)row0 * g.c_rs + col0);
  const int et_col = 2 * (int)g.ldet, c2_col = 16 * (int)g.c2_rs, c_row = 8 * (int)g.c_rs;   // bytes: 1 column, 8 columns, 4 rows
#define FM_ET16(I, J, b) buf_load16(et_buf, et_lane, (32 * (J) + (b)) * et_col + 64 * (I))

  uint4 ev[4][2];
  if constexpr (has_e) {
    // the block's 32 NQ additions to alpha (zeros when there are none), before any store of this tile
    float2 ra = {0.0f, 0.0f};
    if (NQ == 4 || lane < 16 * NQ) {
      if (g.row_alpha) ra = *reinterpret_cast<const float2*>(g.row_alpha + row0 + lane * 2);
      *reinterpret_cast<float2*>(RA + lane * 2) = ra;
    }
#pragma unroll
    for (int J = 0; J < 4; ++J)
#pragma unroll
      for (int b = 0; b < 2; ++b) ev[J][b] = FM_ET16(0, J, b);
  }

#pragma unroll
  for (int I = 0; I < NQ; ++I) {
    f32x4_t al[2];
    if constexpr (has_e) {
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        al[a] = *reinterpret_cast<const f32x4_t*>(RA + 32 * I + 8 * grp + 4 * a);
#pragma unroll
        for (int e = 0; e < 4; ++e) al[a][e] += alpha;
      }
    }
#pragma unroll
    for (int J = 0; J < 4; ++J) {
      // one sub-block at a time (see epilogue_regs)
      __builtin_amdgcn_sched_barrier(0);
      auto block = [&](auto dout_tag) {
        constexpr bool DOUT = decltype(dout_tag)::value;
        float v[2][2][4];   // [a][b][r]
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
          for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 4; ++r) v[a][b][r] = acc[2 * I + a][2 * J + b][r];
        if constexpr (has_e) {
#pragma unroll
          for (int b = 0; b < 2; ++b) {
            const uint32_t w[4] = {ev[J][b].x, ev[J][b].y, ev[J][b].z, ev[J][b].w};   // rows 2 k, 2 k + 1 of the lane's eight
            if (I < NQ - 1) ev[J][b] = FM_ET16(I + 1, J, b);
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const uint32_t ww = w[2 * a + (r >> 1)];
                const float ef = elem_to_f32<F16>((unsigned short)((r & 1) ? (ww >> 16) : (ww & 0xffffu)));
                const float x = MODE == 2 ? beta * v[a][b][r] : v[a][b][r];
                v[a][b][r] = __builtin_fmaf(al[a][r], ef, x);
              }
          }
        }
        if constexpr (DOUT) {
          // row 8 grp + 4 a + r meets column 2 n + b: the lanes with n / 4 == grp hold two elements of the
          // diagonal, rows 2 n and 2 n + 1 of the sub-block; they are split off in fp32 and stored as zero
          float dv[2] = {0.0f, 0.0f};
#pragma unroll
          for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const bool on = 2 * n + b == 8 * grp + 4 * a + r;
                dv[b] = on ? v[a][b][r] : dv[b];
                v[a][b][r] = on ? 0.0f : v[a][b][r];
              }
          if ((n >> 2) == grp) {
            g.diag_out[row0 + 32 * I + 2 * n] = dv[0];
            g.diag_out[row0 + 32 * I + 2 * n + 1] = dv[1];
          }
        }
        if (direct) {
#pragma unroll
          for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int r = 0; r < 4; ++r)
              *reinterpret_cast<uint32_t*>(tw + (4 * a + r) * QD_PITCH + 64 * (J ^ grp)) = pack2<F16>(v[a][0][r], v[a][1][r]);
        }
        if (mirror) {
#pragma unroll
          for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int a = 0; a < 2; ++a)
              *reinterpret_cast<uint2*>(mw + (32 * J + b) * QM_PITCH + 64 * (I & 1) + 8 * a) =
                  uint2{pack2<F16>(v[a][b][0], v[a][b][1]), pack2<F16>(v[a][b][2], v[a][b][3])};
        }
      };
      if (dout && J == I + dshift) block(std::true_type{});
      else block(std::false_type{});
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (has_e) {
      if (I == NQ - 1) __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): see epilogue_regs
    }
    if (direct) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        uint4 d[4];
#pragma unroll
        for (int it = 0; it < 4; ++it)   // rows 4 (4 half + it) + lane / 16: their 64-byte groups are swizzled by 2 half + it / 2
          d[it] = *reinterpret_cast<const uint4*>(tr + 4 * (4 * half + it) * QD_PITCH + 64 * (rgrp ^ (2 * half + (it >> 1))));
#pragma unroll
        for (int it = 0; it < 4; ++it) buf_store16(c_buf, c_lane, (8 * I + 4 * half + it) * c_row, d[it]);
      }
    }
    if (mirror && (I & 1)) {   // two quarters of the mirrored copy: 128 columns x 128 bytes
#pragma unroll
      for (int cg = 0; cg < 4; ++cg) {
        uint2 d[4][2];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const unsigned char* src = mr + 8 * (4 * cg + it) * QM_PITCH;
          d[it][0] = *reinterpret_cast<const uint2*>(src);
          d[it][1] = *reinterpret_cast<const uint2*>(src + 8);
        }
#pragma unroll
        for (int it = 0; it < 4; ++it)
          buf_store16(c2_buf, c2_lane, (4 * cg + it) * c2_col + 128 * (I >> 1),
                      uint4{d[it][0].x, d[it][0].y, d[it][1].x, d[it][1].y});
      }
    }
  }
#undef FM_ET16
}

// The schedule works on items: item i is base part i % ksplit of tile i / ksplit, where every tile's
// k range is cut into `ksplit` equal base parts (1 unless there are too few tiles to fill the chip
// and k is long).  Items [0, rounds * grid) run one per workgroup in `rounds` full rounds; the `rem`
// items left over are cut once more into `split` sub-parts each, one per workgroup, in a last round.
// Anything that is not a whole tile is written to a partial-tile slot: item i of a full round to
// slot i, sub-part q of left-over item j to slot tail_slot0 + j * split + q.
// When whole tiles are left over and there are at most grid / 16 of them, the last round cuts them
// in space instead (sub64): 16 sub-tiles of 64x64 per tile, one per workgroup, each over the whole
// k, so that nothing has to be added up afterwards.
struct FastArgs {
  GemmArgs g;
  float* partials;      // fp32 partial tiles
  int nk;               // k stages per tile
  int grid;             // workgroups launched
  int ksplit;           // base parts per tile
  int rounds;           // full rounds of items
  int rem;              // items of the last, partial round
  int split;            // sub-parts per item of the last round
  int tail_slot0;       // first slot of the last round's sub-parts
  int reduce_tile0;     // first tile the second kernel has to finish
  int sub64;            // the left-over tiles are computed whole-k as 64x64 sub-tiles, 16 workgroups each
  // Sub-tiles handed out in the order the workgroups arrive (below), or nullptr: sub-tile w to workgroup w.
  unsigned long long* tickets;
  unsigned long long epoch;   // this launch's number (48 bits, never 0)
  int half;             // the items are 128x256 half tiles, never cut (the NI == 2 kernels)
};

// k stages [kb, ke) of base part `part` of `parts`, or of its sub-part `sub` of `subs`
// (32-bit arithmetic: nk < 2^15 stages and at most 64 parts; the uncut case costs nothing)
__device__ __forceinline__ void item_range(int nk, int part, int parts, int sub, int subs, int& kb, int& ke) {
  unsigned b0 = 0, b1 = (unsigned)nk;
  if (parts > 1) {
    b0 = (unsigned)nk * (unsigned)part / (unsigned)parts;
    b1 = (unsigned)nk * (unsigned)(part + 1) / (unsigned)parts;
  }
  kb = (int)b0;
  ke = (int)b1;
  if (subs > 1) {
    kb = (int)(b0 + (b1 - b0) * (unsigned)sub / (unsigned)subs);
    ke = (int)(b0 + (b1 - b0) * (unsigned)(sub + 1) / (unsigned)subs);
  }
}

// Position in the schedule -> tile coordinates.  Tiles are visited in 8x8 blocks (row-major over
// the blocks, row-major inside a block; blocks below the diagonal are skipped and blocks on it are
// triangles when the product is symmetric), so the ~32 tiles an XCD works on at any one time touch
// about 8 + 8 operand panels instead of one panel per tile, and its L2 serves most of the copies.
__device__ __forceinline__ void tile_at(const GemmArgs& g, int pos, int& b, int& ti, int& tj) {
  constexpr int SB = 8;
  b = 0;
  if (g.batch > 1) {
    const int per_matrix = g.num_tiles / g.batch;
    b = pos / per_matrix;
    pos -= b * per_matrix;
  }
  // the last `diag_last` diagonal tiles of a symmetric product stand at the end of the order
  const int d0 = g.tiles_m - g.diag_last;   // first of them (tiles_m without any)
  if (g.diag_last > 0 && pos >= g.num_tiles - g.diag_last) {
    ti = tj = d0 + (pos - (g.num_tiles - g.diag_last));
    return;
  }
  const int nbm = (g.tiles_m + SB - 1) / SB, nbn = (g.tiles_n + SB - 1) / SB;
  for (int I = 0; I < nbm; ++I) {
    const int rows = (g.tiles_m - I * SB) < SB ? (g.tiles_m - I * SB) : SB;
    for (int J = g.symmetric ? I : 0; J < nbn; ++J) {
      const int cols = (g.tiles_n - J * SB) < SB ? (g.tiles_n - J * SB) : SB;
      const bool tri = g.symmetric && I == J;
      // diagonal tiles of this block that stand at the end instead
      int gone = 0;
      if (tri && g.diag_last > 0) {
        gone = I * SB + rows - d0;
        gone = gone < 0 ? 0 : gone > rows ? rows : gone;
      }
      const int cnt = tri ? rows * (rows + 1) / 2 - gone : rows * cols;
      if (pos < cnt) {
        int a, b;
        if (!tri) { a = pos / cols; b = pos - a * cols; }
        else if (gone == 0) { tri_decode(pos, rows, a, b); }
        else {   // row a of the triangle holds rows - a tiles, one fewer without its diagonal tile
          for (a = 0; a < rows - 1; ++a) {
            const int in_row = rows - a - (I * SB + a >= d0 ? 1 : 0);
            if (pos < in_row) break;
            pos -= in_row;
          }
          b = a + pos + (I * SB + a >= d0 ? 1 : 0);
        }
        ti = I * SB + a;
        tj = J * SB + b;
        return;
      }
      pos -= cnt;
    }
  }
  ti = tj = 0;   // not reached for pos < num_tiles
}

// Position in the half-tile schedule -> tile and half.  A product that is not symmetric has two
// items per tile, the upper (h = 0) and the lower 128 rows.  A symmetric one has its diagonal tiles
// as one item each (`whole_diag`), so a matrix of T x T tiles makes T (T - 1) + T = T^2 items; the
// order is that of tile_at, the two halves of a tile next to each other.
__device__ __forceinline__ void half_item_at(const GemmArgs& g, int e, int& b, int& ti, int& tj, int& h, bool& whole_diag) {
  whole_diag = false;
  if (!g.symmetric) {
    h = e & 1;
    tile_at(g, e >> 1, b, ti, tj);
    return;
  }
  constexpr int SB = 8;
  b = 0;
  if (g.batch > 1) {
    const int per_matrix = g.tiles_m * g.tiles_m;
    b = e / per_matrix;
    e -= b * per_matrix;
  }
  const int nb = (g.tiles_m + SB - 1) / SB;
  for (int I = 0; I < nb; ++I) {
    const int rows = (g.tiles_m - I * SB) < SB ? (g.tiles_m - I * SB) : SB;
    for (int J = I; J < nb; ++J) {
      const int cols = (g.tiles_m - J * SB) < SB ? (g.tiles_m - J * SB) : SB;
      const int cnt = I == J ? rows * rows : 2 * rows * cols;
      if (e < cnt) {
        if (I == J) {
          int a = 0;
          for (; a < rows - 1; ++a) {            // row a of the triangle: its diagonal tile, then 2 (rows - 1 - a) halves
            const int in_row = 2 * (rows - a) - 1;
            if (e < in_row) break;
            e -= in_row;
          }
          ti = I * SB + a;
          whole_diag = e == 0;
          tj = whole_diag ? ti : ti + 1 + ((e - 1) >> 1);
          h = whole_diag ? 0 : (e - 1) & 1;
        } else {
          const int t = e >> 1, a = t / cols;
          h = e & 1;
          ti = I * SB + a;
          tj = J * SB + (t - a * cols);
        }
        return;
      }
      e -= cnt;
    }
  }
  ti = tj = h = 0;   // not reached for e < the number of items
}

// The k loop of a diagonal item for one kind of wave; the copies of the first two stages are in
// flight and stage 0 has landed everywhere.
template <bool F16, bool TRI>
__device__ __forceinline__ void diag_item_loop(f32x16_t (&acc)[3][4], const unsigned char* smem, const DFragAddr& dfa,
                                               const uint32_t (&vo)[8], const bf16_t* gP, int n, uint32_t ldsw) {
  const int last = n - 1;
  DFrag f0, f1;
#pragma unroll
  for (int q = 0; q < (TRI ? 4 : 8); ++q) f0.f[q] = read_d<0>(smem, dfa, q, 0);
  // stages past the end are the last stage again (into slots nobody reads), so that the number of
  // copies in flight is the same at every wait
#define FM_DSTAGE(AS, S, FIRST)                                                                \
  {                                                                                            \
    const int kn = (S) + 2 < last ? (S) + 2 : last;                                            \
    dstage<F16, TRI, AS, FIRST>(acc, f0, f1, smem, dfa, vo, gP + kn * BKF, ldsw);              \
  }
  FM_DSTAGE(0, 0, true)
  int s = 1;
  for (; s + 3 <= n; s += 3) {
    FM_DSTAGE(1, s, false)
    FM_DSTAGE(2, s + 1, false)
    FM_DSTAGE(0, s + 2, false)
  }
  if (s < n) {
    FM_DSTAGE(1, s, false)
    if (s + 1 < n) FM_DSTAGE(2, s + 1, false)
  }
#undef FM_DSTAGE
  wait_vmcnt<0>();
  __syncthreads();   // no copy in flight and no wave still reading: LDS is free again
}

// A diagonal tile (at m0 on the diagonal) of a symmetric product, over n k stages from gP on.
template <bool F16, int MODE>
__device__ __forceinline__ void diag_item(const GemmArgs& g, int m0, int n, unsigned char* smem, const uint32_t (&vo)[8],
                                          const bf16_t* gP, uint32_t ldsw, int lane, int wave) {
  const bool tri = wave < 2;
  DFragAddr dfa;
  int dlane = lane;   // derived anew for every such item instead of being kept across the others
  asm volatile("" : "+v"(dlane));
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    // waves 2 and 3: rows 64 (wave - 2) + 32q, columns 128 + 32 (q - 2), and rows 32 .. 63 and 0 .. 31 of square wave - 2
    const int r0 = tri ? 128 * wave + 32 * (q & 3)
                       : (q < 2 ? 64 * (wave - 2) + 32 * q : q < 6 ? 128 + 32 * (q - 2) : 128 * (wave - 2) + 32 * (7 - q));
    const int r = r0 + (dlane & 31);
    const uint32_t o = (uint32_t)(r * ROWB + (((dlane >> 5) ^ swz(r)) << 4));
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      dfa.lo[q][ks] = o ^ (ks << 5);
      dfa.hi[q][ks] = (o ^ (ks << 5)) + a_slot_off(2);
    }
  }
  const int k1 = n - 1 < 1 ? n - 1 : 1;
#pragma unroll
  for (int q = 0; q < 8; ++q) dma16o(vo[q], gP, ldsw, a_slot_off(0) + q * 4096);
#pragma unroll
  for (int q = 0; q < 8; ++q) dma16o(vo[q], gP + k1 * BKF, ldsw, a_slot_off(1) + q * 4096);
  wait_vmcnt<8>();
  __syncthreads();
  unsigned char* const wave_lds = smem + wave * EPI_WAVE_BYTES;
  // (each kind of wave has accumulators of its own, pinned to their registers before the write-out)
  if (tri) {
    f32x16_t acc[3][4];
    diag_item_loop<F16, true>(acc, smem, dfa, vo, gP, n, ldsw);
#pragma unroll
    for (int q = 0; q < 9; ++q) asm volatile("" : "+a"(acc[tri_r(tri_i(q), tri_j(q))][tri_c(tri_i(q), tri_j(q))]));
    const int sq = m0 + 128 * wave;
    epilogue_regs<F16, MODE, 2, 1>(g, false, 0, acc, wave_lds, sq, sq, lane);
  } else {
    f32x16_t acc[3][4];
    diag_item_loop<F16, false>(acc, smem, dfa, vo, gP, n, ldsw);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) asm volatile("" : "+a"(acc[i][j]));
    asm volatile("" : "+a"(acc[2][0]));
    // 64 rows of the square above the diagonal, then tile (1, 0) of the first or second square on it
    epilogue_regs<F16, MODE, 2, 0>(g, false, 0, acc, wave_lds, m0 + 64 * (wave - 2), m0 + 128, lane);
    const int sq = m0 + 128 * (wave - 2);
    epilogue_regs<F16, MODE, 2, 2>(g, false, 0, acc, wave_lds, sq, sq, lane);
  }
}

// ---- 64x64 sub-tiles of the tiles left over after the last full round ---------------------------
// One workgroup per sub-tile, four waves of 32x32 (2 x 2 accumulator tiles of the 16x16x32 MFMA), the
// whole k range, so the result needs no second pass and is summed in the same k order as a whole tile.
// A sub-tile moves four times the operand bytes per flop of a 256x256 tile and is bound by the copy
// path (16 KiB per stage against 8 MFMAs per wave), hence a deep ring: 8 stages of 16 KiB, 7 in
// flight.  The fragment reads of a stage are issued a stage ahead, behind the barrier that says it
// has landed everywhere, and ride on the MFMAs of the stage before: wait, barrier, reads and MFMAs one
// after the other cost 510 cycles a stage where the MFMAs take 128.
// Tickets for the sub-tiles of one launch: a 64-bit word in the caller's workspace holds the launch's
// number in its upper 48 bits and the count of tickets drawn in the lower 16.  Launch numbers grow, so
// an atomic maximum with (number, 0), which every workgroup applies when it starts, turns whatever an
// earlier launch left there into "none drawn" and leaves the word alone once this launch counts in it;
// nothing has to be cleared beforehand.  What the maximum returns tells the workgroup whether there
// are tickets: if the word held something beyond this launch's numbers (never cleared, or written by
// something else) it stays as it is, nobody ever draws, and sub-tile w goes to workgroup w; every
// workgroup sees the same.  A draw is one atomic add.  `total` tickets are drawn in all (one per
// sub-tile, and one more per workgroup, that tells it to stop); whoever draws the last one leaves the
// word at zero, so that a replay of the same launch from a HIP graph finds it below its number again.
constexpr int kNoTickets = -1;
__device__ __forceinline__ bool open_tickets(unsigned long long* word, unsigned long long epoch) {
  const unsigned long long old = __hip_atomic_fetch_max(word, epoch << 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return old < ((epoch + 1) << 16);
}
__device__ __forceinline__ int draw_ticket(unsigned long long* word, unsigned long long epoch, int total) {
  const unsigned long long old = __hip_atomic_fetch_add(word, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if ((old >> 16) != epoch) return kNoTickets;   // (not reached: the word was opened for this launch)
  const int ticket = (int)(old & 0xffffull);
  if (ticket == total - 1) __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return ticket;
}

constexpr int SUB = 64;
constexpr int SUB_OPER = SUB * ROWB;          // 64 rows of one operand stage: 8 KiB
constexpr int SUB_STAGE = 2 * SUB_OPER;
constexpr int SUB_DEPTH = 8;
constexpr int SUB_F_PITCH = 36;               // floats per staged column: 32 rows + 4 of padding

template <bool F16>
__device__ __forceinline__ void sub64_tile(const GemmArgs& g, int ti, int tj, int si, int sj, int nk,
                                           unsigned char* smem, int lane, int wave) {
  const bool tdiag = g.symmetric && ti == tj;
  if (tdiag && si > sj) return;               // the mirror image of sub-tile (sj, si) of the same tile
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = ti * BM + si * SUB, n0 = tj * BN + sj * SUB;

  // copy q of this wave fills LDS rows wave*16 + q*8 .. +8 of an operand stage
  uint32_t voA[2], voB[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int row = wave * 16 + q * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ swz(row);
    voA[q] = (uint32_t)(row * (int)g.lda + chunk * 8) * 2u;
    voB[q] = (uint32_t)(row * (int)g.ldb + chunk * 8) * 2u;
  }
  const bf16_t* gA = g.A + (int64_t)m0 * g.lda;
  const bf16_t* gB = g.B + (int64_t)n0 * g.ldb;
  const uint32_t ldsw = FM_LDS_ADDR(smem) + wave * 2048;
  auto issue = [&](int stage, int slot) {   // 4 copies per wave
    const uint32_t base = ldsw + slot * SUB_STAGE;
#pragma unroll
    for (int q = 0; q < 2; ++q) dma16(voA[q], gA + stage * BKF, base + q * 1024);
#pragma unroll
    for (int q = 0; q < 2; ++q) dma16(voB[q], gB + stage * BKF, base + SUB_OPER + q * 1024);
  };
  // per-lane fragment addresses inside a stage: [fragment of 16 rows][k32 substep]
  uint32_t ao[2][2], bo[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int ra = wm * 32 + 16 * i + (lane & 15), rb = wn * 32 + 16 * i + (lane & 15);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      ao[i][kk] = (uint32_t)(ra * ROWB + (((4 * kk + (lane >> 4)) ^ swz(ra)) << 4));
      bo[i][kk] = (uint32_t)(SUB_OPER + rb * ROWB + (((4 * kk + (lane >> 4)) ^ swz(rb)) << 4));
    }
  }
  struct SubFrag { bf16x8_t a[2][2], b[2][2]; };   // [fragment][substep]
  auto read_frag = [&](SubFrag& f, const unsigned char* st, int t) {   // read t of a stage's eight: substep t / 4, a0 b0 a1 b1
    const int kk = t >> 2, i = (t >> 1) & 1;
    if (t & 1) f.b[i][kk] = *reinterpret_cast<const bf16x8_t*>(st + bo[i][kk]);
    else f.a[i][kk] = *reinterpret_cast<const bf16x8_t*>(st + ao[i][kk]);
  };

  f32x4_t acc[2][2];
  // stages past the end are the last stage again (into slots nobody reads), so that the number of
  // copies in flight is the same at every wait
#pragma unroll
  for (int s = 0; s < SUB_DEPTH - 1; ++s) issue(s < nk ? s : nk - 1, s);
  wait_vmcnt<4 * (SUB_DEPTH - 2)>();   // stage 0 has landed
  __syncthreads();
  SubFrag f0, f1;
#pragma unroll
  for (int t = 0; t < 8; ++t) read_frag(f0, smem, t);
  // One iteration: my copies of stage s + 1 have landed, and behind the barrier everybody's, while
  // nobody reads stage s - 1 any more (its fragments were multiplied before the barrier), so its slot
  // takes the copies of stage s + 7; the fragments of stage s + 1 are asked for while those of stage
  // s, read an iteration ago, are multiplied.  (A bare barrier: the reads asked for an iteration ago
  // may still be on their way, their slot is not refilled before they have been multiplied;
  // __syncthreads() would wait for them here.)
  auto iter = [&](int s, const SubFrag& cur, SubFrag& nxt, auto first_tag) {
    constexpr bool FIRST = decltype(first_tag)::value;
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(4 * (SUB_DEPTH - 3)) : "memory");
    const int nx = s + SUB_DEPTH - 1;
    const int nstage = nx < nk ? nx : nk - 1;
    const uint32_t nbase = ldsw + (nx & (SUB_DEPTH - 1)) * SUB_STAGE;
    const unsigned char* st = smem + ((s + 1) & (SUB_DEPTH - 1)) * SUB_STAGE;
#pragma unroll
    for (int q = 0; q < 8; ++q) {   // MFMA q: substep q / 4, tile (q / 2 % 2, q % 2)
      if (q < 2) dma16(voA[q], gA + nstage * BKF, nbase + q * 1024);
      else if (q < 4) dma16(voB[q - 2], gB + nstage * BKF, nbase + SUB_OPER + (q - 2) * 1024);
      read_frag(nxt, st, q);
      const int kk = q >> 2, i = (q >> 1) & 1, j = q & 1;
      if constexpr (FIRST) {
        if (kk == 0) acc[i][j] = mfma_16x16x32<F16>(cur.a[i][kk], cur.b[j][kk], f32x4_t{0.0f, 0.0f, 0.0f, 0.0f});
        else acc[i][j] = mfma_16x16x32<F16>(cur.a[i][kk], cur.b[j][kk], acc[i][j]);
      } else {
        acc[i][j] = mfma_16x16x32<F16>(cur.a[i][kk], cur.b[j][kk], acc[i][j]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  iter(0, f0, f1, std::true_type{});
  int s = 1;
  for (; s + 2 <= nk; s += 2) {
    iter(s, f1, f0, std::false_type{});
    iter(s + 1, f0, f1, std::false_type{});
  }
  if (s < nk) iter(s, f1, f0, std::false_type{});
  wait_vmcnt<0>();
  __syncthreads();   // no copy in flight and no wave still reading: the ring is free

  // accumulators -> a wave-private staging block (column-major, 32 columns of 32 rows), then out:
  // the direct pass writes 1 row x 16 columns per lane and puts the rounded values back, the
  // transposed pass 16 rows x 1 column per lane, so both copies carry the same bits
  float* const F = reinterpret_cast<float*>(smem + wave * (32 * SUB_F_PITCH * 4));
  {   // register r of tile (i, j) of lane l is row 16 i + 4 (l / 16) + r, column 16 j + l % 16 of the block
    const int c = lane & 15, rg = 4 * (lane >> 4);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) *reinterpret_cast<f32x4_t*>(F + (16 * j + c) * SUB_F_PITCH + 16 * i + rg) = acc[i][j];
  }
  const int row0 = m0 + wm * 32, col0 = n0 + wn * 32;
  // a block of a diagonal sub-tile holds its own mirror image (or is one of a pair of blocks that
  // hold each other's, bit for bit): such a sub-tile is written once, by the direct pass
  const bool bdiag = tdiag && si == sj;
  const bool use_e = !F16 && g.E != nullptr;
  const bool mirror = !bdiag && g.C2 != nullptr;
  {
    const int r = lane >> 1, c0 = (lane & 1) * 16;
    const int row = row0 + r, col = col0 + c0;
    float v[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) v[k] = F[(c0 + k) * SUB_F_PITCH + r];
    if (use_e) {
      union { uint4 q[2]; unsigned short h[16]; } e;
      const uint4* src = reinterpret_cast<const uint4*>(g.E + (int64_t)row * g.lde + col);
      e.q[0] = src[0];
      e.q[1] = src[1];
      const float al = g.row_alpha ? g.alpha + g.row_alpha[row] : g.alpha;
#pragma unroll
      for (int k = 0; k < 16; ++k) v[k] = __builtin_fmaf(al, elem_to_f32<F16>(e.h[k]), g.beta * v[k]);
    }
    if (bdiag && wm == wn && g.diag_out != nullptr) {   // this block lies on the diagonal of the product
      const int kd = r - c0;                            // the diagonal element of this row, if 0..15
      float dv = 0.0f;
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const bool on = kd == k;
        dv = on ? v[k] : dv;
        v[k] = on ? 0.0f : v[k];
      }
      if ((unsigned)kd < 16u) g.diag_out[row] = dv;
    }
    union { uint4 q[2]; unsigned short h[16]; } o;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      o.h[k] = f32_to_elem<F16>(v[k]);
      if (mirror) F[(c0 + k) * SUB_F_PITCH + r] = elem_to_f32<F16>(o.h[k]);
    }
    if (g.C) {
      uint4* dst = reinterpret_cast<uint4*>(reinterpret_cast<unsigned short*>(g.C) + (int64_t)row * g.c_rs + col);
      dst[0] = o.q[0];
      dst[1] = o.q[1];
    }
  }
  if (mirror) {
    const int c = lane >> 1, r0 = (lane & 1) * 16;
    union { uint4 q[2]; unsigned short h[16]; } o;
#pragma unroll
    for (int k = 0; k < 16; ++k) o.h[k] = f32_to_elem<F16>(F[c * SUB_F_PITCH + r0 + k]);
    uint4* dst = reinterpret_cast<uint4*>(reinterpret_cast<unsigned short*>(g.C2) + (int64_t)(col0 + c) * g.c2_rs + row0 + r0);
    dst[0] = o.q[0];
    dst[1] = o.q[1];
  }
}

// accumulators of the 32-row group I of a wave's 128x128 block (16x16 tiles) -> F, as stage_store
template <int I>
__device__ __forceinline__ void stage_store16(const f32x4_t (&acc)[8][8], float* F, int lane) {
  const int n = lane & 15, grp = lane >> 4;
#pragma unroll
  for (int J = 0; J < 4; ++J)
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int col = 32 * J + 2 * n + b;
      float* const dst = F + col * QF_PITCH;
      const int x = ((col >> 3) & 7) << 2;
#pragma unroll
      for (int a = 0; a < 2; ++a) *reinterpret_cast<f32x4_t*>(dst + ((8 * grp + 4 * a) ^ x)) = acc[2 * I + a][2 * J + b];
    }
}

// A whole 256x256 tile (NA == 8; or a part of one along k) or a 128x256 half tile (NA == 4): n k stages
// from (gA, gB) on through the operand ring on 16x16x32 MFMAs, then the write-out, or (whole tiles) the
// hand-over of the fp32 sums to `slot`.
template <bool F16, int MODE, int NA>
__device__ __forceinline__ void whole_tile16(const GemmArgs& g, bool diag, int n, float* slot, unsigned char* smem,
                                             const FragAddr16& fa, const uint32_t (&voA)[NA], const uint32_t (&voB)[8],
                                             const bf16_t* gA, const bf16_t* gB, uint32_t ldsw, int row0, int col0,
                                             int lane, int wave, unsigned long long* draw, unsigned long long epoch, int total,
                                             int& ticket) {
  f32x4_t acc[NA][8];
  {
    Frag16<NA> f0, f1;
    // stages past the end are the last stage again (into slots nobody reads), so that the number
    // of copies in flight is the same at every wait
    const int last = n - 1;
    const int k1 = last < 1 ? last : 1;
#pragma unroll
    for (int q = 0; q < NA; ++q) dma16o(voA[q], gA, ldsw, a_slot_off(0) + q * 4096);
#pragma unroll
    for (int q = 0; q < 8; ++q) dma16o(voB[q], gB, ldsw, b_slot_off(0) + q * 4096);
#pragma unroll
    for (int q = 0; q < NA; ++q) dma16o(voA[q], gA + k1 * BKF, ldsw, a_slot_off(1) + q * 4096);
#pragma unroll
    for (int q = 0; q < 8; ++q) dma16o(voB[q], gB + k1 * BKF, ldsw, b_slot_off(1) + q * 4096);
    wait_vmcnt<NA + 8>();
    __syncthreads();
#pragma unroll
    for (int q = 0; q < NA; ++q) f0.a[q] = read_a16<0>(smem, fa, q, 0);
#pragma unroll
    for (int q = 0; q < 8; ++q) f0.b[q] = read_b16<0>(smem, fa, q, 0);
    // The slots come round every 6 stages.
#define FM_STAGE_T(AS, BS, S, FIRST)                                                             \
    {                                                                                            \
      const int kn = (S) + 2 < last ? (S) + 2 : last;                                            \
      stage16<F16, NA, AS, BS, FIRST>(acc, f0, f1, smem, fa, voA, voB, gA + kn * BKF, gB + kn * BKF, ldsw);  \
    }
#define FM_STAGE(AS, BS, S) FM_STAGE_T(AS, BS, S, false)
    if constexpr (MODE == 0) {
      // the first stage stands apart: its first MFMAs start the sums from zero
      FM_STAGE_T(0, 0, 0, true)
      int s = 1;
      for (; s + 6 <= n; s += 6) {
        FM_STAGE(1, 1, s)
        FM_STAGE(2, 0, s + 1)
        FM_STAGE(0, 1, s + 2)
        FM_STAGE(1, 0, s + 3)
        FM_STAGE(2, 1, s + 4)
        FM_STAGE(0, 0, s + 5)
      }
      if (s < n) {
        FM_STAGE(1, 1, s)
        if (s + 1 < n) {
          FM_STAGE(2, 0, s + 1)
          if (s + 2 < n) {
            FM_STAGE(0, 1, s + 2)
            if (s + 3 < n) {
              FM_STAGE(1, 0, s + 3)
              if (s + 4 < n) FM_STAGE(2, 1, s + 4)
            }
          }
        }
      }
    } else {
      // With an operand E the write-out needs more registers, and the loop above in its three pieces
      // (first stage, six stages, last stages) comes out with the sums in other registers in each piece
      // and 800 to 1700 register moves where the pieces meet, by way of vector registers since no
      // accumulation register is free.  So here one loop holds every stage, left wherever the tile's
      // stages end, and the sums are cleared beforehand, by the matrix unit (0 * 0 + 0: a quarter of the
      // instructions that writing the registers takes), while the first copies are on their way.
      bf16x8_t z = {};
      const f32x4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int i = 0; i < NA; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          asm volatile("" : "+v"(z));   // (or the 8 NA products are one product and 8 NA - 1 copies of it)
          acc[i][j] = mfma_16x16x32<F16>(z, z, zero);
          asm volatile("" : "+a"(acc[i][j]));
        }
      for (int s = 0;; s += 6) {
        FM_STAGE(0, 0, s)
        if (s + 1 >= n) break;
        FM_STAGE(1, 1, s + 1)
        if (s + 2 >= n) break;
        FM_STAGE(2, 0, s + 2)
        if (s + 3 >= n) break;
        FM_STAGE(0, 1, s + 3)
        if (s + 4 >= n) break;
        FM_STAGE(1, 0, s + 4)
        if (s + 5 >= n) break;
        FM_STAGE(2, 1, s + 5)
        if (s + 6 >= n) break;
      }
    }
#undef FM_STAGE_T
#undef FM_STAGE
    wait_vmcnt<0>();
    __syncthreads();   // no copy in flight and no wave still reading: LDS is free again
  }
  // the last whole tile of a workgroup that goes on to sub-tiles: its first ticket is drawn here, so
  // that the answer (a trip to memory and back, 3 us) arrives while the tile is written out
  if (draw && threadIdx.x == 0) ticket = draw_ticket(draw, epoch, total);
  unsigned char* const wave_lds = smem + wave * EPI_WAVE_BYTES;
  if constexpr (NA != 8) {   // half tiles are never cut
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) asm volatile("" : "+a"(acc[i][j]));
    epilogue_regs16<F16, MODE, NA>(g, diag, (row0 - col0) / 32, acc, wave_lds, row0, col0, lane);
  } else if (slot) {   // a part of a tile: fp32, a quarter at a time through LDS, to its slot
    const EpiLds L = epi_lds(wave_lds);
    int sl = lane;   // per-lane offsets derived anew for every tile, not kept across the main loop
    asm volatile("" : "+v"(sl));
#define FM_QUARTER(q)                                                        \
    stage_store16<q>(acc, L.F, sl);                                            \
    copy_stage_to_ws(L.F, slot + (wave * 4 + q) * QUARTER_FLOATS, sl);
    FM_QUARTER(0)
    FM_QUARTER(1)
    FM_QUARTER(2)
    FM_QUARTER(3)
#undef FM_QUARTER
  } else {
    // (the accumulators are pinned to their registers first, on this branch only: see the note on
    // element reads at epilogue_regs)
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) asm volatile("" : "+a"(acc[i][j]));
    epilogue_regs16<F16, MODE, NA>(g, diag, (row0 - col0) / 32, acc, wave_lds, row0, col0, lane);
  }
}

// MODE: how whole tiles are written out (see epilogue_regs); chosen by the host from E and beta
template <bool F16, int MODE, int NI>
__global__ __launch_bounds__(256) void gemm_nt_rounds_kernel(FastArgs p) {
  // the operand ring during the main loop (five slots of 32 KiB: A0 A1 B0 B1 A2), the staging of
  // the four waves' write-out afterwards
  __shared__ __align__(1024) unsigned char smem[SMEM_BYTES];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous block of positions
  // so that the tiles it holds at any one time are neighbours in the blocked tile order.
  int w = (int)blockIdx.x;
  {
    const int chunk = p.grid >> 3;   // the workgroups past the last whole group of 8 keep their place
    if (w < chunk * 8) w = (w & 7) * chunk + (w >> 3);
  }

  const uint32_t ldsw = FM_LDS_ADDR(smem) + wave * 1024;   // where this wave's copies land inside a slot
  bool tickets_live = false;   // thread 0: the sub-tile round of this launch hands out tickets
  if constexpr (NI == 4) {
    if (p.tickets != nullptr && tid == 0) tickets_live = open_tickets(p.tickets, p.epoch);
  }

  // fragment addresses: row = lane % 16 of a fragment's 16 LDS rows, k quarter = lane / 16; the wave's
  // rows of operand A begin at 32 NI wm (128 per wave of a whole tile, 64 of a half tile)
  FragAddr16 fa16;
  {
    const int ra = wm * (32 * NI) + (lane & 15), rb = wn * 128 + (lane & 15);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      fa16.a_lo[kk] = (uint32_t)(ra * ROWB + (((4 * kk + (lane >> 4)) ^ swz16(ra)) << 4));
      fa16.a_hi[kk] = fa16.a_lo[kk] + a_slot_off(2);
      fa16.b[kk] = (uint32_t)(rb * ROWB + (((4 * kk + (lane >> 4)) ^ swz16(rb)) << 4)) + b_slot_off(0);
    }
  }

  int first_ticket = kNoTickets;   // thread 0: the ticket drawn ahead of the sub-tile round
  for (int round = 0; round <= p.rounds; ++round) {
    int item, slot_id, kb, ke;
    if (round < p.rounds) {
      item = round * p.grid + w;
      slot_id = item;
      item_range(p.nk, p.ksplit > 1 ? item % p.ksplit : 0, p.ksplit, 0, 1, kb, ke);
    } else if (NI == 2) {   // half tiles are never cut
      if (w >= p.rem) break;
      item = p.rounds * p.grid + w;
      slot_id = 0;
      kb = 0;
      ke = p.nk;
    } else if (NI == 4 && p.sub64) {
      if (p.tickets == nullptr) {   // sub-tile w to workgroup w
        if (w >= p.rem * 16) break;
        int sbi, sti, stj;
        tile_at(p.g, p.rounds * p.grid + (w >> 4), sbi, sti, stj);
        const GemmArgs sg = batch_view(p.g, sbi);
        sub64_tile<F16>(sg, sti, stj, (w >> 2) & 3, w & 3, p.nk, smem, lane, wave);
        break;
      }
      // The workgroups do not leave the last full round together: the XCDs of one chip differ by
      // several per cent over two rounds.  So the sub-tiles are taken by ticket, in the order the
      // workgroups get here, and a workgroup that is done early takes another.
      // (when the tiles left over are all diagonal ones, only the 10 sub-tiles on or above the
      // diagonal of each have a ticket: the other 6 are their mirror images)
      const int per_tile = p.g.diag_last > 0 ? 10 : 16;
      for (bool first = true;; first = false) {
        __syncthreads();   // nobody still uses the first word of LDS, or the ring, for the sub-tile before
        if (tid == 0)   // (the first ticket was drawn behind the main loop of the last whole tile)
          *reinterpret_cast<volatile int*>(smem) = first ? first_ticket : draw_ticket(p.tickets, p.epoch, p.rem * per_tile + p.grid);
        __syncthreads();
        int t = __builtin_amdgcn_readfirstlane(*reinterpret_cast<volatile int*>(smem));
        int tile, si, sj;
        if (t == kNoTickets) {
          if (w >= p.rem * 16) break;
          tile = w >> 4; si = (w >> 2) & 3; sj = w & 3;
        } else {
          if (t >= p.rem * per_tile) break;
          tile = t / per_tile;
          const int idx = t - tile * per_tile;
          if (per_tile == 10) tri_decode(idx, 4, si, sj);
          else { si = idx >> 2; sj = idx & 3; }
        }
        __syncthreads();   // everybody has read the ticket before the copies overwrite it
        int sbi, sti, stj;
        tile_at(p.g, p.rounds * p.grid + tile, sbi, sti, stj);
        const GemmArgs sg = batch_view(p.g, sbi);
        sub64_tile<F16>(sg, sti, stj, si, sj, p.nk, smem, lane, wave);
        if (t == kNoTickets) break;
      }
      break;
    } else {
      if (w >= p.rem * p.split) break;
      const int j = w / p.split, sub = w - j * p.split;
      item = p.rounds * p.grid + j;
      slot_id = p.tail_slot0 + w;
      item_range(p.nk, p.ksplit > 1 ? item % p.ksplit : 0, p.ksplit, sub, p.split, kb, ke);
    }
    const int n = ke - kb;
    int bi, ti, tj, half = 0;
    bool ditem = false;   // NI == 2: a whole diagonal tile of a symmetric product
    if constexpr (NI == 2) half_item_at(p.g, item, bi, ti, tj, half, ditem);
    else tile_at(p.g, p.ksplit > 1 ? item / p.ksplit : item, bi, ti, tj);
    const GemmArgs g = batch_view(p.g, bi);
    const int m0 = ti * BM + half * 128, n0 = tj * BN;

    const bf16_t* gA = g.A + (int64_t)m0 * g.lda + (int64_t)kb * BKF;
    const bf16_t* gB = g.B + (int64_t)n0 * g.ldb + (int64_t)kb * BKF;

    if constexpr (NI == 2) {
      if (ditem) {   // a diagonal tile of a symmetric product: its panel is operand B's (A == B), rows in their own order
        uint32_t vo[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const int row = (q * 4 + wave) * 8 + (lane >> 3);
          vo[q] = (uint32_t)(row * (int)g.ldb + (((lane & 7) ^ swz(row)) * 8)) * 2u;
        }
        diag_item<F16, MODE>(g, m0, n, smem, vo, gB, ldsw, lane, wave);
        __syncthreads();   // the next item's copies land in the memory the staging just used
        continue;
      }
    }

    // DMA copy q of this wave fills LDS rows (q*4 + wave)*8 .. +8 of an operand stage (the output
    // is a whole number of tiles on this path, so every row exists); LDS row `row` holds row
    // perm_a(row) of A's panel and perm_b(row) of B's
    uint32_t voA[2 * NI], voB[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int row = (q * 4 + wave) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ swz16(row);
      // (24-bit multiplies: a row pitch is below 2^21 elements here, and a full 32-bit multiply-add
      // leaves every offset in a pair of registers)
      if (q < 2 * NI) voA[q] = (__umul24((unsigned)perm_a(row), (unsigned)g.lda) + (unsigned)(chunk * 8)) * 2u;
      voB[q] = (__umul24((unsigned)perm_b(row), (unsigned)g.ldb) + (unsigned)(chunk * 8)) * 2u;
    }

    {   // a whole tile, a part of one along k, or a half tile (never on the diagonal of a symmetric product)
      const bool diag = NI == 4 && g.symmetric && ti == tj;
      float* const slot = NI == 4 && n != p.nk ? p.partials + (size_t)slot_id * PART_FLOATS : nullptr;
      const bool draws = NI == 4 && p.sub64 && p.tickets != nullptr && round == p.rounds - 1 && tickets_live;
      whole_tile16<F16, MODE, 2 * NI>(g, diag, n, slot, smem, fa16, voA, voB, gA, gB, ldsw, m0 + wm * (32 * NI), n0 + wn * 128,
                                      lane, wave, draws ? p.tickets : nullptr, p.epoch,
                                      p.rem * (p.g.diag_last > 0 ? 10 : 16) + p.grid, first_ticket);
      __syncthreads();   // the next tile's copies land in the memory the staging just used
    }
  }
}

// Second kernel, for the tiles that were not computed whole: one workgroup per (tile, 128x128
// block, quarter).  Its four waves add the tile's parts in k order, so the bits do not depend on
// which workgroup finished when, into one staging buffer, and then share the iterations of the
// same epilogue the main kernel runs.
template <bool F16>
__global__ __launch_bounds__(256) void gemm_nt_reduce_kernel(FastArgs p) {
  __shared__ __align__(1024) unsigned char smem[EPI_WAVE_BYTES];
  __shared__ int s_slot[kMaxParts];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int t = p.reduce_tile0 + (int)(blockIdx.x >> 4), blk = (blockIdx.x >> 2) & 3, q = blockIdx.x & 3;
  int bi, ti, tj;
  tile_at(p.g, t, bi, ti, tj);
  const GemmArgs g = batch_view(p.g, bi);
  const EpiLds L = epi_lds(smem);
  const int row0 = ti * BM + (blk >> 1) * 128, col0 = tj * BN + (blk & 1) * 128;
  if (g.E) {
    epi_dma_e(g, row0 + 32 * q, col0, lane, L.e_addr[0], wave * 2, wave * 2 + 2);
    if (wave == 0) {
      float2 ra = {0.0f, 0.0f};
      if (g.row_alpha) ra = *reinterpret_cast<const float2*>(g.row_alpha + row0 + lane * 2);
      *reinterpret_cast<float2*>(L.RA + lane * 2) = ra;
    }
  }
  // the slots of this tile's parts, in k order
  const int first_tail_item = p.rounds * p.grid;
  int nparts = 0;
  for (int part = 0; part < p.ksplit; ++part) {
    const int item = t * p.ksplit + part;
    if (item < first_tail_item) {
      if (threadIdx.x == 0) s_slot[nparts] = item;
      nparts += 1;
    } else {
      if ((int)threadIdx.x < p.split) s_slot[nparts + threadIdx.x] = p.tail_slot0 + (item - first_tail_item) * p.split + threadIdx.x;
      nparts += p.split;
    }
  }
  __syncthreads();
  sum_parts_to_stage(p.partials + (blk * 4 + q) * QUARTER_FLOATS, s_slot, nparts, L.F, lane, wave * 4, wave * 4 + 4);
  wait_vmcnt<0>();
  __syncthreads();
  const bool diag = g.symmetric && ti == tj;
  // direct pass, then (after everybody has put its rounded values back) the transposed pass
  epilogue_quarter<F16>(g, diag, L.F, L.E[0], L.RA, 32 * q, row0 + 32 * q, col0, lane, wave * 2, wave * 2 + 2, 1);
  __syncthreads();
  epilogue_quarter<F16>(g, diag, L.F, L.E[0], L.RA, 32 * q, row0 + 32 * q, col0, lane, wave * 2, wave * 2 + 2, 2);
}

// ---- 128x128 tiles, one per workgroup, for problems too small for the rounds above --------------
// Such problems are bound by latency, not by the MFMA pipe: a handful of k stages per tile and
// fewer tiles than CUs.  So the operand ring is deep (four 32 KiB stages in flight through the same
// global -> LDS copies) and there is one barrier per stage.  Each of the 4 waves owns 32 rows x 128
// columns of the tile, which is exactly one quarter of the epilogue above; the operand E of that
// quarter is fetched into LDS of its own before the main loop starts.
constexpr int MID_T = 128;                              // tile edge
constexpr int MID_STAGES = 4;
constexpr int MID_OPER = MID_T * ROWB;                  // 16 KiB
constexpr int MID_STAGE = 2 * MID_OPER;                 // A and B
constexpr int MID_RING = MID_STAGES * MID_STAGE;        // 131072; reused by the accumulator staging
constexpr int MID_SMEM = MID_RING + 4 * QE_BYTES;       // + one E buffer per wave = 163840

// Few tiles and a long k (1024 x 4096: 36 tiles of 64 stages for 256 CUs): every tile is cut along k
// into `ksplit` parts, one workgroup each, which write their 128x128 fp32 sums to slot
// tile * ksplit + part of `partials`; gemm_nt_mid_reduce_kernel adds them in k order and runs the
// epilogue.  Workgroups are numbered part-major, so that neighbours work on the same k range of
// different tiles and share their operand slices in the L2.
struct MidSplit {
  int ksplit;        // 1: whole tiles, written out by this kernel
  float* partials;
};
constexpr int MID_PART_FLOATS = MID_T * MID_T;   // one fp32 partial tile: 64 KiB

template <bool F16>
__global__ __launch_bounds__(256) void gemm_nt_mid_kernel(GemmArgs gb, MidSplit sp) {
  __shared__ __align__(1024) unsigned char smem[MID_SMEM];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // workgroups are dealt round-robin to the 8 XCDs: give each XCD a contiguous run of tiles
  int w = (int)blockIdx.x;
  {
    const int chunk = (int)gridDim.x >> 3;
    if (w < chunk * 8) w = (w & 7) * chunk + (w >> 3);
  }
  const int part = sp.ksplit > 1 ? w / gb.num_tiles : 0;
  const int tile = w - part * gb.num_tiles;
  int bi, ti, tj;
  tile_at(gb, tile, bi, ti, tj);
  const GemmArgs g = batch_view(gb, bi);
  const int m0 = ti * MID_T, n0 = tj * MID_T;
  const int nk_all = g.Kc / BKF;
  const int kb = sp.ksplit > 1 ? nk_all * part / sp.ksplit : 0;
  const int nk = (sp.ksplit > 1 ? nk_all * (part + 1) / sp.ksplit : nk_all) - kb;   // stages of this workgroup
  const int row0 = m0 + wave * 32, col0 = n0;

  // the epilogue operand and the per-row additions first: they are long there when needed
  const bool use_e = !F16 && g.E != nullptr && sp.ksplit == 1;
  unsigned char* const e_buf = smem + MID_RING + wave * QE_BYTES;
  float ra = 0.0f;
  if (use_e) {
    epi_dma_e(g, row0, col0, lane, FM_LDS_ADDR(e_buf), 0, 8);
    if (g.row_alpha) ra = g.row_alpha[row0 + (lane & 31)];
  }

  // copy q of this wave fills LDS rows (q*4 + wave)*8 .. +8 of an operand stage
  uint32_t voA[4], voB[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int row = (q * 4 + wave) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ swz(row);
    voA[q] = (uint32_t)(row * (int)g.lda + chunk * 8) * 2u;
    voB[q] = (uint32_t)(row * (int)g.ldb + chunk * 8) * 2u;
  }
  const bf16_t* gA = g.A + (int64_t)m0 * g.lda + (int64_t)kb * BKF;
  const bf16_t* gB = g.B + (int64_t)n0 * g.ldb + (int64_t)kb * BKF;
  const uint32_t ring = FM_LDS_ADDR(smem) + wave * 1024;
  auto issue = [&](int stage, int slot) {   // 8 copies per wave
    const uint32_t base = ring + slot * MID_STAGE;
#pragma unroll
    for (int q = 0; q < 4; ++q) dma16(voA[q], gA + stage * BKF, base + q * 4096);
#pragma unroll
    for (int q = 0; q < 4; ++q) dma16(voB[q], gB + stage * BKF, base + MID_OPER + q * 4096);
  };

  // The waves take 64x64 each (2x2 MFMA tiles): 4 fragment reads for 4 MFMAs per substep instead
  // of the 5 of a 32x128 strip; the loop is bound by the LDS (reads and incoming copies).
  // Fragment offsets inside an operand stage (row = lane % 32, k half = lane / 32):
  const int wm = wave >> 1, wn = wave & 1;
  uint32_t ao[2], bo[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = wm * 64 + i * 32 + (lane & 31);
    ao[i] = (uint32_t)(r * ROWB + (((lane >> 5) ^ swz(r)) << 4));
    const int rb = wn * 64 + i * 32 + (lane & 31);
    bo[i] = (uint32_t)(rb * ROWB + (((lane >> 5) ^ swz(rb)) << 4));
  }

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Stages past the end are the last stage again (into a slot nobody reads), so that the number of
  // copies in flight is the same at every wait.
#pragma unroll
  for (int s = 0; s < MID_STAGES - 1; ++s) issue(s < nk ? s : nk - 1, s);
  for (int s = 0; s < nk; ++s) {
    wait_vmcnt<8 * (MID_STAGES - 2)>();   // my copies of stage s have landed ...
    __syncthreads();                      // ... and everybody's; stage s-1 is read out everywhere
    // the 8 copies of the stage three ahead go out two per substep, an even stream of requests
    // instead of a burst behind the barrier
    const int nx = s + MID_STAGES - 1;
    const int nstage = nx < nk ? nx : nk - 1;
    const uint32_t nbase = ring + (nx & (MID_STAGES - 1)) * MID_STAGE;
    const unsigned char* sa = smem + (s & (MID_STAGES - 1)) * MID_STAGE;
    const unsigned char* sb = sa + MID_OPER;
    // the 4 fragment reads of substep ks+1 ride on the 4 MFMAs of substep ks
    bf16x8_t fa[2][2], fb[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      fa[0][i] = *reinterpret_cast<const bf16x8_t*>(sa + ao[i]);
      fb[0][i] = *reinterpret_cast<const bf16x8_t*>(sb + bo[i]);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks < 3) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          fa[nxt][i] = *reinterpret_cast<const bf16x8_t*>(sa + (ao[i] ^ ((ks + 1) << 5)));
          fb[nxt][i] = *reinterpret_cast<const bf16x8_t*>(sb + (bo[i] ^ ((ks + 1) << 5)));
        }
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma_32x32x16<F16>(fa[cur][i], fb[cur][j], acc[i][j]);
      if (ks < 2) {
#pragma unroll
        for (int q = 2 * ks; q < 2 * ks + 2; ++q) dma16(voA[q], gA + nstage * BKF, nbase + q * 4096);
      } else {
#pragma unroll
        for (int q = 2 * ks - 4; q < 2 * ks - 2; ++q) dma16(voB[q], gB + nstage * BKF, nbase + MID_OPER + q * 4096);
      }
      if (ks < 3) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  wait_vmcnt<0>();
  __syncthreads();   // no copy in flight and no wave still reading: the ring is free

  // accumulators -> LDS: MFMA tile (i, j) of this wave belongs to quarter 2 wm + i, columns
  // 64 wn + 32 j; then every wave finishes one quarter (the staging areas lie in the ring)
  float* const RA = reinterpret_cast<float*>(smem + 4 * (QF_FLOATS * 4) + wave * 128);
  if (use_e && lane < 32) RA[lane] = ra;   // zeros when there are no per-row additions
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
      stage_tile(acc[i][j], reinterpret_cast<float*>(smem + (2 * wm + i) * (QF_FLOATS * 4)), 2 * wn + j, lane);
  __syncthreads();
  float* const F = reinterpret_cast<float*>(smem + wave * (QF_FLOATS * 4));
  if (sp.ksplit > 1) {   // a part of a tile: quarter `wave` of its fp32 sums, in staging order
    copy_stage_to_ws(F, sp.partials + (size_t)(tile * sp.ksplit + part) * MID_PART_FLOATS + wave * QUARTER_FLOATS, lane);
    return;
  }
  const bool diag = g.symmetric && ti == tj;
  epilogue_quarter<F16>(g, diag, F, e_buf, RA, 0, row0, col0, lane, 0, 8, 3);
}

// Second kernel of the cut 128x128 tiles: one workgroup per (tile, quarter).  Its four waves add
// the quarter's parts in k order, so the bits do not depend on which workgroup finished when, and
// share the iterations of its epilogue.
template <bool F16>
__global__ __launch_bounds__(256) void gemm_nt_mid_reduce_kernel(GemmArgs gb, MidSplit sp) {
  __shared__ __align__(1024) unsigned char smem[EPI_WAVE_BYTES];
  __shared__ int s_slot[kMaxParts];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int t = (int)(blockIdx.x >> 2), q = blockIdx.x & 3;
  int bi, ti, tj;
  tile_at(gb, t, bi, ti, tj);
  const GemmArgs g = batch_view(gb, bi);
  const EpiLds L = epi_lds(smem);
  const int row0 = ti * MID_T + 32 * q, col0 = tj * MID_T;
  if (g.E) {
    epi_dma_e(g, row0, col0, lane, L.e_addr[0], wave * 2, wave * 2 + 2);
    if (wave == 0 && lane < 32) L.RA[lane] = g.row_alpha ? g.row_alpha[row0 + lane] : 0.0f;
  }
  if ((int)threadIdx.x < sp.ksplit) s_slot[threadIdx.x] = t * sp.ksplit + (int)threadIdx.x;
  __syncthreads();
  sum_parts_to_stage(sp.partials + q * QUARTER_FLOATS, s_slot, sp.ksplit, L.F, lane, wave * 4, wave * 4 + 4, MID_PART_FLOATS);
  wait_vmcnt<0>();
  __syncthreads();
  const bool diag = g.symmetric && ti == tj;
  // direct pass, then (after everybody has put its rounded values back) the transposed pass
  epilogue_quarter<F16>(g, diag, L.F, L.E[0], L.RA, 0, row0, col0, lane, wave * 2, wave * 2 + 2, 1);
  __syncthreads();
  epilogue_quarter<F16>(g, diag, L.F, L.E[0], L.RA, 0, row0, col0, lane, wave * 2, wave * 2 + 2, 2);
}

}  // namespace

constexpr size_t kTicketBytes = 256;   // what a workspace holds behind its partial-tile slots
// where this process starts numbering its launches: 2^30 .. 2^46, from the clock and the address space
static unsigned long long first_launch_number() {
  const unsigned long long t = (unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count();
  const unsigned long long a = (unsigned long long)reinterpret_cast<uintptr_t>(&kTicketBytes);
  unsigned long long x = t ^ (a * 0x9E3779B97F4A7C15ull);
  x ^= x >> 29; x *= 0xBF58476D1CE4E5B9ull; x ^= x >> 32;
  return (1ull << 30) + (x & ((1ull << 46) - 1));
}

// Too few tiles for one round (M = 4096 gives 136 symmetric tiles) and a long k: every tile is cut
// along k into as many base parts as fill the chip, each at least 64 stages long so that the fp32
// round trip of its partial tile stays a small part of its time.
static int auto_ksplit(long long num_tiles, int nk, int grid) {
  int ksplit = 1;
  if (num_tiles * 5 < (long long)grid * 3 && nk >= 128) {
    ksplit = (int)(grid / num_tiles);
    if (ksplit < 2) ksplit = 2;
    if (ksplit > nk / 64) ksplit = nk / 64;
    if (ksplit > kMaxKsplit) ksplit = kMaxKsplit;
  }
  return ksplit;
}

// the schedule for `num_tiles` tiles of `nk` k stages; `max_slots` partial-tile slots are there
static void fast_schedule(int num_tiles, int nk, long long max_slots, FastArgs& f) {
  int grid = cu_count();                            // one workgroup per CU (160 KiB of LDS each)
  if (grid > kMaxGrid) grid = kMaxGrid;
  const long long kg = knob(kKnobGrid);             // tuning aid
  if (kg > 0 && kg < grid) grid = (int)kg;
  int ksplit = auto_ksplit(num_tiles, nk, grid);
  const long long kk = knob(kKnobKsplit);           // tuning aid
  if (kk > 0) ksplit = (int)kk;
  if (ksplit < 1 || ksplit > nk || ksplit > kMaxKsplit) ksplit = 1;
  if (ksplit > 1 && (long long)num_tiles * ksplit + grid > max_slots) ksplit = 1;   // slots: items + rem * split
  const int items = num_tiles * ksplit;
  if (grid > items) grid = items;                   // rem * split never exceeds the grid below
  if (grid < 1) grid = 1;
  f.grid = grid;
  f.ksplit = ksplit;
  f.rounds = items / grid;
  f.rem = items % grid;
  f.split = 1;
  if (f.rem > 0) {
    int s = grid / f.rem;                           // sub-parts that fit in one round of workgroups
    const int base_stages = nk / ksplit;
    if (s > base_stages) s = base_stages;
    if (s > 16) s = 16;                             // bounds the partial-tile traffic
    if (s > kMaxParts / ksplit) s = kMaxParts / ksplit;
    // what the workspace holds; with ksplit == 1 and no room the last round runs whole tiles
    const long long room = max_slots - (ksplit > 1 ? (long long)f.rounds * grid : 0);
    if ((long long)f.rem * s > room) s = (int)(room / f.rem);
    f.split = s < 1 ? 1 : s;
  }
  // whole tiles left over, few enough for 16 workgroups each: cut them in space, not along k
  f.sub64 = (ksplit == 1 && f.rem > 0 && f.rem * 16 <= grid && knob(kKnobNoSub64) <= 0) ? 1 : 0;
  if (f.sub64) f.split = 1;
  f.tail_slot0 = ksplit > 1 ? f.rounds * grid : 0;
  // whole tiles need no second kernel: with ksplit == 1 only the left-over items, if they were cut
  f.reduce_tile0 = ksplit > 1 ? 0 : (f.split > 1 ? f.rounds * grid : num_tiles);
}

// what both tile shapes ask of a problem: whole tiles of edge `tile`, whole k stages, 16-byte
// accesses everywhere
static bool tiled_dma_eligible(const GemmArgs& a, int tile) {
  if (a.elem == kElemF32 || (a.elem == kElemF16 && a.E)) return false;
  if (a.Kc < BKF || a.Kc % BKF != 0) return false;
  if (a.lda % 8 != 0 || a.ldb % 8 != 0) return false;
  if ((reinterpret_cast<uintptr_t>(a.A) & 15) || (reinterpret_cast<uintptr_t>(a.B) & 15)) return false;
  if (a.Ma % tile != 0 || a.Nb % tile != 0) return false;       // whole tiles only: no edge masks here
  // in-tile byte offsets stay below 2^31
  if (a.lda >= (1 << 21) || a.ldb >= (1 << 21)) return false;
  if (a.C && (a.c_cs != 1 || a.c_rs >= (1 << 21))) return false;
  if (a.C2 && (a.c2_cs != 1 || a.c2_rs >= (1 << 21))) return false;
  // 16-byte accesses of the epilogue
  if (a.C && (a.c_rs % 8 != 0 || (reinterpret_cast<uintptr_t>(a.C) & 15))) return false;
  if (a.C2 && (a.c2_rs % 8 != 0 || (reinterpret_cast<uintptr_t>(a.C2) & 15))) return false;
  if (a.E && (a.lde % 8 != 0 || a.lde >= (1 << 21) || (reinterpret_cast<uintptr_t>(a.E) & 15))) return false;
  if (a.row_alpha && ((reinterpret_cast<uintptr_t>(a.row_alpha) & 15) || a.bs_ra % 4 != 0)) return false;
  for (int i = 0; i < a.batch && i < kMaxBatch; ++i) {
    if (a.use_c_list && (reinterpret_cast<uintptr_t>(a.c_list[i]) & 15)) return false;
    if (a.use_c2_list && (reinterpret_cast<uintptr_t>(a.c2_list[i]) & 15)) return false;
  }
  if (a.batch > 1 && (a.bs_a % 8 || a.bs_b % 8 || a.bs_e % 8 || a.bs_c % 8 || a.bs_c2 % 8)) return false;
  return true;
}

// Parts per 128x128 tile along k, by estimate in microseconds (measured: 0.36 per stage, 4.5 for a
// tile's start and write-out; cut, 11 for the fp32 round trip and the second launch and 0.035 per
// part for their traffic).  At most as many parts as fill the chip, of at least 8 stages each; the
// tiles stay whole unless the cut saves a tenth.
static double estimate_mid_cut(long long tiles, int nk, int s) {
  return (double)((nk + s - 1) / s) * 0.36 + 11.0 + 0.035 * (double)(tiles * s);
}
static int mid_ksplit(long long tiles, int nk, int grid) {
  const long long k = knob(kKnobKsplit);
  if (k >= 1) {
    const int s = (int)(k > kMaxParts ? kMaxParts : k);
    return s > nk ? nk : s;
  }
  if (tiles * 2 > grid || nk < 16) return 1;
  int smax = (int)(grid / tiles);
  if (smax > nk / 8) smax = nk / 8;
  if (smax > 16) smax = 16;
  int best = 1;
  double t_best = 0.9 * (nk * 0.36 + 4.5);
  for (int s = 2; s <= smax; ++s) {
    const double t = estimate_mid_cut(tiles, nk, s);
    if (t < t_best) { t_best = t; best = s; }
  }
  return best;
}
// (a stage costs 0.36 us while about half the CUs work and 0.52 when all do; a write-out with an
// operand E costs 5 more)
static double estimate_mid(long long tiles, int nk, int grid, bool with_e) {
  const int s = mid_ksplit(tiles, nk, grid);
  if (s > 1) return estimate_mid_cut(tiles, nk, s) + (with_e ? 5.0 : 0.0);
  const double occ = tiles >= grid ? 1.0 : (double)tiles / grid;
  const double stage = 0.36 + 0.36 * (occ > 0.55 ? occ - 0.55 : 0.0);
  return (double)((tiles + grid - 1) / grid) * (nk * stage + (with_e ? 11.0 : 6.0));
}

// Estimates in microseconds, from measured costs of a k stage and of a tile's start and write-out.
// The clock the power cap allows falls as the chip fills, so a stage costs more the more CUs work.
// One round of whole tiles (cut along k into `ksplit` parts, which adds the fp32 parts and the
// second kernel):
static double estimate_whole_round(long long tiles, int nk, int ksplit, int grid) {
  double occ = (double)(tiles * ksplit) / grid;
  if (occ > 1.0) occ = 1.0;
  return (nk / ksplit) * (0.35 + 1.1 * occ) + 15.0 + (ksplit > 1 ? 25.0 : 0.0);
}
// one round of half tiles:
static double estimate_half_round(long long half_items, int nk, int grid) {
  const double occ = (double)half_items / grid;
  return nk * (0.50 + 0.78 * (occ > 0.6 ? occ - 0.6 : 0.0)) + 13.0;
}

// The half-tile schedule (128x256 items, a diagonal tile of a symmetric product as one item) is
// taken when all its items fit into one round and that round is estimated to be shorter than the
// round of whole tiles: those would leave about half of the CUs idle, and half items are never
// cut, so nothing is added up afterwards.  Few tiles with a very long k are better cut along k
// (16 half items of 1024 stages against 160 parts of 64), and with more items than workgroups
// whole tiles win: a stage of a half tile costs more than half a stage of a whole one (48 KiB of
// operands for half the MFMAs).
static bool half_schedule_chosen(long long half_items, long long tiles, int nk, int grid) {
  const long long k = knob(kKnobHalf);
  if (k >= 0) return k > 0;
  if (knob(kKnobKsplit) >= 0 || half_items > grid || tiles > grid || nk < 8) return false;
  return estimate_half_round(half_items, nk, grid) < estimate_whole_round(tiles, nk, auto_ksplit(tiles, nk, grid), grid);
}

// Few tiles (at most a sixteenth of the workgroups) can also run as 64x64 sub-tiles over the whole
// k, 16 workgroups per tile, the way the tiles left after the last full round do: one launch, no
// fp32 parts, and sixteen times the workgroups of whole tiles.  A sub-tile stage moves four times
// the operand bytes per flop, so this pays up to about 64-80 k stages; beyond, the 128x128 tiles cut
// along k win.  Measured on X X^T: 6.5 us + 0.205 us per stage (1024 x 1024 10, 1024 x 2048 13,
// 1024 x 4096 20, 1024 x 8192 34 us); five Newton-Schulz steps at 1024^2 200 -> 176 us, 512 x 2048
// 204 -> 170, 768^2 185 -> 160.
static bool sub64_schedule_chosen(const GemmArgs& a, long long tiles, int nk, int grid) {
  const long long ns = knob(kKnobNoSub64);       // 1: never; 0: whenever it fits; left alone: by the estimate below
  if (ns > 0 || tiles < 1 || tiles * 16 > grid) return false;
  if (ns == 0) return true;
  if (knob(kKnobKsplit) >= 0 || knob(kKnobHalf) >= 0 || knob(kKnobFastMinUnits) >= 0) return false;
  const long long tm = a.Ma / BM, tn = a.Nb / BN, nb = a.batch < 1 ? 1 : a.batch;
  const double t_sub = nk * 0.205 + 6.5 + (a.E ? 2.0 : 0.0);
  const long long small_tiles = (a.symmetric ? 2 * tm * (2 * tm + 1) / 2 : 4 * tm * tn) * nb;
  double t_best = estimate_mid(small_tiles, nk, grid, a.E != nullptr);
  const int ksplit = auto_ksplit(tiles, nk, grid);
  const double t_large = (nk / ksplit) * 1.45 + 15.0 + (ksplit > 1 ? 25.0 : 0.0);
  if (t_large < t_best) t_best = t_large;
  const long long half_items = (a.symmetric ? tm * tm : 2 * tm * tn) * nb;
  if (half_schedule_chosen(half_items, tiles, nk, grid)) {
    const double t_half = estimate_half_round(half_items, nk, grid);
    if (t_half < t_best) t_best = t_half;
  }
  return t_sub < t_best;
}

bool gemm_fast_eligible(const GemmArgs& a) {
  if (!tiled_dma_eligible(a, BM)) return false;
  // the write-out reads the epilogue operand transposed, 16 bytes at a time
  if (a.E && (!a.ET || a.ldet % 8 != 0 || a.ldet >= (1 << 21) || (reinterpret_cast<uintptr_t>(a.ET) & 15) || (a.batch > 1 && a.bs_et % 8))) return false;
  const long long tm = a.Ma / BM, tn = a.Nb / BN;
  const long long tiles = (a.symmetric ? tm * (tm + 1) / 2 : tm * tn) * (a.batch < 1 ? 1 : a.batch);
  const int nk = a.Kc / BKF;
  // the FAST_MIN_UNITS knob replaces the choice below by a threshold on (tile, k-stage) units,
  // e.g. 0 to exercise this path on small inputs
  if (knob(kKnobFastMinUnits) >= 0) return tiles * nk >= knob(kKnobFastMinUnits);
  // More tiles than workgroups: rounds of large tiles.  Otherwise it is one round of 256x256 tiles
  // on some of the CUs against one or more waves of 128x128 tiles on all of them; estimate both in
  // microseconds from the measured cost of a k stage and of a tile's epilogue on each path.
  const int cus = cu_count() < kMaxGrid ? cu_count() : kMaxGrid;
  if (tiles > cus) return true;
  if (sub64_schedule_chosen(a, tiles, nk, cus)) return true;
  const int ksplit = auto_ksplit(tiles, nk, cus);
  const double t_large = (nk / ksplit) * 1.45 + 15.0 + (ksplit > 1 ? 25.0 : 0.0);
  const long long small_tiles = (a.symmetric ? 2 * tm * (2 * tm + 1) / 2 : 4 * tm * tn) * (a.batch < 1 ? 1 : a.batch);
  const double t_small = estimate_mid(small_tiles, nk, cus, a.E != nullptr);
  const long long half_items = (a.symmetric ? tm * tm : 2 * tm * tn) * (a.batch < 1 ? 1 : a.batch);
  // (the 128x128 tiles keep the benefit of the doubt against half tiles)
  if (half_schedule_chosen(half_items, tiles, nk, cus) && estimate_half_round(half_items, nk, cus) < 0.9 * t_small) return true;
  return t_large < t_small;
}

bool gemm_mid_eligible(const GemmArgs& a) { return tiled_dma_eligible(a, MID_T); }

int launch_gemm_mid(GemmArgs a, void* ws, size_t ws_bytes, hipStream_t stream) {
  a.tiles_m = a.Ma / MID_T;
  a.tiles_n = a.Nb / MID_T;
  if (a.batch < 1) a.batch = 1;
  a.num_tiles = (a.symmetric ? a.tiles_m * (a.tiles_m + 1) / 2 : a.tiles_m * a.tiles_n) * a.batch;
  MidSplit sp;
  sp.ksplit = mid_ksplit(a.num_tiles, a.Kc / BKF, cu_count() < kMaxGrid ? cu_count() : kMaxGrid);
  sp.partials = static_cast<float*>(ws);
  // without room for the parts the tiles stay whole
  if (sp.ksplit > 1 && (!ws || (size_t)a.num_tiles * sp.ksplit * MID_PART_FLOATS * sizeof(float) > ws_bytes)) sp.ksplit = 1;
  const unsigned grid = (unsigned)(a.num_tiles * sp.ksplit);
  if (a.elem == kElemF16) hipLaunchKernelGGL(gemm_nt_mid_kernel<true>, dim3(grid), dim3(256), 0, stream, a, sp);
  else hipLaunchKernelGGL(gemm_nt_mid_kernel<false>, dim3(grid), dim3(256), 0, stream, a, sp);
  if (sp.ksplit > 1) {
    if (a.elem == kElemF16) hipLaunchKernelGGL(gemm_nt_mid_reduce_kernel<true>, dim3(a.num_tiles * 4), dim3(256), 0, stream, a, sp);
    else hipLaunchKernelGGL(gemm_nt_mid_reduce_kernel<false>, dim3(a.num_tiles * 4), dim3(256), 0, stream, a, sp);
  }
  return (int)hipGetLastError();
}

size_t gemm_fast_workspace_bytes(int Ma, int Nb, int batch) {
  if (batch < 1) batch = 1;
  // the 128x128 path cuts its tiles along k when at most half the CUs would have one: one round of parts
  size_t mid_need = 0;
  if (Ma >= MID_T && Nb >= MID_T && Ma % MID_T == 0 && Nb % MID_T == 0) {
    const long long m = Ma / MID_T, n = Nb / MID_T;
    const long long fewest = (Ma == Nb ? m * (m + 1) / 2 : m * n) * batch;
    if (fewest * 2 <= kMaxGrid) mid_need = (size_t)kMaxGrid * MID_PART_FLOATS * sizeof(float);
  }
  if (Ma < BM || Nb < BN || Ma % BM != 0 || Nb % BN != 0) return mid_need;   // never on the 256x256 path
  const long long tm = Ma / BM, tn = Nb / BN;
  // a square output may be a symmetric product (fewer tiles) or a general one: take the larger need
  long long need = 0;
  for (int sym = 0; sym < (Ma == Nb ? 2 : 1); ++sym) {
    const long long tiles = (sym ? tm * (tm + 1) / 2 : tm * tn) * batch;
    long long slots;
    if (tiles * 5 < (long long)kMaxGrid * 3) {
      // every tile may be cut into base parts (auto_ksplit), and the left-over items once more
      slots = tiles * kMaxKsplit + kMaxGrid;
      if (slots > kMaxSlots) slots = kMaxSlots;
    } else {
      // only the items left after the last full round are cut, into at most one round of parts
      slots = kMaxGrid;
    }
    if (slots > need) need = slots;
  }
  const size_t fast_need = (size_t)need * PART_FLOATS * sizeof(float);
  // (the ticket word of the sub-tile rounds lies behind the slots; a product of more tiles than CUs
  // that cuts nothing still has it)
  return (fast_need > mid_need ? fast_need : mid_need) + kTicketBytes;
}

int launch_gemm_fast(GemmArgs a, void* ws, size_t ws_bytes, hipStream_t stream) {
  a.tiles_m = a.Ma / BM;
  a.tiles_n = a.Nb / BN;
  if (a.batch < 1) a.batch = 1;
  a.num_tiles = (a.symmetric ? a.tiles_m * (a.tiles_m + 1) / 2 : a.tiles_m * a.tiles_n) * a.batch;
  FastArgs f;
  f.g = a;
  f.nk = a.Kc / BKF;
  // the last 256 bytes of a workspace are the ticket word's (below), the partial-tile slots lie in front of them
  const size_t slot_bytes = ws && ws_bytes >= kTicketBytes ? ws_bytes - kTicketBytes : 0;
  const long long have = (long long)(slot_bytes / (PART_FLOATS * sizeof(float)));
  fast_schedule(a.num_tiles, f.nk, have < kMaxSlots ? have : kMaxSlots, f);
  f.half = 0;
  int grid = cu_count() < kMaxGrid ? cu_count() : kMaxGrid;
  const long long kg = knob(kKnobGrid);
  if (kg > 0 && kg < grid) grid = (int)kg;
  const long long half_items = a.symmetric ? (long long)a.tiles_m * a.tiles_m * a.batch : 2LL * a.num_tiles;   // a diagonal tile is one item
  if (sub64_schedule_chosen(a, a.num_tiles, f.nk, grid)) {   // every tile as 16 sub-tiles of 64x64, one workgroup each
    f.grid = a.num_tiles * 16;
    f.ksplit = 1;
    f.rounds = 0;
    f.rem = a.num_tiles;
    f.split = 1;
    f.sub64 = 1;
    f.tail_slot0 = 0;
    f.reduce_tile0 = a.num_tiles;
  } else if (half_items < (1LL << 30) && half_schedule_chosen(half_items, a.num_tiles, f.nk, grid)) {   // 128x256 half tiles, whole, in rounds
    const int items = (int)half_items;
    if (grid > items) grid = items;
    f.half = 1;
    f.grid = grid;
    f.ksplit = 1;
    f.rounds = items / grid;
    f.rem = items % grid;
    f.split = 1;
    f.sub64 = 0;
    f.tail_slot0 = 0;
    f.reduce_tile0 = a.num_tiles;
  }
  // Sub-tiles left over from a symmetric product: let them be diagonal tiles.  Such a tile needs one
  // operand panel where another needs two (the last round is bound by what the L2s fetch), and 10 of
  // its 16 sub-tiles are distinct.  The bits are those of any other order.
  if (f.sub64 && f.rounds > 0 && a.symmetric && a.batch == 1 && f.rem <= a.tiles_m && knob(kKnobDiagLast) != 0)
    f.g.diag_last = f.rem;
  f.partials = static_cast<float*>(ws);
  // The sub-tiles behind full rounds go out by ticket when there is a workspace to count in: the
  // word is the first of its last 256-byte block.  65535 tickets at most.  Launch numbers start at a
  // value of this process's own (so that a word another process left in the same memory does not
  // carry a number this one will reach) and stay below 2^47.
  f.tickets = nullptr;
  f.epoch = 0;
  if (f.sub64 && f.rounds > 0 && ws && ws_bytes >= 2 * kTicketBytes && f.rem * 16 + f.grid < 65536 && knob(kKnobNoTickets) <= 0) {
    // (fewer than 65536 tickets; whether a tile has 10 or 16 is the kernel's business)
    static std::atomic<unsigned long long> launches{first_launch_number()};
    f.epoch = launches.fetch_add(1, std::memory_order_relaxed) & 0x7fffffffffffull;
    if (f.epoch != 0)
      f.tickets = reinterpret_cast<unsigned long long*>(static_cast<unsigned char*>(ws) + (ws_bytes / kTicketBytes - 1) * kTicketBytes);
  }
  if (f.half) {
    if (a.elem == kElemF16) hipLaunchKernelGGL((gemm_nt_rounds_kernel<true, 0, 2>), dim3(f.grid), dim3(256), 0, stream, f);
    else if (!a.E) hipLaunchKernelGGL((gemm_nt_rounds_kernel<false, 0, 2>), dim3(f.grid), dim3(256), 0, stream, f);
    else if (a.beta == 1.0f) hipLaunchKernelGGL((gemm_nt_rounds_kernel<false, 1, 2>), dim3(f.grid), dim3(256), 0, stream, f);
    else hipLaunchKernelGGL((gemm_nt_rounds_kernel<false, 2, 2>), dim3(f.grid), dim3(256), 0, stream, f);
    return (int)hipGetLastError();
  }
  const int slots = f.tail_slot0 + f.rem * f.split;
  const int reduce_tiles = a.num_tiles - f.reduce_tile0;
  if (reduce_tiles > 0 && (slots > have || f.ksplit * f.split > kMaxParts)) return kErrWorkspace;
  if (a.elem == kElemF16) {
    hipLaunchKernelGGL((gemm_nt_rounds_kernel<true, 0, 4>), dim3(f.grid), dim3(256), 0, stream, f);
    if (reduce_tiles > 0)
      hipLaunchKernelGGL(gemm_nt_reduce_kernel<true>, dim3(reduce_tiles * 16), dim3(256), 0, stream, f);
  } else {
    if (!a.E) hipLaunchKernelGGL((gemm_nt_rounds_kernel<false, 0, 4>), dim3(f.grid), dim3(256), 0, stream, f);
    else if (a.beta == 1.0f) hipLaunchKernelGGL((gemm_nt_rounds_kernel<false, 1, 4>), dim3(f.grid), dim3(256), 0, stream, f);
    else hipLaunchKernelGGL((gemm_nt_rounds_kernel<false, 2, 4>), dim3(f.grid), dim3(256), 0, stream, f);
    if (reduce_tiles > 0)
      hipLaunchKernelGGL(gemm_nt_reduce_kernel<false>, dim3(reduce_tiles * 16), dim3(256), 0, stream, f);
  }
  return (int)hipGetLastError();
}

}  // namespace fm
