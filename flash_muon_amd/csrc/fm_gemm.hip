// MFMA contraction for gfx950, any shape, stride and alignment: acc = A * B^T with both operands
// k-contiguous ("NT"), fp32 accumulation in 32x32 MFMA tiles (32x32x16 for bf16 and fp16 operands,
// 32x32x2 for fp32 operands), LDS double buffering, fused epilogue and an optional mirrored
// (transposed) second store.  X*X^T, b*A + c*A*A and a*X + P*X are all instances of it (see GemmArgs).
#include "fm_internal.h"
#include <atomic>
#include <cstdlib>

namespace fm {

constexpr int ROW_BYTES = 128;         // one LDS row: the k extent of a stage, 64 16-bit or 32 32-bit elements

__device__ __forceinline__ uint32_t lds_off(int row, int chunk) {
  return (uint32_t)(row * ROW_BYTES + ((chunk ^ swz(row)) << 4));
}

// ES: bytes per element (2 or 4).  A 16-byte chunk holds 16 / ES consecutive k.
template <int ROWS, int NT, bool ALIGNED, int ES>
struct TileLoader {
  static constexpr int N = ROWS * 8 / NT;   // 16-byte chunks per thread
  static constexpr int EPC = 16 / ES;       // elements per chunk
  static_assert(ROWS * 8 % NT == 0, "tile rows must divide over the threads");
  const unsigned char* ptr[N];   // row base + chunk offset, per chunk
  uint32_t soff[N];              // swizzled LDS byte offset, per chunk
  int kch[N];                    // k offset of the chunk inside a stage

  __device__ __forceinline__ void init(const void* base, int64_t ld, int row0, int nrows, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      int idx = tid + i * NT;
      int row = idx >> 3, ch = idx & 7;
      int grow = row0 + row;
      if (grow > nrows - 1) grow = nrows - 1;   // rows past the end repeat the last row; never stored
      ptr[i] = static_cast<const unsigned char*>(base) + ((int64_t)grow * ld + ch * EPC) * ES;
      soff[i] = lds_off(row, ch);
      kch[i] = ch * EPC;
    }
  }

  __device__ __forceinline__ void load(uint4 (&r)[N], int k0, int K) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      int k = k0 + kch[i];
      const unsigned char* src = ptr[i] + (int64_t)k0 * ES;
      if (ALIGNED) {
        if (k < K) r[i] = *reinterpret_cast<const uint4*>(src);
        else r[i] = make_uint4(0, 0, 0, 0);
      } else if (ES == 2) {
        union { uint4 v; unsigned short h[8]; } u;
        const unsigned short* s = reinterpret_cast<const unsigned short*>(src);
#pragma unroll
        for (int e = 0; e < 8; ++e) u.h[e] = (k + e < K) ? s[e] : (unsigned short)0;
        r[i] = u.v;
      } else {
        union { uint4 v; uint32_t w[4]; } u;
        const uint32_t* s = reinterpret_cast<const uint32_t*>(src);
#pragma unroll
        for (int e = 0; e < 4; ++e) u.w[e] = (k + e < K) ? s[e] : 0u;
        r[i] = u.v;
      }
    }
  }

  __device__ __forceinline__ void store(unsigned char* lds, const uint4 (&r)[N]) const {
#pragma unroll
    for (int i = 0; i < N; ++i) *reinterpret_cast<uint4*>(lds + soff[i]) = r[i];
  }
};

// One 16-byte fragment pair into the accumulator: one 32x32x16 MFMA for 16-bit elements; for fp32
// the chunk holds 4 consecutive k of this lane's k group, which are 4 steps of the 32x32x2 MFMA
// (A and B use the same k order, and a sum does not care which order that is).
template <int ET>
__device__ __forceinline__ f32x16_t mfma_chunk(bf16x8_t a, bf16x8_t b, f32x16_t c) {
  if constexpr (ET == kElemF32) {
    const f32x4_t fa = __builtin_bit_cast(f32x4_t, a), fb = __builtin_bit_cast(f32x4_t, b);
#pragma unroll
    for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[e], fb[e], c, 0, 0, 0);
    return c;
  } else {
    return mfma_32x32x16<ET == kElemF16>(a, b, c);
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool ALIGNED, int ET>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_nt_kernel(GemmArgs pb) {
  const GemmArgs p = batch_view(pb, (int)blockIdx.y);
  constexpr int NT = 64 * WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int ES = ET == kElemF32 ? 4 : 2;
  constexpr int BK = ROW_BYTES / ES;     // elements of k per stage
  constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES;
  constexpr int STAGE = A_BYTES + B_BYTES;

  __shared__ __align__(16) unsigned char smem[2 * STAGE];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  int ti, tj;
  if (p.symmetric) {
    tri_decode((int)blockIdx.x, p.tiles_m, ti, tj);
  } else {
    ti = (int)blockIdx.x / p.tiles_n;
    tj = (int)blockIdx.x % p.tiles_n;
  }
  const int m0 = ti * BM, n0 = tj * BN;

  TileLoader<BM, NT, ALIGNED, ES> la;
  TileLoader<BN, NT, ALIGNED, ES> lb;
  la.init(p.A, p.lda, m0, p.Ma, tid);
  lb.init(p.B, p.ldb, n0, p.Nb, tid);

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // per-lane fragment addresses: row = lane % 32 of each 32-row block, k half = lane / 32
  uint32_t a_off[TM], b_off[TN];
  int a_sw[TM], b_sw[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    int row = wm * WM + i * 32 + (lane & 31);
    a_off[i] = (uint32_t)(row * ROW_BYTES);
    a_sw[i] = swz(row);
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    int row = wn * WN + j * 32 + (lane & 31);
    b_off[j] = (uint32_t)(A_BYTES + row * ROW_BYTES);
    b_sw[j] = swz(row);
  }
  const int khalf = lane >> 5;

  const int nk = (p.Kc + BK - 1) / BK;
  uint4 ra[TileLoader<BM, NT, ALIGNED, ES>::N], rb[TileLoader<BN, NT, ALIGNED, ES>::N];

  la.load(ra, 0, p.Kc);
  lb.load(rb, 0, p.Kc);
  la.store(smem, ra);
  lb.store(smem + A_BYTES, rb);
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    unsigned char* cur = smem + (kt & 1) * STAGE;
    unsigned char* nxt = smem + ((kt + 1) & 1) * STAGE;
    const bool more = kt + 1 < nk;
    if (more) {
      la.load(ra, (kt + 1) * BK, p.Kc);
      lb.load(rb, (kt + 1) * BK, p.Kc);
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {   // 8 chunks per row: chunk 2*ks + khalf belongs to this lane
      bf16x8_t fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        fa[i] = *reinterpret_cast<const bf16x8_t*>(cur + a_off[i] + (((ks * 2 + khalf) ^ a_sw[i]) << 4));
#pragma unroll
      for (int j = 0; j < TN; ++j)
        fb[j] = *reinterpret_cast<const bf16x8_t*>(cur + b_off[j] + (((ks * 2 + khalf) ^ b_sw[j]) << 4));
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = mfma_chunk<ET>(fa[i], fb[j], acc[i][j]);
    }
    if (more) {
      la.store(nxt, ra);
      lb.store(nxt + A_BYTES, rb);
    }
    __syncthreads();
  }

  // Epilogue.  In the 32x32 accumulator, register r of lane l holds
  // row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the MFMA tile.
  const bool diag = p.symmetric && (ti == tj);
  const bool has_e = p.E != nullptr;
  unsigned short* C = reinterpret_cast<unsigned short*>(p.C);
  unsigned short* C2 = reinterpret_cast<unsigned short*>(p.C2);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wn * WN + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * WM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (row < p.Ma && col < p.Nb) {
          float v = acc[i][j][r];
          if (has_e) {
            const float al = p.row_alpha ? p.alpha + p.row_alpha[row] : p.alpha;
            v = al * elem_to_f32<false>(__builtin_bit_cast(unsigned short, p.E[(int64_t)row * p.lde + col])) + p.beta * v;
          }
          if (p.diag_out && row == col) {
            p.diag_out[row] = v;
            v = 0.0f;
          }
          // On a diagonal tile only the elements on or above the diagonal are kept, and the
          // strictly-upper ones are mirrored, so the two triangles come from the same register.
          const bool direct = C && (!diag || col >= row);
          const bool mirror = C2 && (!p.symmetric || (diag ? col > row : true));
          const int64_t o1 = (int64_t)row * p.c_rs + (int64_t)col * p.c_cs;
          const int64_t o2 = (int64_t)col * p.c2_rs + (int64_t)row * p.c2_cs;
          if constexpr (ET == kElemF32) {
            if (direct) reinterpret_cast<float*>(p.C)[o1] = v;
            if (mirror) reinterpret_cast<float*>(p.C2)[o2] = v;
          } else {
            const unsigned short h = f32_to_elem<ET == kElemF16>(v);
            if (direct) C[o1] = h;
            if (mirror) C2[o2] = h;
          }
        }
      }
    }
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
static int launch_cfg(GemmArgs a, bool aligned, hipStream_t stream) {
  a.tiles_m = (a.Ma + BM - 1) / BM;
  a.tiles_n = (a.Nb + BN - 1) / BN;
  a.num_tiles = a.symmetric ? a.tiles_m * (a.tiles_m + 1) / 2 : a.tiles_m * a.tiles_n;   // per matrix here
  dim3 grid((unsigned)a.num_tiles, (unsigned)a.batch), block(64 * WAVES_M * WAVES_N);
#define FM_LAUNCH_GENERAL(ET)                                                                              \
  do {                                                                                                    \
    if (aligned)                                                                                          \
      hipLaunchKernelGGL((gemm_nt_kernel<BM, BN, WAVES_M, WAVES_N, true, ET>), grid, block, 0, stream, a);  \
    else                                                                                                  \
      hipLaunchKernelGGL((gemm_nt_kernel<BM, BN, WAVES_M, WAVES_N, false, ET>), grid, block, 0, stream, a); \
  } while (0)
  if (a.elem == kElemF32) FM_LAUNCH_GENERAL(kElemF32);
  else if (a.elem == kElemF16) FM_LAUNCH_GENERAL(kElemF16);
  else FM_LAUNCH_GENERAL(kElemBf16);
#undef FM_LAUNCH_GENERAL
  return (int)hipGetLastError();
}

int launch_gemm_general(GemmArgs a, hipStream_t stream) {
  const int epc = a.elem == kElemF32 ? 4 : 8;   // elements per 16-byte chunk
  const bool aligned = (a.lda % epc == 0) && (a.ldb % epc == 0) && (a.Kc % epc == 0) &&
                       ((reinterpret_cast<uintptr_t>(a.A) & 15) == 0) &&
                       ((reinterpret_cast<uintptr_t>(a.B) & 15) == 0);
  // Large outputs take 256x256 tiles (8 waves, 128x64 per wave); small ones take 128x128 tiles
  // (4 waves, 64x64 per wave) so that more workgroups exist than the chip has CUs.
  const int64_t big_tiles = (int64_t)((a.Ma + 255) / 256) * ((a.Nb + 255) / 256);
  const int64_t work_tiles = (a.symmetric ? (big_tiles + (a.Ma + 255) / 256) / 2 : big_tiles) * a.batch;
  if (work_tiles >= 256) return launch_cfg<256, 256, 2, 4>(a, aligned, stream);
  return launch_cfg<128, 128, 2, 2>(a, aligned, stream);
}

int launch_gemm_nt(GemmArgs a, void* ws, size_t ws_bytes, hipStream_t stream) {
  if (a.batch < 1) a.batch = 1;
  if (gemm_fast_eligible(a)) {
    // a workspace too small for this shape's schedule sends the problem down the slower paths
    const int rc = launch_gemm_fast(a, ws, ws_bytes, stream);
    if (rc != kErrWorkspace) return rc;
  }
  if (gemm_mid_eligible(a) && knob(kKnobNoMid) <= 0) return launch_gemm_mid(a, ws, ws_bytes, stream);
  return launch_gemm_general(a, stream);
}

// ---- knobs and device facts, read once ---------------------------------------------------------
namespace {
struct KnobState {
  std::atomic<long long> v[kKnobCount];
  KnobState() {
    static const char* const names[kKnobCount] = {"FLASHMUON_GRID", "FLASHMUON_KSPLIT", "FLASHMUON_FAST_MIN_UNITS",
                                                  "FLASHMUON_NO_MID", "FLASHMUON_NO_SUB64", "FLASHMUON_HALF",
                                                  "FLASHMUON_DIAG_LAST", "FLASHMUON_NO_TICKETS"};
    for (int i = 0; i < kKnobCount; ++i) {
      const char* e = std::getenv(names[i]);
      v[i].store(e ? std::atoll(e) : -1, std::memory_order_relaxed);
    }
  }
};
KnobState& knob_state() { static KnobState s; return s; }
}  // namespace

long long knob(int which) { return knob_state().v[which].load(std::memory_order_relaxed); }
int set_knob(int which, long long value) {
  if (which < 0 || which >= kKnobCount) return -1;
  knob_state().v[which].store(value, std::memory_order_relaxed);
  return 0;
}

int cu_count() {
  constexpr int kMaxDev = 64;
  static std::atomic<int> cached[kMaxDev];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

}  // namespace fm
