// Internal declarations shared by the translation units of libflashmuon_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

namespace fm {

typedef __bf16 bf16_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

constexpr int kMaxBatch = 32;         // matrices per batched launch
constexpr int kElemBf16 = 0, kElemF16 = 1, kElemF32 = 2;

// what the launch functions return besides hipError_t values (which are >= 0)
constexpr int kErrWorkspace = -2;     // the schedule needs more partial-tile slots than the workspace holds

// Tuning knobs (fm_set_knob, include/flashmuon.h); the FLASHMUON_* environment variables of the same
// names give their initial values, read once when the library is first used.  A negative value
// means "decide automatically".
constexpr int kKnobGrid = 0, kKnobKsplit = 1, kKnobFastMinUnits = 2, kKnobNoMid = 3, kKnobNoSub64 = 4, kKnobHalf = 5, kKnobDiagLast = 6, kKnobNoTickets = 7, kKnobCount = 8;
long long knob(int which);
int set_knob(int which, long long value);
// compute units of the current device (queried once per device)
int cu_count();

// 16-byte chunk c of a 128-byte LDS row r lives at chunk position c ^ swz(r).  Any 8 consecutive
// rows get 8 distinct positions within a 128-byte bank group and any 16 consecutive rows get 16
// distinct positions within 256 bytes, so a ds_read_b128 of one chunk column over 32 rows is
// conflict free.
__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }

// Upper-triangular tile index t (row-major over rows i, columns j >= i) -> (i, j).
__device__ __forceinline__ void tri_decode(int t, int T, int& i, int& j) {
  float fT = (float)(2 * T + 1);
  int ii = (int)((fT - __builtin_sqrtf(fT * fT - 8.0f * (float)t)) * 0.5f);
  if (ii < 0) ii = 0;
  if (ii > T - 1) ii = T - 1;
  // S(i) = number of tiles in rows < i
  while (ii > 0 && (ii * T - (ii * (ii - 1)) / 2) > t) --ii;
  while (ii + 1 < T && ((ii + 1) * T - ((ii + 1) * ii) / 2) <= t) ++ii;
  i = ii;
  j = ii + (t - (ii * T - (ii * (ii - 1)) / 2));
}

// The GEMM kernels exist for two 16-bit element types with the same memory layout; pointers are
// typed bf16_t in both cases and F16 says what the bits mean.
template <bool F16>
__device__ __forceinline__ f32x16_t mfma_32x32x16(bf16x8_t a, bf16x8_t b, f32x16_t c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
// one round-to-nearest-even conversion of an fp32 result to the element type, as its bits
template <bool F16> __device__ __forceinline__ unsigned short f32_to_elem(float v) {
  if constexpr (F16) return __builtin_bit_cast(unsigned short, (_Float16)v);
  else return __builtin_bit_cast(unsigned short, (bf16_t)v);
}
template <bool F16> __device__ __forceinline__ float elem_to_f32(unsigned short h) {
  if constexpr (F16) return (float)__builtin_bit_cast(_Float16, h);
  else return __builtin_bit_cast(float, (uint32_t)h << 16);
}

// Arguments of the one NT contraction every GEMM-shaped kernel here is an instance of:
//     acc[i][j] = sum_k A[i][k] * B[j][k]            (A: Ma x Kc, B: Nb x Kc, k contiguous)
//     v         = E ? (alpha + row_alpha[i]) * E[i][j] + beta * acc : acc   (row_alpha optional)
//     if diag_out and i == j:  diag_out[i] = v (fp32) and v = 0
//     C [i*c_rs  + j*c_cs ] = round(v)               (if C  != nullptr)
//     C2[j*c2_rs + i*c2_cs] = round(v)               (if C2 != nullptr; the mirrored copy)
// A, B, E, C and C2 hold bf16; without E they may hold fp16 or fp32 instead (`elem`; pointers stay
// typed bf16_t, leading dimensions and strides stay in elements).
// With `symmetric` set, A == B, only tiles on or above the diagonal are computed and C2 == C.
struct GemmArgs {
  const bf16_t* A;  int64_t lda;
  const bf16_t* B;  int64_t ldb;
  const bf16_t* E;  int64_t lde;
  const bf16_t* ET; int64_t ldet;   // E transposed (Nb x Ma), optional: the 256x256 path reads the operand through it
  bf16_t* C;  int64_t c_rs, c_cs;
  bf16_t* C2; int64_t c2_rs, c2_cs;
  int Ma, Nb, Kc;
  float alpha, beta;
  const float* row_alpha;   // optional per-row addition to alpha
  float* diag_out;          // optional fp32 copy of the diagonal, which is then stored as zero
  int symmetric;
  int elem;                 // element type of A, B, C, C2: kElemBf16, kElemF16, or kElemF32 (general path only)
  // `batch` independent problems of the same shape in one launch: matrix b of an operand starts
  // b * stride elements after matrix 0 (strides of absent operands are ignored)
  int batch;
  int64_t bs_a, bs_b, bs_e, bs_et, bs_c, bs_c2, bs_ra, bs_do;
  // outputs that are not evenly spaced: when set, matrix b writes to c_list[b] / c2_list[b]
  int use_c_list, use_c2_list;
  bf16_t* c_list[kMaxBatch];
  bf16_t* c2_list[kMaxBatch];
  int tiles_m, tiles_n;   // number of block tiles along each output dimension of one matrix
  int num_tiles;          // tiles actually computed, over the whole batch
  int diag_last;          // 256x256 schedule, one symmetric matrix: its last `diag_last` diagonal tiles end the tile order
};

// the arguments of matrix b of a batch, as a single-matrix problem
__host__ __device__ inline GemmArgs batch_view(const GemmArgs& g, int b) {
  GemmArgs v = g;
  v.A += b * g.bs_a;
  v.B += b * g.bs_b;
  if (v.E) v.E += b * g.bs_e;
  if (v.ET) v.ET += b * g.bs_et;
  if (g.use_c_list) v.C = g.c_list[b]; else if (v.C) v.C += b * g.bs_c;
  if (g.use_c2_list) v.C2 = g.c2_list[b]; else if (v.C2) v.C2 += b * g.bs_c2;
  if (v.row_alpha) v.row_alpha += b * g.bs_ra;
  if (v.diag_out) v.diag_out += b * g.bs_do;
  return v;
}

// Enqueue the contraction described by `args` on `stream`: on the 256x256 path when the shape, the
// alignment and the workspace allow it, on the 128x128 copy-fed path for smaller aligned problems,
// and on the general tiled path otherwise.
// Returns a hipError_t value.
int launch_gemm_nt(GemmArgs args, void* ws, size_t ws_bytes, hipStream_t stream);
int launch_gemm_general(GemmArgs args, hipStream_t stream);
bool gemm_fast_eligible(const GemmArgs& a);
// bytes of fp32 partial tiles the 256x256 path can need for `batch` Ma x Nb outputs, whatever k is
// (0 when no schedule of this shape cuts a tile)
size_t gemm_fast_workspace_bytes(int Ma, int Nb, int batch);
// kErrWorkspace when the schedule needs more than ws holds
int launch_gemm_fast(GemmArgs args, void* ws, size_t ws_bytes, hipStream_t stream);
bool gemm_mid_eligible(const GemmArgs& a);
int launch_gemm_mid(GemmArgs args, void* ws, size_t ws_bytes, hipStream_t stream);

// up to kMaxBatch device pointers, passed to a kernel by value
struct PtrList { void* p[kMaxBatch]; };

// the batched forms take HOST arrays of `batch` device pointers; matrix i reads / writes its own
// slot of the strided arrays (out and sumsq: stride in floats; partials: kSumsqBlocks floats)
int launch_sumsq_batched(const void* const* G, int batch, int dtype, int rows, int cols, int64_t ldg,
                         float* out, int out_stride, float* partials, hipStream_t stream);
int launch_scale_cast_batched(const void* const* G, int batch, int dtype, int rows, int cols, int64_t ldg,
                              const float* sumsq, int sumsq_stride, float eps, bf16_t* const* D, int64_t ldd,
                              bf16_t* const* T, int64_t ldt, hipStream_t stream, int rows_p = 0, int cols_p = 0);
int launch_sumsq(const void* G, int dtype, int rows, int cols, int64_t ldg, float* out,
                 float* partials, hipStream_t stream);
int launch_scale_cast(const void* G, int dtype, int rows, int cols, int64_t ldg,
                      const float* sumsq, float eps, bf16_t* D, int64_t ldd, bf16_t* T, int64_t ldt,
                      hipStream_t stream);
int launch_momentum_nesterov_batched(void* const* g, void* const* buf, int batch, int dtype, int64_t n,
                                     float w_buf, float w_nes, int nesterov, hipStream_t stream);
int launch_weight_update_batched(void* const* p, const bf16_t* const* u, int batch, int p_dtype, int64_t n,
                                 float decay_mul, float alpha, hipStream_t stream);
int launch_copy2d_batched(const bf16_t* src, int64_t lds, int64_t bs_src, bf16_t* const* dst, int64_t ldd,
                          int batch, int rows, int cols, int rows_d, int cols_d, hipStream_t stream);
int launch_momentum_nesterov(void* g, void* buf, int dtype, int64_t n, float w_buf, float w_nes,
                             int nesterov, hipStream_t stream);
int launch_weight_update(void* p, int p_dtype, const bf16_t* u, int64_t n, float decay_mul,
                         float alpha, hipStream_t stream);

// n (at most 64) 64-bit words at p set to zero by a one-block launch
int launch_zero_words(void* p, int n, hipStream_t stream);

constexpr int kSumsqBlocks = 1024;   // partial sums written by the first reduction stage

}  // namespace fm
