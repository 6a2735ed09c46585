// HBM-bound kernels of the Muon step for gfx950: sum of squares, normalise + cast (+ transpose),
// momentum / Nesterov update and the decayed weight update.  All are streaming kernels with
// 16-byte accesses per lane on the aligned path and a scalar path for everything else.
#include "fm_internal.h"

namespace fm {

// ---- element access by dtype code -------------------------------------------------------------
template <int DT> struct Elem;
template <> struct Elem<0> {  // bf16
  typedef unsigned short raw;
  static __device__ __forceinline__ float ld(raw v) { return (float)__builtin_bit_cast(bf16_t, v); }
  static __device__ __forceinline__ raw st(float f) { return __builtin_bit_cast(raw, (bf16_t)f); }
};
template <> struct Elem<1> {  // fp16
  typedef unsigned short raw;
  static __device__ __forceinline__ float ld(raw v) { return (float)__builtin_bit_cast(_Float16, v); }
  static __device__ __forceinline__ raw st(float f) { return __builtin_bit_cast(raw, (_Float16)f); }
};
template <> struct Elem<2> {  // fp32
  typedef float raw;
  static __device__ __forceinline__ float ld(raw v) { return v; }
  static __device__ __forceinline__ raw st(float f) { return f; }
};

// value of an input element after the `.bfloat16()` cast the reference applies first
template <int DT>
__device__ __forceinline__ float as_bf16_value(typename Elem<DT>::raw v) {
  return (float)(bf16_t)Elem<DT>::ld(v);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Block-wide sum with a fixed tree: lanes by xor-shuffle, then waves in index order.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red /* NT/64 floats of LDS */) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.0f;
#pragma unroll
  for (int w = 0; w < NT / 64; ++w) s += red[w];
  __syncthreads();
  return s;
}

// ---- sum of squares -----------------------------------------------------------------------------
// blockIdx.y is the matrix of a batch: its pointer comes from the list, its partial sums go to its
// own run of gridDim.x floats
template <int DT, bool FLAT_VEC>
__global__ __launch_bounds__(256) void sumsq_partial_kernel(PtrList Gl, int rows, int cols,
                                                            int64_t ldg, float* partials) {
  typedef typename Elem<DT>::raw raw;
  __shared__ float red[4];
  const void* Gv = Gl.p[blockIdx.y];
  partials += (size_t)blockIdx.y * gridDim.x;
  const raw* G = reinterpret_cast<const raw*>(Gv);
  const int64_t n = (int64_t)rows * cols;
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  if (FLAT_VEC) {
    // contiguous, 16-byte aligned, n a multiple of the vector width
    constexpr int V = 16 / sizeof(raw);
    const int64_t nv = n / V;
    const uint4* G4 = reinterpret_cast<const uint4*>(Gv);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nv; i += (int64_t)gridDim.x * 256) {
      union { uint4 v; raw e[V]; } u;
      u.v = G4[i];
#pragma unroll
      for (int e = 0; e < V; e += 4) {
        float a = as_bf16_value<DT>(u.e[e]), b = as_bf16_value<DT>(u.e[e + 1]);
        float c = as_bf16_value<DT>(u.e[e + 2]), d = as_bf16_value<DT>(u.e[e + 3]);
        s0 += a * a; s1 += b * b; s2 += c * c; s3 += d * d;
      }
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
      int64_t r = i / cols, c = i - r * cols;
      float a = as_bf16_value<DT>(G[r * ldg + c]);
      s0 += a * a;
    }
  }
  float s = block_sum<256>((s0 + s1) + (s2 + s3), red);
  if (threadIdx.x == 0) partials[blockIdx.x] = s;
}

// one block per matrix: its n partial sums, its own output slot
__global__ __launch_bounds__(256) void sumsq_final_kernel(const float* partials, int n, float* out,
                                                          int out_stride) {
  __shared__ float red[4];
  partials += (size_t)blockIdx.x * n;
  out += (size_t)blockIdx.x * out_stride;
  float s = 0.0f;
  for (int i = threadIdx.x; i < n; i += 256) s += partials[i];
  s = block_sum<256>(s, red);
  if (threadIdx.x == 0) out[0] = s;
}

int launch_sumsq_batched(const void* const* G, int batch, int dtype, int rows, int cols, int64_t ldg,
                         float* out, int out_stride, float* partials, hipStream_t stream) {
  const int64_t n = (int64_t)rows * cols;
  const int esz = dtype == 2 ? 4 : 2;
  bool flat = (ldg == cols) && (n % (16 / esz) == 0);
  PtrList gl = {};
  for (int i = 0; i < batch; ++i) {
    gl.p[i] = const_cast<void*>(G[i]);
    flat = flat && ((reinterpret_cast<uintptr_t>(G[i]) & 15) == 0);
  }
  dim3 grid(kSumsqBlocks, (unsigned)batch), block(256);
#define FM_SUMSQ(DT)                                                                               \
  if (flat) hipLaunchKernelGGL((sumsq_partial_kernel<DT, true>), grid, block, 0, stream, gl, rows, \
                               cols, ldg, partials);                                               \
  else hipLaunchKernelGGL((sumsq_partial_kernel<DT, false>), grid, block, 0, stream, gl, rows,     \
                          cols, ldg, partials);
  if (dtype == 0) { FM_SUMSQ(0) } else if (dtype == 1) { FM_SUMSQ(1) } else { FM_SUMSQ(2) }
#undef FM_SUMSQ
  hipLaunchKernelGGL(sumsq_final_kernel, dim3((unsigned)batch), dim3(256), 0, stream,
                     (const float*)partials, kSumsqBlocks, out, out_stride);
  return (int)hipGetLastError();
}

int launch_sumsq(const void* G, int dtype, int rows, int cols, int64_t ldg, float* out,
                 float* partials, hipStream_t stream) {
  return launch_sumsq_batched(&G, 1, dtype, rows, cols, ldg, out, 0, partials, stream);
}

// 16-byte accesses of data that is touched once per call: marked non-temporal, so that the stream
// does not push anything else out of the caches
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ld_stream(const void* p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return uint4{v.x, v.y, v.z, v.w};
}
__device__ __forceinline__ void st_stream(void* p, uint4 v) {
  const u32x4_t w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<u32x4_t*>(p));
}

// ---- normalise, cast, transpose -----------------------------------------------------------------
// One 64x64 tile of G per block: D gets the tile in place, T gets it transposed through LDS.
// D is rows_p x cols_p and T cols_p x rows_p with rows_p >= rows, cols_p >= cols: what lies beyond
// G in them is written as zero.
// blockIdx.z is the matrix of a batch (pointers from the lists, sums of squares sumsq_stride apart).
template <int DT>
__global__ __launch_bounds__(256) void scale_cast_kernel(PtrList Gl, int rows, int cols, int rows_p, int cols_p,
                                                         int64_t ldg, const float* sumsq, int sumsq_stride,
                                                         float eps, PtrList Dl, int64_t ldd,
                                                         PtrList Tl, int64_t ldt,
                                                         int g_vec, int d_vec, int t_vec) {
  typedef typename Elem<DT>::raw raw;
  constexpr int PITCH = 66;   // u16 per LDS row: 33 dwords, so column reads spread over the banks
  __shared__ unsigned short tile[64 * PITCH];
  const raw* G = reinterpret_cast<const raw*>(Gl.p[blockIdx.z]);
  unsigned short* D = reinterpret_cast<unsigned short*>(Dl.p[blockIdx.z]);
  unsigned short* T = reinterpret_cast<unsigned short*>(Tl.p[blockIdx.z]);
  const float denom = __builtin_sqrtf(sumsq[(size_t)blockIdx.z * sumsq_stride]) + eps;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tid = threadIdx.x;
  const int ch = tid & 7;   // 8-element chunk along the contiguous dimension

#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int lr = pass * 32 + (tid >> 3);
    const int r = r0 + lr, c = c0 + ch * 8;
    unsigned short o[8];
    if (r < rows) {
      const raw* src = G + (int64_t)r * ldg + c;
      if (g_vec && c + 8 <= cols) {
        union { uint4 v[sizeof(raw) / 2]; raw e[8]; } u;
#pragma unroll
        for (int q = 0; q < (int)sizeof(raw) / 2; ++q) u.v[q] = reinterpret_cast<const uint4*>(src)[q];
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = Elem<0>::st(as_bf16_value<DT>(u.e[e]) / denom);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          o[e] = (c + e < cols) ? Elem<0>::st(as_bf16_value<DT>(src[e]) / denom) : (unsigned short)0;
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = 0;
    }
    if (D && r < rows_p) {
      unsigned short* dst = D + (int64_t)r * ldd + c;
      if (d_vec && c + 8 <= cols_p) {
        union { uint4 v; unsigned short h[8]; } w;
#pragma unroll
        for (int e = 0; e < 8; ++e) w.h[e] = o[e];
        *reinterpret_cast<uint4*>(dst) = w.v;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) if (c + e < cols_p) dst[e] = o[e];
      }
    }
    if (T) {
#pragma unroll
      for (int e = 0; e < 8; ++e) tile[lr * PITCH + ch * 8 + e] = o[e];
    }
  }
  if (!T) return;
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int lc = pass * 32 + (tid >> 3);   // column of G = row of T
    const int c = c0 + lc, r = r0 + ch * 8;
    if (c < cols_p) {
      unsigned short* dst = T + (int64_t)c * ldt + r;
      union { uint4 v; unsigned short h[8]; } w;
#pragma unroll
      for (int e = 0; e < 8; ++e) w.h[e] = tile[(ch * 8 + e) * PITCH + lc];
      if (t_vec && r + 8 <= rows_p) {
        *reinterpret_cast<uint4*>(dst) = w.v;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) if (r + e < rows_p) dst[e] = w.h[e];
      }
    }
  }
}

// The same for whole 128x128 tiles of 16-byte aligned matrices with nothing to pad: a lane moves 8
// columns of two rows at a time (256 contiguous bytes of G, D and T per 16 lanes), and the tile
// goes through LDS as 32-bit words (rows 2 p and 2 p + 1 of one column), so that a row of T leaves
// in 16-byte reads: word p of column c sits at word p ^ 4 (c / 8 % 16) of the column's 64, which
// keeps both the writes of a wave (16 column chunks x 4 row pairs) and its reads (16 consecutive
// groups of a column) on 64 different banks.
template <int DT>
__global__ __launch_bounds__(256) void scale_cast_tile128_kernel(PtrList Gl, int64_t ldg, const float* sumsq,
                                                                 int sumsq_stride, float eps, PtrList Dl, int64_t ldd,
                                                                 PtrList Tl, int64_t ldt) {
  typedef typename Elem<DT>::raw raw;
  __shared__ __align__(16) uint32_t tile[128 * 64];
  const raw* G = reinterpret_cast<const raw*>(Gl.p[blockIdx.z]) + (int64_t)blockIdx.y * 128 * ldg + blockIdx.x * 128;
  unsigned short* D = reinterpret_cast<unsigned short*>(Dl.p[blockIdx.z]) + (int64_t)blockIdx.y * 128 * ldd + blockIdx.x * 128;
  unsigned short* T = reinterpret_cast<unsigned short*>(Tl.p[blockIdx.z]) + (int64_t)blockIdx.x * 128 * ldt + blockIdx.y * 128;
  const float denom = __builtin_sqrtf(sumsq[(size_t)blockIdx.z * sumsq_stride]) + eps;
  const int tid = threadIdx.x;
  const int ch = tid & 15;   // 8-element chunk along the contiguous dimension
  constexpr int NV = sizeof(raw) / 2;   // 16-byte loads per 8 elements

  union In { uint4 v[NV]; raw e[8]; };
  In in[4][2];
#pragma unroll
  for (int pass = 0; pass < 4; ++pass)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const raw* src = G + (int64_t)(2 * (pass * 16 + (tid >> 4)) + h) * ldg + ch * 8;
#pragma unroll
      for (int q = 0; q < NV; ++q) in[pass][h].v[q] = reinterpret_cast<const uint4*>(src)[q];
    }
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int rp = pass * 16 + (tid >> 4);   // rows 2 rp and 2 rp + 1 of the tile
    union { uint4 v; unsigned short h[8]; uint32_t w[4]; } o[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int e = 0; e < 8; ++e) o[h].h[e] = Elem<0>::st(as_bf16_value<DT>(in[pass][h].e[e]) / denom);
      *reinterpret_cast<uint4*>(D + (int64_t)(2 * rp + h) * ldd + ch * 8) = o[h].v;
    }
    uint32_t* const col = tile + (ch * 8) * 64 + (rp ^ (4 * ch));   // columns 8 ch .. + 7 share ch = column / 8 % 16
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      col[(2 * e) * 64] = __builtin_amdgcn_perm(o[1].w[e], o[0].w[e], 0x05040100u);       // column 8 ch + 2 e: row 2 rp | row 2 rp + 1
      col[(2 * e + 1) * 64] = __builtin_amdgcn_perm(o[1].w[e], o[0].w[e], 0x07060302u);   // column 8 ch + 2 e + 1
    }
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    const int c = pass * 16 + (tid >> 4);   // column of G = row of T; its rows 8 ch .. + 7 of the tile
    const uint4 v = *reinterpret_cast<const uint4*>(tile + c * 64 + 4 * (ch ^ ((c >> 3) & 15)));
    *reinterpret_cast<uint4*>(T + (int64_t)c * ldt + ch * 8) = v;
  }
}

int launch_scale_cast_batched(const void* const* G, int batch, int dtype, int rows, int cols, int64_t ldg,
                              const float* sumsq, int sumsq_stride, float eps, bf16_t* const* D, int64_t ldd,
                              bf16_t* const* T, int64_t ldt, hipStream_t stream, int rows_p, int cols_p) {
  if (rows_p < rows) rows_p = rows;
  if (cols_p < cols) cols_p = cols;
  const int esz = dtype == 2 ? 4 : 2;
  int gv = (ldg * esz) % 16 == 0, dv = D != nullptr && ldd % 8 == 0, tv = T != nullptr && ldt % 8 == 0;
  PtrList gl = {}, dl = {}, tl = {};
  for (int i = 0; i < batch; ++i) {
    gl.p[i] = const_cast<void*>(G[i]);
    gv = gv && (reinterpret_cast<uintptr_t>(G[i]) & 15) == 0;
    if (D) { dl.p[i] = D[i]; dv = dv && (reinterpret_cast<uintptr_t>(D[i]) & 15) == 0; }
    if (T) { tl.p[i] = T[i]; tv = tv && (reinterpret_cast<uintptr_t>(T[i]) & 15) == 0; }
  }
  if (D && T && gv && dv && tv && rows_p == rows && cols_p == cols && rows % 128 == 0 && cols % 128 == 0) {
    dim3 grid128((unsigned)(cols / 128), (unsigned)(rows / 128), (unsigned)batch);
#define FM_SCALE128(DT) hipLaunchKernelGGL(scale_cast_tile128_kernel<DT>, grid128, dim3(256), 0, stream, gl, ldg, sumsq, \
                                           sumsq_stride, eps, dl, ldd, tl, ldt)
    if (dtype == 0) FM_SCALE128(0);
    else if (dtype == 1) FM_SCALE128(1);
    else FM_SCALE128(2);
#undef FM_SCALE128
    return (int)hipGetLastError();
  }
  dim3 grid((unsigned)((cols_p + 63) / 64), (unsigned)((rows_p + 63) / 64), (unsigned)batch), block(256);
#define FM_SCALE(DT) hipLaunchKernelGGL(scale_cast_kernel<DT>, grid, block, 0, stream, gl, rows, cols, rows_p, cols_p, ldg, \
                                        sumsq, sumsq_stride, eps, dl, ldd, tl, ldt, gv, dv, tv)
  if (dtype == 0) FM_SCALE(0);
  else if (dtype == 1) FM_SCALE(1);
  else FM_SCALE(2);
#undef FM_SCALE
  return (int)hipGetLastError();
}

int launch_scale_cast(const void* G, int dtype, int rows, int cols, int64_t ldg,
                      const float* sumsq, float eps, bf16_t* D, int64_t ldd, bf16_t* T, int64_t ldt,
                      hipStream_t stream) {
  return launch_scale_cast_batched(&G, 1, dtype, rows, cols, ldg, sumsq, 0, eps, D ? &D : nullptr, ldd,
                                   T ? &T : nullptr, ldt, stream, rows, cols);
}

// ---- a few zero words (a fill launch rather than hipMemsetAsync, so that callers can be captured) ---
__global__ void zero_words_kernel(unsigned long long* p, int n) {
  if ((int)threadIdx.x < n) p[threadIdx.x] = 0ull;
}
int launch_zero_words(void* p, int n, hipStream_t stream) {
  hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(64), 0, stream, static_cast<unsigned long long*>(p), n < 64 ? n : 64);
  return (int)hipGetLastError();
}

// ---- momentum + Nesterov ------------------------------------------------------------------------
__device__ __forceinline__ float lerp_torch(float s, float e, float w) {
  // the two-branch form torch's lerp uses (weights below 0.5 interpolate from the start point)
  return (__builtin_fabsf(w) < 0.5f) ? s + w * (e - s) : e - (e - s) * (1.0f - w);
}

template <int DT>
__device__ __forceinline__ void momentum_one(typename Elem<DT>::raw& g, typename Elem<DT>::raw& b,
                                             float w_buf, float w_nes, int nesterov) {
  float gf = Elem<DT>::ld(g), bf = Elem<DT>::ld(b);
  b = Elem<DT>::st(lerp_torch(bf, gf, w_buf));
  if (nesterov) g = Elem<DT>::st(lerp_torch(gf, Elem<DT>::ld(b), w_nes));
}

// blockIdx.y is the tensor of a batch
template <int DT>
__global__ __launch_bounds__(256) void momentum_kernel(PtrList gl, PtrList bl, int64_t n, float w_buf,
                                                       float w_nes, int nesterov, int vec) {
  void* gv = gl.p[blockIdx.y];
  void* bv = bl.p[blockIdx.y];
  typedef typename Elem<DT>::raw raw;
  constexpr int V = 16 / sizeof(raw);
  raw* g = reinterpret_cast<raw*>(gv);
  raw* b = reinterpret_cast<raw*>(bv);
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int64_t done = 0;
  if (vec) {
    const int64_t nv = n / V;
    uint4* g4 = reinterpret_cast<uint4*>(gv);
    uint4* b4 = reinterpret_cast<uint4*>(bv);
    for (int64_t i = t; i < nv; i += stride) {
      union { uint4 v; raw e[V]; } ug, ub;
      ug.v = ld_stream(g4 + i); ub.v = ld_stream(b4 + i);
#pragma unroll
      for (int e = 0; e < V; ++e) momentum_one<DT>(ug.e[e], ub.e[e], w_buf, w_nes, nesterov);
      st_stream(b4 + i, ub.v);
      if (nesterov) st_stream(g4 + i, ug.v);
    }
    done = nv * V;
  }
  for (int64_t i = done + t; i < n; i += stride) momentum_one<DT>(g[i], b[i], w_buf, w_nes, nesterov);
}

static inline unsigned stream_grid(int64_t n_vec) {
  // one 16-byte unit per thread: a grid capped at 32 blocks per CU, whose threads stride over the
  // rest, sweeps a tensor in several interleaved passes and measured 12 % slower on 45 M elements
  // (2080 against 1850 us for the momentum of 32 such tensors)
  int64_t blocks = (n_vec + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > (1 << 22)) blocks = 1 << 22;   // the loop strides over what is left
  return (unsigned)blocks;
}

int launch_momentum_nesterov_batched(void* const* g, void* const* buf, int batch, int dtype, int64_t n,
                                     float w_buf, float w_nes, int nesterov, hipStream_t stream) {
  int vec = 1;
  PtrList gl = {}, bl = {};
  for (int i = 0; i < batch; ++i) {
    gl.p[i] = g[i]; bl.p[i] = buf[i];
    vec = vec && ((reinterpret_cast<uintptr_t>(g[i]) & 15) == 0) && ((reinterpret_cast<uintptr_t>(buf[i]) & 15) == 0);
  }
  const int V = dtype == 2 ? 4 : 8;
  dim3 grid(stream_grid((n + V - 1) / V), (unsigned)batch), block(256);
  if (dtype == 0) hipLaunchKernelGGL(momentum_kernel<0>, grid, block, 0, stream, gl, bl, n, w_buf, w_nes, nesterov, vec);
  else if (dtype == 1) hipLaunchKernelGGL(momentum_kernel<1>, grid, block, 0, stream, gl, bl, n, w_buf, w_nes, nesterov, vec);
  else hipLaunchKernelGGL(momentum_kernel<2>, grid, block, 0, stream, gl, bl, n, w_buf, w_nes, nesterov, vec);
  return (int)hipGetLastError();
}

int launch_momentum_nesterov(void* g, void* buf, int dtype, int64_t n, float w_buf, float w_nes,
                             int nesterov, hipStream_t stream) {
  return launch_momentum_nesterov_batched(&g, &buf, 1, dtype, n, w_buf, w_nes, nesterov, stream);
}

// ---- weight update ------------------------------------------------------------------------------
// blockIdx.y is the tensor of a batch
template <int DT>
__global__ __launch_bounds__(256) void weight_update_kernel(PtrList pl, PtrList ul,
                                                            int64_t n, float decay_mul, float alpha,
                                                            int vec) {
  typedef typename Elem<DT>::raw raw;
  void* pv = pl.p[blockIdx.y];
  const unsigned short* u = reinterpret_cast<const unsigned short*>(ul.p[blockIdx.y]);
  raw* p = reinterpret_cast<raw*>(pv);
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int64_t done = 0;
  if (vec) {
    // 8 elements per lane: 16 bytes of u, 16 (or 32) bytes of p
    const int64_t nv = n / 8;
    for (int64_t i = t; i < nv; i += stride) {
      union { uint4 v; unsigned short h[8]; } uu;
      union { uint4 v[sizeof(raw) / 2]; raw e[8]; } up;
      uu.v = ld_stream(reinterpret_cast<const uint4*>(u) + i);
#pragma unroll
      for (int q = 0; q < (int)sizeof(raw) / 2; ++q) up.v[q] = ld_stream(reinterpret_cast<uint4*>(pv) + i * (sizeof(raw) / 2) + q);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float pf = Elem<DT>::ld(Elem<DT>::st(Elem<DT>::ld(up.e[e]) * decay_mul));
        up.e[e] = Elem<DT>::st(pf + alpha * Elem<0>::ld(uu.h[e]));
      }
#pragma unroll
      for (int q = 0; q < (int)sizeof(raw) / 2; ++q) st_stream(reinterpret_cast<uint4*>(pv) + i * (sizeof(raw) / 2) + q, up.v[q]);
    }
    done = nv * 8;
  }
  for (int64_t i = done + t; i < n; i += stride) {
    float pf = Elem<DT>::ld(Elem<DT>::st(Elem<DT>::ld(p[i]) * decay_mul));
    p[i] = Elem<DT>::st(pf + alpha * Elem<0>::ld(u[i]));
  }
}

int launch_weight_update_batched(void* const* p, const bf16_t* const* u, int batch, int p_dtype, int64_t n,
                                 float decay_mul, float alpha, hipStream_t stream) {
  int vec = 1;
  PtrList pl = {}, ul = {};
  for (int i = 0; i < batch; ++i) {
    pl.p[i] = p[i]; ul.p[i] = const_cast<bf16_t*>(u[i]);
    vec = vec && ((reinterpret_cast<uintptr_t>(p[i]) & 15) == 0) && ((reinterpret_cast<uintptr_t>(u[i]) & 15) == 0);
  }
  dim3 grid(stream_grid((n + 7) / 8), (unsigned)batch), block(256);
  if (p_dtype == 0) hipLaunchKernelGGL(weight_update_kernel<0>, grid, block, 0, stream, pl, ul, n, decay_mul, alpha, vec);
  else if (p_dtype == 1) hipLaunchKernelGGL(weight_update_kernel<1>, grid, block, 0, stream, pl, ul, n, decay_mul, alpha, vec);
  else hipLaunchKernelGGL(weight_update_kernel<2>, grid, block, 0, stream, pl, ul, n, decay_mul, alpha, vec);
  return (int)hipGetLastError();
}

int launch_weight_update(void* p, int p_dtype, const bf16_t* u, int64_t n, float decay_mul,
                         float alpha, hipStream_t stream) {
  return launch_weight_update_batched(&p, &u, 1, p_dtype, n, decay_mul, alpha, stream);
}

// ---- 2-D copy with zero padding, for the whole-tile copies of matrices whose sides are not ---------
// dst[b] (rows_d x cols_d, pitch ldd) = src[b] (rows x cols at src + b * bs_src, pitch lds) where
// that exists and zero elsewhere, 16-bit elements.  A lane moves 8 consecutive elements of a row, as
// one 16-byte access on a side that is aligned for it (`src_vec`, `dst_vec`) and element by element
// otherwise; blockIdx.y strides over the rows, blockIdx.z is the matrix.
__global__ __launch_bounds__(256) void copy2d_kernel(const unsigned short* src, int64_t lds, int64_t bs_src,
                                                     PtrList dl, int64_t ldd, int rows, int cols, int rows_d,
                                                     int cols_d, int src_vec, int dst_vec) {
  const int c0 = ((int)blockIdx.x * 256 + (int)threadIdx.x) * 8;
  if (c0 >= cols_d) return;
  for (int r = (int)blockIdx.y; r < rows_d; r += (int)gridDim.y) {
    union { uint4 v; unsigned short e[8]; } u;
    u.v = uint4{0u, 0u, 0u, 0u};
    if (r < rows) {
      const unsigned short* s = src + (int64_t)blockIdx.z * bs_src + (int64_t)r * lds + c0;
      if (src_vec && c0 + 8 <= cols) {
        u.v = *reinterpret_cast<const uint4*>(s);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (c0 + e < cols) u.e[e] = s[e];
      }
    }
    unsigned short* d = reinterpret_cast<unsigned short*>(dl.p[blockIdx.z]) + (int64_t)r * ldd + c0;
    if (dst_vec && c0 + 8 <= cols_d) {
      *reinterpret_cast<uint4*>(d) = u.v;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (c0 + e < cols_d) d[e] = u.e[e];
    }
  }
}

int launch_copy2d_batched(const bf16_t* src, int64_t lds, int64_t bs_src, bf16_t* const* dst, int64_t ldd,
                          int batch, int rows, int cols, int rows_d, int cols_d, hipStream_t stream) {
  if (batch <= 0 || rows_d <= 0 || cols_d <= 0) return 0;
  const int src_vec = lds % 8 == 0 && bs_src % 8 == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0;
  int dst_vec = ldd % 8 == 0;
  PtrList dl = {};
  for (int i = 0; i < batch; ++i) {
    dl.p[i] = dst[i];
    dst_vec = dst_vec && (reinterpret_cast<uintptr_t>(dst[i]) & 15) == 0;
  }
  dim3 grid((unsigned)((cols_d + 2047) / 2048), (unsigned)(rows_d < 65535 ? rows_d : 65535), (unsigned)batch);
  hipLaunchKernelGGL(copy2d_kernel, grid, dim3(256), 0, stream, reinterpret_cast<const unsigned short*>(src), lds, bs_src,
                     dl, ldd, rows, cols, rows_d, cols_d, src_vec, dst_vec);
  return (int)hipGetLastError();
}

}  // namespace fm
