// extern "C" entry points of libflashmuon_hip.so: argument validation, workspace carving and the
// Newton-Schulz composition.  No torch types, no allocation, no synchronisation.
#include "../../include/flashmuon.h"
#include "fm_internal.h"
#include <atomic>

using namespace fm;

namespace {

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct Range { uintptr_t lo, hi; };
// byte range of a rows x cols matrix with row stride ld and element size esz
inline Range mat_range(const void* p, int64_t rows, int64_t cols, int64_t ld, int esz) {
  Range r;
  r.lo = reinterpret_cast<uintptr_t>(p);
  r.hi = (rows <= 0 || cols <= 0) ? r.lo : r.lo + (uintptr_t)(((rows - 1) * ld + cols) * esz);
  return r;
}
inline bool overlaps(Range a, Range b) { return a.lo < b.hi && b.lo < a.hi; }
inline bool misaligned(const void* p, int esz) { return (reinterpret_cast<uintptr_t>(p) % esz) != 0; }
inline int dtype_size(int dt) { return dt == FM_F32 ? 4 : 2; }
inline bool bad_dtype(int dt) { return dt != FM_BF16 && dt != FM_F16 && dt != FM_F32; }
inline int hip_status(int rc) { return rc == 0 ? FM_OK : (rc == kErrWorkspace ? FM_ERR_WORKSPACE : FM_ERR_LAUNCH); }
// a workspace is only used when it is 256-byte aligned; otherwise the call runs without one
inline void* usable_ws(void* ws) { return (reinterpret_cast<uintptr_t>(ws) % 256 == 0) ? ws : nullptr; }

// workspace of fm_newtonschulz_batched_bf16, carved in this order; per-matrix arrays are
// batch-major with the strides below
struct NsLayout {
  size_t sumsq, partials, pdiag, x[2], xt[2], a, p, gemm, total;
  size_t pdiag_stride;   // floats between the fp32 diagonals of consecutive matrices
  int M, K;              // the sizes the iteration runs on: those of the matrix, or padded (below)
  bool padded;
};
// A matrix whose sides are not whole 128-tiles would take the general GEMM path in every stage
// (0.5-0.8 times the vendor GEMMs).  Its iterates live in the workspace anyway, so they are kept
// zero-padded to whole tiles instead: zero rows and columns stay zero through every step, and the
// tiled paths run.  Whole 256x256 tiles pay for up to 128 more rows and columns, also where the
// sides are whole multiples of 128 already, once the 256x256 path has enough of them: for a single
// matrix from a short side of 2176 on (five steps at 2176^2 0.43 ms, at 2304^2 0.41; 3200^2 0.96
// and 3328^2 0.78; 5248^2 3.27 and 5376^2 2.61; but 1920^2 0.31 and 2048^2 0.34), for a batch as
// soon as its 256x256 tiles fill the GPU (32 of 1664^2 4.6 ms, of 1792^2 4.2; 2688 x 7168 36 and
// 2816 x 7168 26).  The long side alone goes to a multiple of 256 where the short one is one already
// (32 of 2048 x 5504 15.4 ms, of 2048 x 5632 11.9; one matrix 0.72 and 0.59; below 1536 rows a single
// matrix gains nothing).
constexpr int kPad256From = 2944;       // the stand-alone product: there the copies have to be paid for
static int ns_pad(int n) {
  int p = (n + 127) / 128 * 128;
  if (p >= kPad256From && p % 256 != 0) p += 128;
  return p;
}
NsLayout ns_layout(int batch, int rows, int cols) {
  const int m = rows < cols ? rows : cols, k = rows < cols ? cols : rows;
  const size_t B = (size_t)batch;
  NsLayout l;
  l.M = (m + 127) / 128 * 128;
  l.K = (k + 127) / 128 * 128;
  {
    const int64_t t = (l.M + 255) / 256;
    const bool both = l.M >= 2176 || (l.M >= 1152 && (int64_t)batch * t * (t + 1) / 2 >= 120);
    if (both) l.M = (int)t * 256;
    if (l.M % 256 == 0 && (both || l.M >= 1536 || (batch >= 4 && l.M >= 768))) l.K = (k + 255) / 256 * 256;
  }
  l.padded = l.M != m || l.K != k;
  const size_t M = (size_t)l.M, K = (size_t)l.K;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes, 256); return o; };
  l.sumsq = take(B * 64 * sizeof(float));                 // one float per matrix, 256 bytes apart
  l.partials = take(B * kSumsqBlocks * sizeof(float));
  l.pdiag_stride = align_up(M, 64);
  l.pdiag = take(B * l.pdiag_stride * sizeof(float));
  for (int i = 0; i < 2; ++i) { l.x[i] = take(B * M * K * 2); l.xt[i] = take(B * M * K * 2); }
  l.a = take(B * M * M * 2);
  l.p = take(B * M * M * 2);
  // partial tiles of the three products of a step: two M x M (symmetric) and one M x K, `batch` each
  const size_t g1 = gemm_fast_workspace_bytes(l.M, l.M, batch), g2 = gemm_fast_workspace_bytes(l.M, l.K, batch);
  l.gemm = take(g1 > g2 ? g1 : g2);
  l.total = off;
  return l;
}

// ---- scratch of fm_syrk_bf16_static -------------------------------------------------------------
// 256 partial tiles of 256 KiB: what the 256x256 schedule needs at most when it cuts only the items
// of its last round (more than that only buys a deeper k split of outputs with few tiles, which
// this entry point then does without).  Every GPU the library runs on holds its own copy of the
// array, at its own address, until the process ends.
constexpr size_t kStaticScratchBytes = (size_t)256 * 256 * 256 * sizeof(float);   // 64 MiB
static __device__ __align__(256) unsigned char fm_static_scratch[kStaticScratchBytes];

// device address of the array on the current device, looked up once per device (in host code the
// array's name is only a handle for this lookup, never an address a kernel could use)
int static_scratch(void** out) {
  constexpr int kMaxDev = 64;
  static std::atomic<void*> per_device[kMaxDev];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) return FM_ERR_LAUNCH;
  void* p = per_device[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(fm_static_scratch)) != hipSuccess || !p) return FM_ERR_LAUNCH;
    per_device[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return FM_OK;
}

}  // namespace

extern "C" {

const char* fm_status_string(int status) {
  switch (status) {
    case FM_OK: return "ok";
    case FM_ERR_NULL: return "a required pointer is NULL";
    case FM_ERR_SHAPE: return "invalid or inconsistent dimensions";
    case FM_ERR_STRIDE: return "leading dimension smaller than the row length";
    case FM_ERR_DTYPE: return "unsupported dtype code";
    case FM_ERR_ALIAS: return "an output overlaps an input";
    case FM_ERR_WORKSPACE: return "workspace missing or too small";
    case FM_ERR_LAUNCH: return "kernel launch failed";
    case FM_ERR_ALIGN: return "pointer not aligned to its element size";
    default: return "unknown status";
  }
}

const char* fm_version(void) { return "0.1.0"; }

size_t fm_gemm_workspace_bytes(int rows_out, int cols_out) {
  if (rows_out <= 0 || cols_out <= 0) return 0;
  return gemm_fast_workspace_bytes(rows_out, cols_out, 1);
}

int fm_set_knob(int which, long long value) { return set_knob(which, value) == 0 ? FM_OK : FM_ERR_SHAPE; }

// X * X^T of a matrix whose sides are not whole 128-tiles, through zero-padded copies: X padded in
// the workspace, the product of that on the tiled paths into a padded Y beside it, and the M x M
// part copied out.  Taken from 65536 elements of X on (below that the general path's single launch
// wins); 16-bit elements only.  The tiled paths need whole 128-row tiles and whole 64-wide k stages,
// so a shape that has both is left alone and k is padded to a multiple of 64 only.
struct SyrkPad { int Mp, Kp; size_t x, y, gemm, total; };
constexpr int64_t kSyrkPadMinElems = 256 * 256;
static bool syrk_pad_layout(int M, int K, SyrkPad* p) {
  if (M <= 0 || K <= 0 || (M % 128 == 0 && K % 64 == 0) || (int64_t)M * K < kSyrkPadMinElems) return false;
  p->Mp = ns_pad(M);
  p->Kp = (K + 63) / 64 * 64;
  p->x = 0;
  p->y = align_up((size_t)p->Mp * p->Kp * 2, 256);
  p->gemm = p->y + align_up((size_t)p->Mp * p->Mp * 2, 256);
  p->total = p->gemm + gemm_fast_workspace_bytes(p->Mp, p->Mp, 1);
  return true;
}

size_t fm_syrk_workspace_bytes(int M, int K) {
  if (M <= 0) return 0;
  const size_t plain = gemm_fast_workspace_bytes(M, M, 1);
  SyrkPad p;
  if (!syrk_pad_layout(M, K, &p)) return plain;
  return p.total > plain ? p.total : plain;
}

static int syrk_impl(const void* X, int64_t ldx, void* Y, int64_t ldy_row, int64_t ldy_col, int M, int K,
                     void* ws, size_t ws_bytes, fm_stream_t stream, int elem, bool may_pad = true) {
  if (M < 0 || K < 0) return FM_ERR_SHAPE;
  if (M == 0) return FM_OK;
  if (!X && K > 0) return FM_ERR_NULL;
  if (!Y) return FM_ERR_NULL;
  if (ldx < K) return FM_ERR_STRIDE;
  if (ldy_row == 0 || ldy_col == 0) return FM_ERR_STRIDE;
  if (M > 1) {
    // distinct (i, j) must not share an address: the larger stride has to step over a whole line
    // of the smaller one (true of every dense or padded row- or column-major layout)
    const int64_t ar = ldy_row < 0 ? -ldy_row : ldy_row, ac = ldy_col < 0 ? -ldy_col : ldy_col;
    const int64_t lo = ar < ac ? ar : ac, hi = ar < ac ? ac : ar;
    if (hi < (int64_t)M * lo) return FM_ERR_STRIDE;
  }
  const int es = elem == kElemF32 ? 4 : 2;
  if (misaligned(X, es) || misaligned(Y, es)) return FM_ERR_ALIGN;
  {   // Y must not overlap X: every tile of Y is written while other tiles still read X
    const int64_t ar = ldy_row < 0 ? -ldy_row : ldy_row, ac = ldy_col < 0 ? -ldy_col : ldy_col;
    const int64_t back = (ldy_row < 0 ? (M - 1) * ar : 0) + (ldy_col < 0 ? (M - 1) * ac : 0);
    Range y;
    y.lo = reinterpret_cast<uintptr_t>(Y) - (uintptr_t)(back * es);
    y.hi = y.lo + (uintptr_t)(((M - 1) * (ar + ac) + 1) * es);
    if (K > 0 && overlaps(mat_range(X, M, K, ldx, es), y)) return FM_ERR_ALIAS;
  }
  hipStream_t hs = static_cast<hipStream_t>(stream);
  GemmArgs a = {};
  a.E = nullptr; a.lde = 0;
  a.alpha = 0.0f; a.beta = 1.0f; a.symmetric = 1; a.elem = elem;
  SyrkPad p;
  // Y is symmetric, so a unit stride in either direction makes its lines rows for the copy out
  const int64_t ldy = ldy_col == 1 ? ldy_row : ldy_row == 1 ? ldy_col : 0;
  if (may_pad && elem != kElemF32 && ldy >= M && usable_ws(ws) && syrk_pad_layout(M, K, &p) && ws_bytes >= p.total &&
      !overlaps(mat_range(X, M, K, ldx, es), Range{reinterpret_cast<uintptr_t>(ws), reinterpret_cast<uintptr_t>(ws) + p.total}) &&
      !overlaps(mat_range(Y, M, M, ldy, es), Range{reinterpret_cast<uintptr_t>(ws), reinterpret_cast<uintptr_t>(ws) + p.total})) {
    unsigned char* w = static_cast<unsigned char*>(ws);
    bf16_t* Xp = reinterpret_cast<bf16_t*>(w + p.x);
    bf16_t* Yp = reinterpret_cast<bf16_t*>(w + p.y);
    bf16_t* xl[1] = {Xp};
    bf16_t* yl[1] = {static_cast<bf16_t*>(Y)};
    if (launch_copy2d_batched(static_cast<const bf16_t*>(X), ldx, 0, xl, p.Kp, 1, M, K, p.Mp, p.Kp, hs)) return FM_ERR_LAUNCH;
    a.A = a.B = Xp; a.lda = a.ldb = p.Kp;
    a.C = a.C2 = Yp; a.c_rs = a.c2_rs = p.Mp; a.c_cs = a.c2_cs = 1;
    a.Ma = a.Nb = p.Mp; a.Kc = p.Kp;
    if (launch_gemm_nt(a, w + p.gemm, ws_bytes - p.gemm, hs)) return FM_ERR_LAUNCH;
    return hip_status(launch_copy2d_batched(Yp, p.Mp, 0, yl, ldy, 1, M, M, M, M, hs));
  }
  a.A = a.B = static_cast<const bf16_t*>(X); a.lda = a.ldb = ldx;
  a.C = a.C2 = static_cast<bf16_t*>(Y);
  a.c_rs = a.c2_rs = ldy_row; a.c_cs = a.c2_cs = ldy_col;
  a.Ma = a.Nb = M; a.Kc = K;
  return hip_status(launch_gemm_nt(a, usable_ws(ws), ws_bytes, hs));
}

int fm_syrk_bf16(const void* X, int64_t ldx, void* Y, int64_t ldy_row, int64_t ldy_col, int M, int K,
                 void* ws, size_t ws_bytes, fm_stream_t stream) {
  return syrk_impl(X, ldx, Y, ldy_row, ldy_col, M, K, ws, ws_bytes, stream, kElemBf16);
}

int fm_syrk_bf16_static(const void* X, int64_t ldx, void* Y, int64_t ldy_row, int64_t ldy_col, int M, int K,
                        fm_stream_t stream) {
  if (M > FM_STATIC_MAX_M || K > FM_STATIC_MAX_K) return FM_ERR_SHAPE;
  void* scratch = nullptr;
  const int rc = static_scratch(&scratch);
  if (rc != FM_OK) return rc;
  // the schedules, and the bits, of fm_syrk_bf16 given a workspace of these 64 MiB (no padded copies)
  return syrk_impl(X, ldx, Y, ldy_row, ldy_col, M, K, scratch, kStaticScratchBytes, stream, kElemBf16, false);
}

int fm_syrk_f16(const void* X, int64_t ldx, void* Y, int64_t ldy_row, int64_t ldy_col, int M, int K,
                void* ws, size_t ws_bytes, fm_stream_t stream) {
  return syrk_impl(X, ldx, Y, ldy_row, ldy_col, M, K, ws, ws_bytes, stream, kElemF16);
}

int fm_syrk_f32(const void* X, int64_t ldx, void* Y, int64_t ldy_row, int64_t ldy_col, int M, int K,
                void* ws, size_t ws_bytes, fm_stream_t stream) {
  return syrk_impl(X, ldx, Y, ldy_row, ldy_col, M, K, ws, ws_bytes, stream, kElemF32);
}

int fm_syrk_poly_bf16(const void* A, int64_t lda, void* P, int64_t ldp, int M, float b, float c,
                      float* diag_out, void* ws, size_t ws_bytes, fm_stream_t stream) {
  if (M < 0) return FM_ERR_SHAPE;
  if (M == 0) return FM_OK;
  if (!A || !P) return FM_ERR_NULL;
  if (lda < M || ldp < M) return FM_ERR_STRIDE;
  if (misaligned(A, 2) || misaligned(P, 2) || misaligned(diag_out, 4)) return FM_ERR_ALIGN;
  if (overlaps(mat_range(A, M, M, lda, 2), mat_range(P, M, M, ldp, 2))) return FM_ERR_ALIAS;
  if (diag_out && (overlaps(mat_range(diag_out, 1, M, M, 4), mat_range(A, M, M, lda, 2)) ||
                   overlaps(mat_range(diag_out, 1, M, M, 4), mat_range(P, M, M, ldp, 2))))
    return FM_ERR_ALIAS;
  GemmArgs a = {};
  a.A = a.B = a.E = a.ET = static_cast<const bf16_t*>(A); a.lda = a.ldb = a.lde = a.ldet = lda;   // A is symmetric
  a.C = a.C2 = static_cast<bf16_t*>(P);
  a.c_rs = a.c2_rs = ldp; a.c_cs = a.c2_cs = 1;
  a.Ma = a.Nb = a.Kc = M;
  a.alpha = b; a.beta = c; a.symmetric = 1;
  a.diag_out = diag_out;
  return hip_status(launch_gemm_nt(a, usable_ws(ws), ws_bytes, static_cast<hipStream_t>(stream)));
}

int fm_gemm_axpby_bf16(const void* P, int64_t ldp, const void* XT, int64_t ldxt, const void* X,
                       int64_t ldx, void* Xout, int64_t ldo, void* XoutT, int64_t ldot, int M, int K,
                       float alpha, const float* row_alpha, void* ws, size_t ws_bytes,
                       fm_stream_t stream) {
  if (M < 0 || K < 0) return FM_ERR_SHAPE;
  if (M == 0 || K == 0) return FM_OK;
  if (!P || !XT || !X) return FM_ERR_NULL;
  if (!Xout && !XoutT) return FM_ERR_NULL;
  if (ldp < M || ldxt < M || ldx < K) return FM_ERR_STRIDE;
  if ((Xout && ldo < K) || (XoutT && ldot < M)) return FM_ERR_STRIDE;
  if (misaligned(P, 2) || misaligned(XT, 2) || misaligned(X, 2) || misaligned(Xout, 2) ||
      misaligned(XoutT, 2) || misaligned(row_alpha, 4))
    return FM_ERR_ALIGN;
  const Range in[3] = {mat_range(P, M, M, ldp, 2), mat_range(XT, K, M, ldxt, 2),
                       mat_range(X, M, K, ldx, 2)};
  const Range o1 = mat_range(Xout, M, K, ldo, 2), o2 = mat_range(XoutT, K, M, ldot, 2);
  for (int i = 0; i < 3; ++i) {
    if (Xout && overlaps(in[i], o1)) return FM_ERR_ALIAS;
    if (XoutT && overlaps(in[i], o2)) return FM_ERR_ALIAS;
  }
  if (Xout && XoutT && overlaps(o1, o2)) return FM_ERR_ALIAS;
  GemmArgs a = {};
  a.A = static_cast<const bf16_t*>(P); a.lda = ldp;
  a.B = static_cast<const bf16_t*>(XT); a.ldb = ldxt;
  a.E = static_cast<const bf16_t*>(X); a.lde = ldx;
  a.ET = a.B; a.ldet = ldxt;
  a.C = static_cast<bf16_t*>(Xout); a.c_rs = ldo; a.c_cs = 1;
  a.C2 = static_cast<bf16_t*>(XoutT); a.c2_rs = ldot; a.c2_cs = 1;
  a.Ma = M; a.Nb = K; a.Kc = M;
  a.alpha = alpha; a.beta = 1.0f; a.symmetric = 0;
  a.row_alpha = row_alpha;
  return hip_status(launch_gemm_nt(a, usable_ws(ws), ws_bytes, static_cast<hipStream_t>(stream)));
}

size_t fm_sumsq_workspace_bytes(void) { return kSumsqBlocks * sizeof(float); }

int fm_sumsq(const void* G, int dtype, int rows, int cols, int64_t ldg, float* out, void* ws,
             size_t ws_bytes, fm_stream_t stream) {
  if (bad_dtype(dtype)) return FM_ERR_DTYPE;
  if (rows < 0 || cols < 0) return FM_ERR_SHAPE;
  if (!out) return FM_ERR_NULL;
  if (!G && (int64_t)rows * cols > 0) return FM_ERR_NULL;
  if (ldg < cols) return FM_ERR_STRIDE;
  if (!ws || ws_bytes < fm_sumsq_workspace_bytes()) return FM_ERR_WORKSPACE;
  if (misaligned(G, dtype_size(dtype)) || misaligned(out, 4) || misaligned(ws, 4)) return FM_ERR_ALIGN;
  return hip_status(launch_sumsq(G, dtype, rows, cols, ldg, out, static_cast<float*>(ws),
                                 static_cast<hipStream_t>(stream)));
}

int fm_scale_cast_bf16(const void* G, int dtype, int rows, int cols, int64_t ldg, const float* sumsq,
                       float eps, void* D, int64_t ldd, void* T, int64_t ldt, fm_stream_t stream) {
  if (bad_dtype(dtype)) return FM_ERR_DTYPE;
  if (rows < 0 || cols < 0) return FM_ERR_SHAPE;
  if (rows == 0 || cols == 0) return FM_OK;
  if (!G || !sumsq) return FM_ERR_NULL;
  if (!D && !T) return FM_ERR_NULL;
  if (ldg < cols || (D && ldd < cols) || (T && ldt < rows)) return FM_ERR_STRIDE;
  if (misaligned(G, dtype_size(dtype)) || misaligned(D, 2) || misaligned(T, 2) || misaligned(sumsq, 4))
    return FM_ERR_ALIGN;
  const Range g = mat_range(G, rows, cols, ldg, dtype_size(dtype));
  if (D && overlaps(g, mat_range(D, rows, cols, ldd, 2))) return FM_ERR_ALIAS;
  if (T && overlaps(g, mat_range(T, cols, rows, ldt, 2))) return FM_ERR_ALIAS;
  return hip_status(launch_scale_cast(G, dtype, rows, cols, ldg, sumsq, eps, static_cast<bf16_t*>(D),
                                      ldd, static_cast<bf16_t*>(T), ldt,
                                      static_cast<hipStream_t>(stream)));
}

size_t fm_newtonschulz_batched_workspace_bytes(int batch, int rows, int cols) {
  if (batch <= 0 || rows <= 0 || cols <= 0) return 0;
  return ns_layout(batch, rows, cols).total;
}

size_t fm_newtonschulz_workspace_bytes(int rows, int cols) {
  return fm_newtonschulz_batched_workspace_bytes(1, rows, cols);
}

int fm_newtonschulz_batched_bf16(const void* const* G, int dtype, int batch, int rows, int cols,
                                 int64_t ldg, void* const* out, int64_t ldout, int steps, float a,
                                 float b, float c, float eps, void* ws, size_t ws_bytes,
                                 fm_stream_t stream) {
  if (bad_dtype(dtype)) return FM_ERR_DTYPE;
  if (rows < 0 || cols < 0 || steps < 0 || batch < 0 || batch > kMaxBatch) return FM_ERR_SHAPE;
  if (rows == 0 || cols == 0 || batch == 0) return FM_OK;
  if (!G || !out) return FM_ERR_NULL;
  if (ldg < cols || ldout < cols) return FM_ERR_STRIDE;
  for (int i = 0; i < batch; ++i) {
    if (!G[i] || !out[i]) return FM_ERR_NULL;
    if (misaligned(G[i], dtype_size(dtype)) || misaligned(out[i], 2)) return FM_ERR_ALIGN;
    const Range oi = mat_range(out[i], rows, cols, ldout, 2);
    for (int j = 0; j < batch; ++j) {
      if (overlaps(mat_range(G[j], rows, cols, ldg, dtype_size(dtype)), oi)) return FM_ERR_ALIAS;
      if (j != i && overlaps(mat_range(out[j], rows, cols, ldout, 2), oi)) return FM_ERR_ALIAS;
    }
  }
  const NsLayout l = ns_layout(batch, rows, cols);
  if (!ws || ws_bytes < l.total) return FM_ERR_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(ws) % 256 != 0) return FM_ERR_ALIGN;
  {
    Range w;
    w.lo = reinterpret_cast<uintptr_t>(ws);
    w.hi = w.lo + l.total;
    for (int i = 0; i < batch; ++i)
      if (overlaps(mat_range(G[i], rows, cols, ldg, dtype_size(dtype)), w) ||
          overlaps(mat_range(out[i], rows, cols, ldout, 2), w))
        return FM_ERR_ALIAS;
  }

  unsigned char* w = static_cast<unsigned char*>(ws);
  void* gws = w + l.gemm;
  const size_t gws_bytes = l.total - l.gemm;
  hipStream_t hs = static_cast<hipStream_t>(stream);
  // the last 256 bytes of the GEMM scratch hold the ticket word of the sub-tile rounds: whatever the
  // caller's memory held there could pass for a launch number no launch ever reaches (the products
  // would still be right, on the fixed assignment of sub-tiles), so it starts from zero
  if (steps > 0 && gws_bytes >= 256 && launch_zero_words(w + l.total - 256, 32, hs)) return FM_ERR_LAUNCH;
  const bool tall = rows > cols;
  const bool padded = l.padded && steps > 0;
  const int M = padded ? l.M : (tall ? cols : rows), K = padded ? l.K : (tall ? rows : cols);
  const int64_t mk = (int64_t)M * K, mm = (int64_t)M * M;

  // The iteration runs on X (M x K) with M <= K.  G is X when it is wide and X^T when it is
  // tall, so the scaled cast of G is X in one case and X^T in the other.
  bf16_t* X = reinterpret_cast<bf16_t*>(w + l.x[0]);
  bf16_t* XT = reinterpret_cast<bf16_t*>(w + l.xt[0]);
  {
    // Frobenius norms, then the scaled bf16 cast in both orientations: one launch each for the batch
    float* sumsq = reinterpret_cast<float*>(w + l.sumsq);
    float* partials = reinterpret_cast<float*>(w + l.partials);
    for (int i = 0; i < batch; ++i)
      if (misaligned(G[i], dtype_size(dtype))) return FM_ERR_ALIGN;
    if (launch_sumsq_batched(G, batch, dtype, rows, cols, ldg, sumsq, 64, partials, hs)) return FM_ERR_LAUNCH;
    bf16_t* d[kMaxBatch];
    bf16_t* t[kMaxBatch];
    for (int i = 0; i < batch; ++i) {
      if (steps == 0) { d[i] = static_cast<bf16_t*>(out[i]); t[i] = nullptr; }
      else if (!tall) { d[i] = X + i * mk; t[i] = XT + i * mk; }
      else            { d[i] = XT + i * mk; t[i] = X + i * mk; }
    }
    const int64_t ldd = steps == 0 ? ldout : (!tall ? K : M), ldt = !tall ? M : K;
    // with padding: G's orientation is (tall ? K x M : M x K) there, and what lies beyond G is zeroed
    if (launch_scale_cast_batched(G, batch, dtype, rows, cols, ldg, sumsq, 64, eps, d, ldd,
                                  steps == 0 ? nullptr : t, ldt, hs, padded ? (tall ? K : M) : rows,
                                  padded ? (tall ? M : K) : cols))
      return FM_ERR_LAUNCH;
  }
  if (steps == 0) return FM_OK;

  bf16_t* A = reinterpret_cast<bf16_t*>(w + l.a);
  bf16_t* P = reinterpret_cast<bf16_t*>(w + l.p);
  float* pdiag = reinterpret_cast<float*>(w + l.pdiag);   // diagonal of P, kept in fp32
  for (int s = 0; s < steps; ++s) {
    const bool last = s + 1 == steps;
    bf16_t* Xn = reinterpret_cast<bf16_t*>(w + l.x[(s + 1) & 1]);
    bf16_t* XTn = reinterpret_cast<bf16_t*>(w + l.xt[(s + 1) & 1]);
    GemmArgs g = {};
    // A = X X^T
    g.A = g.B = X; g.lda = g.ldb = K; g.bs_a = g.bs_b = mk;
    g.C = g.C2 = A; g.c_rs = g.c2_rs = M; g.c_cs = g.c2_cs = 1; g.bs_c = g.bs_c2 = mm;
    g.Ma = g.Nb = M; g.Kc = K; g.beta = 1.0f; g.symmetric = 1; g.batch = batch;
    if (launch_gemm_nt(g, gws, gws_bytes, hs)) return FM_ERR_LAUNCH;
    // P = b A + c A A, diagonal in fp32
    g = GemmArgs{};
    g.A = g.B = g.E = g.ET = A; g.lda = g.ldb = g.lde = g.ldet = M;
    g.bs_a = g.bs_b = g.bs_e = g.bs_et = mm;
    g.C = g.C2 = P; g.c_rs = g.c2_rs = M; g.c_cs = g.c2_cs = 1; g.bs_c = g.bs_c2 = mm;
    g.Ma = g.Nb = g.Kc = M; g.alpha = b; g.beta = c; g.symmetric = 1; g.batch = batch;
    g.diag_out = pdiag; g.bs_do = (int64_t)l.pdiag_stride;
    if (launch_gemm_nt(g, gws, gws_bytes, hs)) return FM_ERR_LAUNCH;
    // X' = (a + diag) X + P X, and its transpose; the last step writes the caller's orientation only
    g = GemmArgs{};
    g.A = P; g.lda = M; g.bs_a = mm;
    g.B = XT; g.ldb = M; g.bs_b = mk;
    g.E = X; g.lde = K; g.bs_e = mk;
    g.ET = XT; g.ldet = M; g.bs_et = mk;
    g.Ma = M; g.Nb = K; g.Kc = M; g.alpha = a; g.beta = 1.0f; g.symmetric = 0; g.batch = batch;
    g.row_alpha = pdiag; g.bs_ra = (int64_t)l.pdiag_stride;
    g.c_cs = g.c2_cs = 1;
    if (!last) {
      g.C = Xn; g.c_rs = K; g.bs_c = mk;
      g.C2 = XTn; g.c2_rs = M; g.bs_c2 = mk;
    } else if (padded) {  // the orientation the caller wants, into the workspace, and from there out
      if (!tall) { g.C = Xn; g.c_rs = K; g.bs_c = mk; }
      else { g.C2 = XTn; g.c2_rs = M; g.bs_c2 = mk; }
    } else if (!tall) {   // the result has G's shape: X itself
      g.C = static_cast<bf16_t*>(out[0]); g.c_rs = ldout; g.use_c_list = 1;
      for (int i = 0; i < batch; ++i) g.c_list[i] = static_cast<bf16_t*>(out[i]);
    } else {              // or its transpose
      g.C2 = static_cast<bf16_t*>(out[0]); g.c2_rs = ldout; g.use_c2_list = 1;
      for (int i = 0; i < batch; ++i) g.c2_list[i] = static_cast<bf16_t*>(out[i]);
    }
    if (launch_gemm_nt(g, gws, gws_bytes, hs)) return FM_ERR_LAUNCH;
    X = Xn; XT = XTn;
  }
  if (padded) {
    bf16_t* o[kMaxBatch];
    for (int i = 0; i < batch; ++i) o[i] = static_cast<bf16_t*>(out[i]);
    if (launch_copy2d_batched(tall ? XT : X, tall ? M : K, mk, o, ldout, batch, rows, cols, rows, cols, hs))
      return FM_ERR_LAUNCH;
  }
  return FM_OK;
}

int fm_newtonschulz_bf16(const void* G, int dtype, int rows, int cols, int64_t ldg, void* out,
                         int64_t ldout, int steps, float a, float b, float c, float eps, void* ws,
                         size_t ws_bytes, fm_stream_t stream) {
  const void* gs[1] = {G};
  void* os[1] = {out};
  if (rows > 0 && cols > 0 && (!G || !out)) return FM_ERR_NULL;
  return fm_newtonschulz_batched_bf16(gs, dtype, 1, rows, cols, ldg, os, ldout, steps, a, b, c, eps,
                                      ws, ws_bytes, stream);
}

int fm_momentum_nesterov(void* g, void* buf, int dtype, int64_t n, float w_buf, float w_nes,
                         int nesterov, fm_stream_t stream) {
  if (bad_dtype(dtype)) return FM_ERR_DTYPE;
  if (n < 0) return FM_ERR_SHAPE;
  if (n == 0) return FM_OK;
  if (!g || !buf) return FM_ERR_NULL;
  const int esz = dtype_size(dtype);
  if (misaligned(g, esz) || misaligned(buf, esz)) return FM_ERR_ALIGN;
  if (overlaps(mat_range(g, 1, n, n, esz), mat_range(buf, 1, n, n, esz))) return FM_ERR_ALIAS;
  return hip_status(launch_momentum_nesterov(g, buf, dtype, n, w_buf, w_nes, nesterov,
                                             static_cast<hipStream_t>(stream)));
}

int fm_momentum_nesterov_batched(void* const* g, void* const* buf, int batch, int dtype, int64_t n,
                                 float w_buf, float w_nes, int nesterov, fm_stream_t stream) {
  if (bad_dtype(dtype)) return FM_ERR_DTYPE;
  if (n < 0 || batch < 0 || batch > kMaxBatch) return FM_ERR_SHAPE;
  if (n == 0 || batch == 0) return FM_OK;
  if (!g || !buf) return FM_ERR_NULL;
  const int esz = dtype_size(dtype);
  for (int i = 0; i < batch; ++i) {
    if (!g[i] || !buf[i]) return FM_ERR_NULL;
    if (misaligned(g[i], esz) || misaligned(buf[i], esz)) return FM_ERR_ALIGN;
    for (int j = 0; j < batch; ++j) {
      if (overlaps(mat_range(g[i], 1, n, n, esz), mat_range(buf[j], 1, n, n, esz))) return FM_ERR_ALIAS;
      if (j != i && (overlaps(mat_range(g[i], 1, n, n, esz), mat_range(g[j], 1, n, n, esz)) ||
                     overlaps(mat_range(buf[i], 1, n, n, esz), mat_range(buf[j], 1, n, n, esz))))
        return FM_ERR_ALIAS;
    }
  }
  return hip_status(launch_momentum_nesterov_batched(g, buf, batch, dtype, n, w_buf, w_nes, nesterov,
                                                     static_cast<hipStream_t>(stream)));
}

int fm_weight_update_batched(void* const* p, int p_dtype, const void* const* u_bf16, int batch, int64_t n,
                             float decay_mul, float alpha, fm_stream_t stream) {
  if (bad_dtype(p_dtype)) return FM_ERR_DTYPE;
  if (n < 0 || batch < 0 || batch > kMaxBatch) return FM_ERR_SHAPE;
  if (n == 0 || batch == 0) return FM_OK;
  if (!p || !u_bf16) return FM_ERR_NULL;
  const int esz = dtype_size(p_dtype);
  for (int i = 0; i < batch; ++i) {
    if (!p[i] || !u_bf16[i]) return FM_ERR_NULL;
    if (misaligned(p[i], esz) || misaligned(u_bf16[i], 2)) return FM_ERR_ALIGN;
    for (int j = 0; j < batch; ++j) {
      if (overlaps(mat_range(p[i], 1, n, n, esz), mat_range(u_bf16[j], 1, n, n, 2))) return FM_ERR_ALIAS;
      if (j != i && overlaps(mat_range(p[i], 1, n, n, esz), mat_range(p[j], 1, n, n, esz))) return FM_ERR_ALIAS;
    }
  }
  return hip_status(launch_weight_update_batched(p, reinterpret_cast<const bf16_t* const*>(u_bf16), batch,
                                                 p_dtype, n, decay_mul, alpha,
                                                 static_cast<hipStream_t>(stream)));
}

int fm_weight_update(void* p, int p_dtype, const void* u_bf16, int64_t n, float decay_mul,
                     float alpha, fm_stream_t stream) {
  if (bad_dtype(p_dtype)) return FM_ERR_DTYPE;
  if (n < 0) return FM_ERR_SHAPE;
  if (n == 0) return FM_OK;
  if (!p || !u_bf16) return FM_ERR_NULL;
  const int esz = dtype_size(p_dtype);
  if (misaligned(p, esz) || misaligned(u_bf16, 2)) return FM_ERR_ALIGN;
  if (overlaps(mat_range(p, 1, n, n, esz), mat_range(u_bf16, 1, n, n, 2))) return FM_ERR_ALIAS;
  return hip_status(launch_weight_update(p, p_dtype, static_cast<const bf16_t*>(u_bf16), n,
                                         decay_mul, alpha, static_cast<hipStream_t>(stream)));
}

}  // extern "C"
