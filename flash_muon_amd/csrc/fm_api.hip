// extern "C" entry points of libflashmuon_hip.so: argument validation, workspace carving and the
// Newton-Schulz composition.  No torch types, no allocation, no synchronisation.
#include "../../include/flashmuon.h"
#include "fm_internal.h"

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
inline int hip_status(int hip_err) { return hip_err == 0 ? FM_OK : FM_ERR_LAUNCH; }
// a workspace is only used when it is 256-byte aligned; otherwise the call runs without one
inline void* usable_ws(void* ws) { return (reinterpret_cast<uintptr_t>(ws) % 256 == 0) ? ws : nullptr; }

// workspace of fm_newtonschulz_bf16, carved in this order
struct NsLayout {
  size_t sumsq, partials, pdiag, x[2], xt[2], a, p, gemm, total;
};
NsLayout ns_layout(int rows, int cols) {
  const size_t M = (size_t)(rows < cols ? rows : cols), K = (size_t)(rows < cols ? cols : rows);
  NsLayout l;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes, 256); return o; };
  l.sumsq = take(sizeof(float));
  l.partials = take(kSumsqBlocks * sizeof(float));
  l.pdiag = take(M * sizeof(float));
  for (int i = 0; i < 2; ++i) { l.x[i] = take(M * K * 2); l.xt[i] = take(M * K * 2); }
  l.a = take(M * M * 2);
  l.p = take(M * M * 2);
  l.gemm = take(fm_gemm_workspace_bytes((int)M, (int)K));
  l.total = off;
  return l;
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
  return gemm_fast_workspace_bytes(rows_out, cols_out, false);
}

int fm_syrk_bf16(const void* X, int64_t ldx, void* Y, int64_t ldy_row, int64_t ldy_col, int M, int K,
                 void* ws, size_t ws_bytes, fm_stream_t stream) {
  if (M < 0 || K < 0) return FM_ERR_SHAPE;
  if (M == 0) return FM_OK;
  if (!X && K > 0) return FM_ERR_NULL;
  if (!Y) return FM_ERR_NULL;
  if (ldx < K) return FM_ERR_STRIDE;
  if (ldy_row == 0 || ldy_col == 0) return FM_ERR_STRIDE;
  if (misaligned(X, 2) || misaligned(Y, 2)) return FM_ERR_ALIGN;
  GemmArgs a = {};
  a.A = a.B = static_cast<const bf16_t*>(X); a.lda = a.ldb = ldx;
  a.E = nullptr; a.lde = 0;
  a.C = a.C2 = static_cast<bf16_t*>(Y);
  a.c_rs = a.c2_rs = ldy_row; a.c_cs = a.c2_cs = ldy_col;
  a.Ma = a.Nb = M; a.Kc = K;
  a.alpha = 0.0f; a.beta = 1.0f; a.symmetric = 1;
  return hip_status(launch_gemm_nt(a, usable_ws(ws), ws_bytes, static_cast<hipStream_t>(stream)));
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
  a.A = a.B = a.E = a.ET = static_cast<const bf16_t*>(A); a.lda = a.ldb = a.lde = a.ldet = lda;
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

size_t fm_newtonschulz_workspace_bytes(int rows, int cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return ns_layout(rows, cols).total;
}

int fm_newtonschulz_bf16(const void* G, int dtype, int rows, int cols, int64_t ldg, void* out,
                         int64_t ldout, int steps, float a, float b, float c, float eps, void* ws,
                         size_t ws_bytes, fm_stream_t stream) {
  if (bad_dtype(dtype)) return FM_ERR_DTYPE;
  if (rows < 0 || cols < 0 || steps < 0) return FM_ERR_SHAPE;
  if (rows == 0 || cols == 0) return FM_OK;
  if (!G || !out) return FM_ERR_NULL;
  if (ldg < cols || ldout < cols) return FM_ERR_STRIDE;
  if (misaligned(G, dtype_size(dtype)) || misaligned(out, 2)) return FM_ERR_ALIGN;
  if (overlaps(mat_range(G, rows, cols, ldg, dtype_size(dtype)), mat_range(out, rows, cols, ldout, 2)))
    return FM_ERR_ALIAS;
  const NsLayout l = ns_layout(rows, cols);
  if (!ws || ws_bytes < l.total) return FM_ERR_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(ws) % 256 != 0) return FM_ERR_ALIGN;

  unsigned char* w = static_cast<unsigned char*>(ws);
  float* sumsq = reinterpret_cast<float*>(w + l.sumsq);
  void* partials = w + l.partials;
  void* gws = w + l.gemm;
  const size_t gws_bytes = l.total - l.gemm;
  const bool tall = rows > cols;
  const int M = tall ? cols : rows, K = tall ? rows : cols;

  int st = fm_sumsq(G, dtype, rows, cols, ldg, sumsq, partials, fm_sumsq_workspace_bytes(), stream);
  if (st) return st;

  // The iteration runs on X (M x K) with M <= K.  G is X when it is wide and X^T when it is
  // tall, so the scaled cast of G is X in one case and X^T in the other.
  void* X = w + l.x[0];
  void* XT = w + l.xt[0];
  if (steps == 0) return fm_scale_cast_bf16(G, dtype, rows, cols, ldg, sumsq, eps, out, ldout, nullptr, 0, stream);
  if (!tall) st = fm_scale_cast_bf16(G, dtype, rows, cols, ldg, sumsq, eps, X, K, XT, M, stream);
  else       st = fm_scale_cast_bf16(G, dtype, rows, cols, ldg, sumsq, eps, XT, M, X, K, stream);
  if (st) return st;

  void* A = w + l.a;
  void* P = w + l.p;
  float* pdiag = reinterpret_cast<float*>(w + l.pdiag);   // diagonal of P, kept in fp32
  for (int s = 0; s < steps; ++s) {
    const bool last = s + 1 == steps;
    st = fm_syrk_bf16(X, K, A, M, 1, M, K, gws, gws_bytes, stream);
    if (st) return st;
    st = fm_syrk_poly_bf16(A, M, P, M, M, b, c, pdiag, gws, gws_bytes, stream);
    if (st) return st;
    void* Xn = w + l.x[(s + 1) & 1];
    void* XTn = w + l.xt[(s + 1) & 1];
    if (!last)
      st = fm_gemm_axpby_bf16(P, M, XT, M, X, K, Xn, K, XTn, M, M, K, a, pdiag, gws, gws_bytes, stream);
    else if (!tall)   // the result has G's shape: X itself
      st = fm_gemm_axpby_bf16(P, M, XT, M, X, K, out, ldout, nullptr, 0, M, K, a, pdiag, gws, gws_bytes, stream);
    else              // or its transpose
      st = fm_gemm_axpby_bf16(P, M, XT, M, X, K, nullptr, 0, out, ldout, M, K, a, pdiag, gws, gws_bytes, stream);
    if (st) return st;
    X = Xn; XT = XTn;
  }
  return FM_OK;
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
