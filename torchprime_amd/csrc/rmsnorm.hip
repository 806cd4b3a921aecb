// RMSNorm forward / backward for gfx950.  HBM-bound: one wavefront owns one row, the row is read
// once with 16-byte loads and kept in registers between the reduction and the scale.
//
// Semantics follow LlamaRMSNorm.forward (torchprime/torch_xla_models/model/llama/model.py:46-52;
// same body at model/mixtral/model.py:53-59 and model/deepseek_v3/model.py:38-44):
//   h = x.float(); var = mean(h*h, -1); h = h * rsqrt(var + eps); return weight * h.to(x.dtype)
// i.e. the normalised value is rounded to the input dtype BEFORE the weight multiply.
#include "common.hpp"

namespace tp {

constexpr int RMS_MAX_PARTS = 1024;  // partial dw rows written by the backward

static inline int rms_parts(int64_t rows) {
  int64_t p = (rows + 3) / 4;
  return (int)(p < RMS_MAX_PARTS ? p : RMS_MAX_PARTS);
}

// ------------------------------------------------------------------------------------------------
// forward, vector path: NV 16-byte vectors of x per lane
// ------------------------------------------------------------------------------------------------
template <typename XT, typename WT, typename OT, int NV>
__global__ __launch_bounds__(256) void rmsnorm_fwd_vec(const XT* __restrict__ x, const WT* __restrict__ w,
                                                       OT* __restrict__ y, float* __restrict__ rstd,
                                                       int64_t rows, int hidden, int64_t xs, int64_t ys,
                                                       float eps) {
  constexpr int E = 16 / sizeof(XT);
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int nvec = hidden / E;
  const XT* xr = x + row * xs;
  OT* yr = y + row * ys;

  float xv[NV][E];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int v = lane + 64 * i;
    if (v < nvec) {
      load_f<XT, E>(xr + (int64_t)v * E, xv[i]);
#pragma unroll
      for (int e = 0; e < E; e++) ss += xv[i][e] * xv[i][e];
    }
  }
  ss = wave_sum(ss);
  const float r = rsqrtf(ss / (float)hidden + eps);
  if (lane == 0) rstd[row] = r;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int v = lane + 64 * i;
    if (v < nvec) {
      float wv[E], o[E];
      load_f<WT, E>(w + (int64_t)v * E, wv);
#pragma unroll
      for (int e = 0; e < E; e++) o[e] = wv[e] * round_to<XT>(xv[i][e] * r);
      store_f<OT, E>(yr + (int64_t)v * E, o);
    }
  }
}

// forward, any hidden / alignment: two passes over the row with scalar accesses
template <typename XT, typename WT, typename OT>
__global__ __launch_bounds__(256) void rmsnorm_fwd_generic(const XT* __restrict__ x, const WT* __restrict__ w,
                                                           OT* __restrict__ y, float* __restrict__ rstd,
                                                           int64_t rows, int hidden, int64_t xs, int64_t ys,
                                                           float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const XT* xr = x + row * xs;
  OT* yr = y + row * ys;
  float ss = 0.f;
  for (int c = lane; c < hidden; c += 64) {
    const float f = Elem<XT>::to_f(xr[c]);
    ss += f * f;
  }
  ss = wave_sum(ss);
  const float r = rsqrtf(ss / (float)hidden + eps);
  if (lane == 0) rstd[row] = r;
  for (int c = lane; c < hidden; c += 64)
    yr[c] = Elem<OT>::from_f(Elem<WT>::to_f(w[c]) * round_to<XT>(Elem<XT>::to_f(xr[c]) * r));
}

// ------------------------------------------------------------------------------------------------
// backward, vector path.  Each wave walks rows gw, gw+nw, ...; dw partial sums stay in registers
// and are folded over the block's four waves through LDS, one partial row per block.
// ------------------------------------------------------------------------------------------------
template <typename XT, typename WT, typename OT, int NV>
__global__ __launch_bounds__(256) void rmsnorm_bwd_vec(const OT* __restrict__ dy, const XT* __restrict__ x,
                                                       const WT* __restrict__ w, const float* __restrict__ rstd,
                                                       XT* __restrict__ dx, float* __restrict__ ws, int64_t rows,
                                                       int hidden, int64_t dys, int64_t xs, int64_t dxs) {
  constexpr int E = 16 / sizeof(XT);
  extern __shared__ float red[];  // hidden floats
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nvec = hidden / E;
  const int64_t gw = (int64_t)blockIdx.x * 4 + wave, nw = (int64_t)gridDim.x * 4;
  const float inv_h = 1.f / (float)hidden;

  float wv[NV][E], wacc[NV][E];
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int v = lane + 64 * i;
#pragma unroll
    for (int e = 0; e < E; e++) { wacc[i][e] = 0.f; wv[i][e] = 0.f; }
    if (v < nvec) load_f<WT, E>(w + (int64_t)v * E, wv[i]);
  }
  for (int64_t row = gw; row < rows; row += nw) {
    const float r = rstd[row];
    const XT* xr = x + row * xs;
    const OT* gr = dy + row * dys;
    XT* dr = dx + row * dxs;
    float n[NV][E], g[NV][E];
    float c = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int v = lane + 64 * i;
      if (v < nvec) {
        float dyv[E];
        load_f<XT, E>(xr + (int64_t)v * E, n[i]);
        load_f<OT, E>(gr + (int64_t)v * E, dyv);
#pragma unroll
        for (int e = 0; e < E; e++) {
          n[i][e] *= r;
          g[i][e] = dyv[e] * wv[i][e];
          c += g[i][e] * n[i][e];
          wacc[i][e] += dyv[e] * round_to<XT>(n[i][e]);
        }
      }
    }
    c = wave_sum(c) * inv_h;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int v = lane + 64 * i;
      if (v < nvec) {
        float o[E];
#pragma unroll
        for (int e = 0; e < E; e++) o[e] = r * (g[i][e] - n[i][e] * c);
        store_f<XT, E>(dr + (int64_t)v * E, o);
      }
    }
  }
  // fold the four waves in a fixed order
  for (int k = 0; k < 4; k++) {
    if (wave == k) {
#pragma unroll
      for (int i = 0; i < NV; i++) {
        const int v = lane + 64 * i;
        if (v < nvec) {
#pragma unroll
          for (int e = 0; e < E; e++) {
            if (k == 0) red[v * E + e] = wacc[i][e];
            else red[v * E + e] += wacc[i][e];
          }
        }
      }
    }
    __syncthreads();
  }
  float* out = ws + (int64_t)blockIdx.x * hidden;
  for (int c = threadIdx.x; c < hidden; c += 256) out[c] = red[c];
}

// backward dx, any hidden / alignment
template <typename XT, typename WT, typename OT>
__global__ __launch_bounds__(256) void rmsnorm_bwd_dx_generic(const OT* __restrict__ dy, const XT* __restrict__ x,
                                                              const WT* __restrict__ w, const float* __restrict__ rstd,
                                                              XT* __restrict__ dx, int64_t rows, int hidden,
                                                              int64_t dys, int64_t xs, int64_t dxs) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float r = rstd[row];
  const XT* xr = x + row * xs;
  const OT* gr = dy + row * dys;
  XT* dr = dx + row * dxs;
  float c = 0.f;
  for (int j = lane; j < hidden; j += 64)
    c += Elem<OT>::to_f(gr[j]) * Elem<WT>::to_f(w[j]) * (Elem<XT>::to_f(xr[j]) * r);
  c = wave_sum(c) / (float)hidden;
  for (int j = lane; j < hidden; j += 64) {
    const float n = Elem<XT>::to_f(xr[j]) * r;
    const float g = Elem<OT>::to_f(gr[j]) * Elem<WT>::to_f(w[j]);
    dr[j] = Elem<XT>::from_f(r * (g - n * c));
  }
}
// backward dw partials, any hidden: thread = column, rows p, p+P, ...
template <typename XT, typename OT>
__global__ __launch_bounds__(256) void rmsnorm_bwd_dw_generic(const OT* __restrict__ dy, const XT* __restrict__ x,
                                                              const float* __restrict__ rstd, float* __restrict__ ws,
                                                              int64_t rows, int hidden, int64_t dys, int64_t xs) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= hidden) return;
  float acc = 0.f;
  for (int64_t row = blockIdx.y; row < rows; row += gridDim.y)
    acc += Elem<OT>::to_f(dy[row * dys + c]) * round_to<XT>(Elem<XT>::to_f(x[row * xs + c]) * rstd[row]);
  ws[(int64_t)blockIdx.y * hidden + c] = acc;
}

// dw[c] = sum_p ws[p, c], fixed order
template <typename WT>
__global__ __launch_bounds__(256) void rmsnorm_dw_reduce(const float* __restrict__ ws, WT* __restrict__ dw, int parts,
                                                         int hidden) {
  __shared__ float red[256];
  const int c = blockIdx.x * 64 + (threadIdx.x & 63);
  const int g = threadIdx.x >> 6;
  float acc = 0.f;
  if (c < hidden) {
#pragma unroll 8
    for (int p = g; p < parts; p += 4) acc += ws[(int64_t)p * hidden + c];
  }
  red[threadIdx.x] = acc;
  __syncthreads();
  if (g == 0 && c < hidden) {
    const float s = ((red[threadIdx.x] + red[threadIdx.x + 64]) + red[threadIdx.x + 128]) + red[threadIdx.x + 192];
    dw[c] = Elem<WT>::from_f(s);
  }
}

// ------------------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------------------
template <typename XT, typename WT, typename OT>
static int fwd_typed(const void* x, const void* w, void* y, float* rstd, int64_t rows, int hidden, int64_t xs,
                     int64_t ys, float eps, hipStream_t st) {
  constexpr int E = 16 / sizeof(XT);
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  const XT* xp = (const XT*)x; const WT* wp = (const WT*)w; OT* yp = (OT*)y;
  const bool vec = hidden % E == 0 && aligned16(x) && aligned16(w) && aligned16(y) && (xs * sizeof(XT)) % 16 == 0 &&
                   (ys * sizeof(OT)) % 16 == 0 && hidden / E <= 64 * 32;
  if (vec) {
    const int per = (hidden / E + 63) / 64;
#define TP_RMS_FWD(NV) rmsnorm_fwd_vec<XT, WT, OT, NV><<<grid, block, 0, st>>>(xp, wp, yp, rstd, rows, hidden, xs, ys, eps)
    if (per <= 1) TP_RMS_FWD(1);
    else if (per <= 2) TP_RMS_FWD(2);
    else if (per <= 4) TP_RMS_FWD(4);
    else if (per <= 8) TP_RMS_FWD(8);
    else if (per <= 16) TP_RMS_FWD(16);
    else TP_RMS_FWD(32);
#undef TP_RMS_FWD
  } else {
    rmsnorm_fwd_generic<XT, WT, OT><<<grid, block, 0, st>>>(xp, wp, yp, rstd, rows, hidden, xs, ys, eps);
  }
  return check_launch("tp_rmsnorm_fwd");
}

template <typename XT, typename WT, typename OT>
static int bwd_typed(const void* dy, const void* x, const void* w, const float* rstd, void* dx, void* dw, float* ws,
                     int64_t rows, int hidden, int64_t dys, int64_t xs, int64_t dxs, hipStream_t st) {
  constexpr int E = 16 / sizeof(XT);
  const OT* gp = (const OT*)dy; const XT* xp = (const XT*)x; const WT* wp = (const WT*)w; XT* dxp = (XT*)dx;
  const int parts = rms_parts(rows);
  const int per = (hidden / E + 63) / 64;
  const bool vec = hidden % E == 0 && aligned16(dy) && aligned16(x) && aligned16(w) && aligned16(dx) &&
                   (dys * sizeof(OT)) % 16 == 0 && (xs * sizeof(XT)) % 16 == 0 && (dxs * sizeof(XT)) % 16 == 0 &&
                   per * E <= 128 && (size_t)hidden * 4 <= 64 * 1024;
  if (vec) {
    const dim3 grid(parts), block(256);
    const size_t sh = (size_t)hidden * sizeof(float);
#define TP_RMS_BWD(NV) rmsnorm_bwd_vec<XT, WT, OT, NV><<<grid, block, sh, st>>>(gp, xp, wp, rstd, dxp, ws, rows, hidden, dys, xs, dxs)
    if (per <= 1) TP_RMS_BWD(1);
    else if (per <= 2) TP_RMS_BWD(2);
    else if (per <= 4) TP_RMS_BWD(4);
    else if (per <= 8) TP_RMS_BWD(8);
    else if (per <= 16) TP_RMS_BWD(16);
    else TP_RMS_BWD(32);
#undef TP_RMS_BWD
  } else {
    rmsnorm_bwd_dx_generic<XT, WT, OT><<<dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st>>>(gp, xp, wp, rstd, dxp, rows,
                                                                                              hidden, dys, xs, dxs);
    rmsnorm_bwd_dw_generic<XT, OT><<<dim3((hidden + 255) / 256, parts), dim3(256), 0, st>>>(gp, xp, rstd, ws, rows, hidden,
                                                                                          dys, xs);
  }
  rmsnorm_dw_reduce<WT><<<dim3((hidden + 63) / 64), dim3(256), 0, st>>>(ws, (WT*)dw, parts, hidden);
  return check_launch("tp_rmsnorm_bwd");
}

}  // namespace tp

using namespace tp;

extern "C" int tp_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd, int64_t rows, int hidden,
                              int64_t x_row_stride, int64_t y_row_stride, float eps, int x_dtype, int w_dtype,
                              void* stream) {
  TP_REQUIRE(x && w && y && rstd, TP_ERR_BAD_ARG, "tp_rmsnorm_fwd: null pointer");
  TP_REQUIRE(rows >= 0 && hidden > 0, TP_ERR_BAD_ARG, "tp_rmsnorm_fwd: bad shape rows=%lld hidden=%d", (long long)rows, hidden);
  TP_REQUIRE(x_row_stride >= hidden && y_row_stride >= hidden, TP_ERR_BAD_ARG, "tp_rmsnorm_fwd: row stride smaller than hidden");
  if (rows == 0) return TP_OK;
  hipStream_t st = (hipStream_t)stream;
#define TP_GO(XT, WT, OT) return fwd_typed<XT, WT, OT>(x, w, y, rstd, rows, hidden, x_row_stride, y_row_stride, eps, st)
  if (x_dtype == TP_BF16 && w_dtype == TP_BF16) TP_GO(bf16_t, bf16_t, bf16_t);
  if (x_dtype == TP_BF16 && w_dtype == TP_F32) TP_GO(bf16_t, float, float);
  if (x_dtype == TP_F16 && w_dtype == TP_F16) TP_GO(f16_t, f16_t, f16_t);
  if (x_dtype == TP_F16 && w_dtype == TP_F32) TP_GO(f16_t, float, float);
  if (x_dtype == TP_F32 && w_dtype == TP_F32) TP_GO(float, float, float);
#undef TP_GO
  TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_rmsnorm_fwd: unsupported dtypes x=%d w=%d", x_dtype, w_dtype);
}

extern "C" size_t tp_rmsnorm_bwd_workspace_bytes(int64_t rows, int hidden) {
  if (rows <= 0 || hidden <= 0) return 0;
  return (size_t)rms_parts(rows) * (size_t)hidden * sizeof(float);
}

extern "C" int tp_rmsnorm_bwd(const void* dy, const void* x, const void* w, const float* rstd, void* dx, void* dw,
                              float* ws, int64_t rows, int hidden, int64_t dy_row_stride, int64_t x_row_stride,
                              int64_t dx_row_stride, int x_dtype, int w_dtype, void* stream) {
  TP_REQUIRE(dy && x && w && rstd && dx && dw && ws, TP_ERR_BAD_ARG, "tp_rmsnorm_bwd: null pointer");
  TP_REQUIRE(rows > 0 && hidden > 0, TP_ERR_BAD_ARG, "tp_rmsnorm_bwd: bad shape rows=%lld hidden=%d", (long long)rows, hidden);
  TP_REQUIRE(dy_row_stride >= hidden && x_row_stride >= hidden && dx_row_stride >= hidden, TP_ERR_BAD_ARG,
             "tp_rmsnorm_bwd: row stride smaller than hidden");
  hipStream_t st = (hipStream_t)stream;
#define TP_GO(XT, WT, OT) \
  return bwd_typed<XT, WT, OT>(dy, x, w, rstd, dx, dw, ws, rows, hidden, dy_row_stride, x_row_stride, dx_row_stride, st)
  if (x_dtype == TP_BF16 && w_dtype == TP_BF16) TP_GO(bf16_t, bf16_t, bf16_t);
  if (x_dtype == TP_BF16 && w_dtype == TP_F32) TP_GO(bf16_t, float, float);
  if (x_dtype == TP_F16 && w_dtype == TP_F16) TP_GO(f16_t, f16_t, f16_t);
  if (x_dtype == TP_F16 && w_dtype == TP_F32) TP_GO(f16_t, float, float);
  if (x_dtype == TP_F32 && w_dtype == TP_F32) TP_GO(float, float, float);
#undef TP_GO
  TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_rmsnorm_bwd: unsupported dtypes x=%d w=%d", x_dtype, w_dtype);
}
