// RMSNorm forward / backward for gfx950.  HBM-bound: one wavefront owns one row, the row is read
// once with 16-byte loads and kept in registers between the reduction and the scale.
//
// Semantics follow LlamaRMSNorm.forward (torchprime/torch_xla_models/model/llama/model.py:46-52;
// same body at model/mixtral/model.py:53-59 and model/deepseek_v3/model.py:38-44):
//   h = x.float(); var = mean(h*h, -1); h = h * rsqrt(var + eps); return weight * h.to(x.dtype)
// i.e. the normalised value is rounded to the input dtype BEFORE the weight multiply.
#include <mutex>

#include "common.hpp"

namespace tp {

// Partial dw rows written by the backward (a multiple of 4).  The row-walking kernel is fastest with about 512
// blocks of four waves (two per CU) at two 16-byte vectors per thread and about twice that at one vector, and
// slower with more (measured at 512 ... 4096 partial rows over hidden 512 ... 5120).  Rows short enough for a
// single wave go four to a block, so they need four times the partial rows for the same number of blocks: the
// count follows the row length.
constexpr int RMS_MIN_PARTS = 512, RMS_MAX_PARTS = 4096;

static inline int rms_parts(int64_t rows, int hidden) {
  const int cap = hidden <= 512 ? 4096 : hidden <= 1536 ? 2048 : hidden <= 2048 ? 1024 : RMS_MIN_PARTS;
  const int64_t p = (rows + 3) / 4 * 4;
  return (int)(p < cap ? p : cap);
}

// sum over the WAVES waves that share a row (fixed order); `red` holds one float per wave of the block
template <int WAVES>
__device__ __forceinline__ float row_sum(float v, float* red, int wave) {
  v = wave_sum(v);
  if (WAVES == 1) return v;
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = red[0];
#pragma unroll
  for (int i = 1; i < WAVES; i++) s += red[i];
  return s;
}

// ------------------------------------------------------------------------------------------------
// forward, vector path.  A row is shared by WAVES waves (1 for short rows, else the whole 256-thread
// block), each thread holding NV 16-byte vectors: few bytes per thread and many waves in flight is what
// streams fastest on this part.  x and y are non-temporal (touched once), the weight is not.
// ------------------------------------------------------------------------------------------------
template <typename XT, typename WT, typename OT, int NV, int WAVES>
__global__ __launch_bounds__(256) void rmsnorm_fwd_vec(const XT* __restrict__ x, const WT* __restrict__ w,
                                                       OT* __restrict__ y, float* __restrict__ rstd,
                                                       int64_t rows, int hidden, int64_t xs, int64_t ys,
                                                       float eps, const XT* __restrict__ res, XT* __restrict__ hsum,
                                                       int64_t rss, int64_t hss) {
  constexpr int E = 16 / sizeof(XT);
  constexpr int RPB = 4 / WAVES, TPR = 64 * WAVES;
  __shared__ float red[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = (int64_t)blockIdx.x * RPB + wave / WAVES;
  const int t = (wave % WAVES) * 64 + lane;
  if (row >= rows) return;  // uniform per block when WAVES == 4
  const int nvec = hidden / E;
  const XT* xr = x + row * xs;
  OT* yr = y + row * ys;

  // every load is issued before the first use: out-of-range vectors re-read the row's last one, so no
  // branch sits between the loads and they all travel together
  float xv[NV][E];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int v = t + TPR * i;
    load_f_nt<XT, E>(xr + (int64_t)(v < nvec ? v : nvec - 1) * E, xv[i]);
  }
  if (res) {
    // fused residual add (model/llama/model.py:288-291): h = residual + x, rounded to the activation dtype as the
    // eager add does; h is written out (it is the next residual) and normalised in place of x
    const XT* rr = res + row * rss;
    XT* hr = hsum + row * hss;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int v = t + TPR * i;
      float rv[E];
      load_f_nt<XT, E>(rr + (int64_t)(v < nvec ? v : nvec - 1) * E, rv);
#pragma unroll
      for (int e = 0; e < E; e++) xv[i][e] = round_to<XT>(rv[e] + xv[i][e]);
      if (v < nvec) store_f_nt<XT, E>(hr + (int64_t)v * E, xv[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < NV; i++) {
    if (t + TPR * i < nvec) {
#pragma unroll
      for (int e = 0; e < E; e++) ss += xv[i][e] * xv[i][e];
    }
  }
  ss = row_sum<WAVES>(ss, red, wave);
  const float r = rsqrtf(ss / (float)hidden + eps);
  if (t == 0) rstd[row] = r;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int v = t + TPR * i;
    if (v < nvec) {
      float wv[E], o[E];
      load_f<WT, E>(w + (int64_t)v * E, wv);
#pragma unroll
      for (int e = 0; e < E; e++) o[e] = wv[e] * round_to<XT>(xv[i][e] * r);
      store_f_nt<OT, E>(yr + (int64_t)v * E, o);
    }
  }
}

// forward, any hidden / alignment: two passes over the row with scalar accesses
template <typename XT, typename WT, typename OT>
__global__ __launch_bounds__(256) void rmsnorm_fwd_generic(const XT* __restrict__ x, const WT* __restrict__ w,
                                                           OT* __restrict__ y, float* __restrict__ rstd,
                                                           int64_t rows, int hidden, int64_t xs, int64_t ys,
                                                           float eps, const XT* __restrict__ res, XT* __restrict__ hsum,
                                                           int64_t rss, int64_t hss) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const XT* xr = x + row * xs;
  OT* yr = y + row * ys;
  if (res) {  // h = residual + x first; the wave then normalises the row it has just written
    XT* hr = hsum + row * hss;
    for (int c = lane; c < hidden; c += 64) hr[c] = Elem<XT>::from_f(Elem<XT>::to_f(res[row * rss + c]) + Elem<XT>::to_f(xr[c]));
    xr = hr;
  }
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
// backward, vector path.  Same thread layout as the forward; a block walks rows r, r + gridDim.x*RPB, ...
// Each thread owns fixed columns, so its dw partial sums stay in registers over all the rows it sees and
// go straight to one partial row per (block, row slot): no atomics, no cross-thread fold.
// ------------------------------------------------------------------------------------------------
template <typename XT, typename WT, typename OT, int NV, int WAVES, bool RES>
__global__ __launch_bounds__(64 * (WAVES > 4 ? WAVES : 4)) void rmsnorm_bwd_vec(const OT* __restrict__ dy, const XT* __restrict__ x,
                                                       const WT* __restrict__ w, const float* __restrict__ rstd,
                                                       XT* __restrict__ dx, float* __restrict__ ws, int64_t rows,
                                                       int hidden, int64_t dys, int64_t xs, int64_t dxs,
                                                       const XT* __restrict__ dres, int64_t drs) {
  constexpr int E = 16 / sizeof(XT);
  constexpr int BW = WAVES > 4 ? WAVES : 4;  // waves per block: four, or all the waves of a long row
  constexpr int RPB = BW / WAVES, TPR = 64 * WAVES;
  // Rows are requested one ahead while a thread's share of a row is small enough for both rows to sit in registers.
  constexpr bool AHEAD = NV <= 2 && !(WAVES == 16 && RES && sizeof(OT) > sizeof(XT));  // (that one would spill at 128 registers)
  __shared__ float red[2][BW];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slot = wave / WAVES;
  const int t = (wave % WAVES) * 64 + lane;
  const int nvec = hidden / E;
  const float inv_h = 1.f / (float)hidden;
  const int64_t step = (int64_t)gridDim.x * RPB;

  Raw<WT, E> rw[NV];  // the weights stay packed and are converted where they are used: half the registers for 16-bit ones
  float wacc[NV][E];
  int off[NV];  // element offset of each of the thread's vectors (out-of-range vectors re-read the row's last one)
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int v = t + TPR * i;
#pragma unroll
    for (int e = 0; e < E; e++) wacc[i][e] = 0.f;
    off[i] = (v < nvec ? v : nvec - 1) * E;
    rw[i] = load_raw_nt<WT, E>(w + off[i]);
  }
  // The words of a row are requested raw and converted when the row's turn comes.  With AHEAD the next row is
  // requested before the arithmetic, the block-wide reduction and the stores of this one, so that a CU's resident
  // blocks keep about twice the bytes in flight (measured: 3-4 % faster at two vectors per thread, 8 % slower at four).
  Raw<XT, E> rx[NV], ra[RES ? NV : 1];
  Raw<OT, E> rg[NV];
  float r_next = 0.f;
  auto request = [&](int64_t row) {
#pragma unroll
    for (int i = 0; i < NV; i++) {
      rx[i] = load_raw_nt<XT, E>(x + row * xs + off[i]);
      rg[i] = load_raw_nt<OT, E>(dy + row * dys + off[i]);
    }
    if (RES) {
#pragma unroll
      for (int i = 0; i < NV; i++) ra[RES ? i : 0] = load_raw_nt<XT, E>(dres + row * drs + off[i]);
    }
    r_next = rstd[row];
  };
  const int64_t row0 = (int64_t)blockIdx.x * RPB + slot;
  if (AHEAD && row0 < rows) request(row0);
  int it = 0;
  // with WAVES == 4 all waves of the block share the row, so the loop bound is uniform for the barrier
  for (int64_t row = row0; row < rows; row += step, it++) {
    if (!AHEAD) request(row);
    const float r = r_next;
    XT* dr = dx + row * dxs;
    float n[NV][E], g[NV][E];
    float c = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      unpack_f<XT, E>(rx[i], n[i]);
      unpack_f<OT, E>(rg[i], g[i]);
    }
    float a[RES ? NV : 1][E];
    if (RES) {
#pragma unroll
      for (int i = 0; i < NV; i++) unpack_f<XT, E>(ra[RES ? i : 0], a[RES ? i : 0]);
    }
    if (AHEAD && row + step < rows) request(row + step);
#pragma unroll
    for (int i = 0; i < NV; i++) {
      if (t + TPR * i < nvec) {
        float wv[E];
        Raw<WT, E> q = rw[i];
#pragma unroll
        for (int k = 0; k < (int)(sizeof(q.q) / sizeof(q.q[0])); k++) asm volatile("" : "+v"(q.q[k]));  // (keeps the conversion inside the loop)
        unpack_f<WT, E>(q, wv);
#pragma unroll
        for (int e = 0; e < E; e++) {
          const float dyv = g[i][e];
          n[i][e] *= r;
          g[i][e] = dyv * wv[e];
          c += g[i][e] * n[i][e];
          wacc[i][e] += dyv * round_to<XT>(n[i][e]);
        }
      }
    }
    c = row_sum<WAVES>(c, red[it & 1], wave) * inv_h;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int v = t + TPR * i;
      float o[E];
#pragma unroll
      for (int e = 0; e < E; e++) o[e] = r * (g[i][e] - n[i][e] * c);
      if (RES) {
        // fused residual: the gradient that reached h through the residual path joins here, each addend rounded
        // to the activation dtype first, as autograd's accumulation of two bf16 gradients does
#pragma unroll
        for (int e = 0; e < E; e++) o[e] = round_to<XT>(o[e]) + a[RES ? i : 0][e];
      }
      if (v < nvec) store_f_nt<XT, E>(dr + (int64_t)v * E, o);
    }
  }
  float* out = ws + ((int64_t)blockIdx.x * RPB + slot) * hidden;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int v = t + TPR * i;
    if (v < nvec) store_f<float, E>(out + (int64_t)v * E, wacc[i]);
  }
}

// backward dx, any hidden / alignment
template <typename XT, typename WT, typename OT>
__global__ __launch_bounds__(256) void rmsnorm_bwd_dx_generic(const OT* __restrict__ dy, const XT* __restrict__ x,
                                                              const WT* __restrict__ w, const float* __restrict__ rstd,
                                                              XT* __restrict__ dx, int64_t rows, int hidden,
                                                              int64_t dys, int64_t xs, int64_t dxs,
                                                              const XT* __restrict__ dres, int64_t drs) {
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
    float o = r * (g - n * c);
    if (dres) o = round_to<XT>(o) + Elem<XT>::to_f(dres[row * drs + j]);
    dr[j] = Elem<XT>::from_f(o);
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

// dw[c] = sum_p ws[p, c], fixed order: 16 columns per block, 16 row groups folded through LDS (the
// partial rows were just written and mostly still sit in cache, so many small blocks beat few wide ones)
template <typename WT>
__global__ __launch_bounds__(256) void rmsnorm_dw_reduce(const float* __restrict__ ws, WT* __restrict__ dw, int parts,
                                                         int hidden) {
  __shared__ float red[256];
  const int c = blockIdx.x * 16 + (threadIdx.x & 15);
  const int g = threadIdx.x >> 4;
  float acc = 0.f;
  if (c < hidden) {
#pragma unroll 8
    for (int p = g; p < parts; p += 16) acc += ws[(int64_t)p * hidden + c];
  }
  red[threadIdx.x] = acc;
  __syncthreads();
  if (g == 0 && c < hidden) {
    float s = red[threadIdx.x];
#pragma unroll
    for (int k = 1; k < 16; k++) s += red[threadIdx.x + 16 * k];
    dw[c] = Elem<WT>::from_f(s);
  }
}

// ------------------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------------------
template <typename XT, typename WT, typename OT>
static int fwd_typed(const void* x, const void* w, void* y, float* rstd, int64_t rows, int hidden, int64_t xs,
                     int64_t ys, float eps, hipStream_t st, const void* res = nullptr, void* hsum = nullptr,
                     int64_t rss = 0, int64_t hss = 0) {
  constexpr int E = 16 / sizeof(XT);
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  const XT* xp = (const XT*)x; const WT* wp = (const WT*)w; OT* yp = (OT*)y;
  const XT* rp = (const XT*)res; XT* hp = (XT*)hsum;
  const bool vec = hidden % E == 0 && aligned16(x) && aligned16(w) && aligned16(y) && (xs * sizeof(XT)) % 16 == 0 &&
                   aligned16(res) && aligned16(hsum) && (rss * sizeof(XT)) % 16 == 0 && (hss * sizeof(XT)) % 16 == 0 &&
                   (ys * sizeof(OT)) % 16 == 0 && hidden / E <= 256 * 8;
  if (vec) {
    const int nvec = hidden / E;
#define TP_RMS_FWD(NV, WAVES)                                                                                  \
  rmsnorm_fwd_vec<XT, WT, OT, NV, WAVES><<<dim3((unsigned)((rows + 4 / WAVES - 1) / (4 / WAVES))), block, 0, st>>>( \
      xp, wp, yp, rstd, rows, hidden, xs, ys, eps, rp, hp, rss, hss)
    // two vectors per thread over a whole block measured fastest at hidden 4096 (against one vector over
    // 512 threads, or a wave per row)
    if (nvec <= 64) TP_RMS_FWD(1, 1);
    else if (nvec <= 128) TP_RMS_FWD(2, 1);
    else if (nvec <= 192) TP_RMS_FWD(3, 1);  // (a 256-thread row would leave a quarter of its lanes idle: hidden 1536)
    else if (nvec <= 256) TP_RMS_FWD(1, 4);
    else if (nvec <= 512) TP_RMS_FWD(2, 4);
    else if (nvec <= 1024) TP_RMS_FWD(4, 4);
    else TP_RMS_FWD(8, 4);
#undef TP_RMS_FWD
  } else {
    rmsnorm_fwd_generic<XT, WT, OT><<<grid, block, 0, st>>>(xp, wp, yp, rstd, rows, hidden, xs, ys, eps, rp, hp, rss, hss);
  }
  return check_launch("tp_rmsnorm_fwd");
}

template <typename XT, typename WT, typename OT>
static int bwd_typed(const void* dy, const void* x, const void* w, const float* rstd, void* dx, void* dw, float* ws,
                     int64_t rows, int hidden, int64_t dys, int64_t xs, int64_t dxs, hipStream_t st,
                     const void* dres = nullptr, int64_t drs = 0) {
  constexpr int E = 16 / sizeof(XT);
  const OT* gp = (const OT*)dy; const XT* xp = (const XT*)x; const WT* wp = (const WT*)w; XT* dxp = (XT*)dx;
  const XT* drp = (const XT*)dres;
  const int parts = rms_parts(rows, hidden);
  const int nvec = hidden / E;
  const bool vec = hidden % E == 0 && aligned16(dy) && aligned16(x) && aligned16(w) && aligned16(dx) &&
                   (dys * sizeof(OT)) % 16 == 0 && (xs * sizeof(XT)) % 16 == 0 && (dxs * sizeof(XT)) % 16 == 0 &&
                   aligned16(dres) && (drs * sizeof(XT)) % 16 == 0 && nvec <= 256 * 8;
  if (vec) {
#define TP_RMS_BWD(NV, WAVES)                                                                             \
  do {                                                                                                    \
    constexpr int BW = WAVES > 4 ? WAVES : 4;                                                             \
    const dim3 grid(parts / (BW / WAVES)), block(64 * BW);                                                \
    if (drp)                                                                                              \
      rmsnorm_bwd_vec<XT, WT, OT, NV, WAVES, true><<<grid, block, 0, st>>>(                               \
          gp, xp, wp, rstd, dxp, ws, rows, hidden, dys, xs, dxs, drp, drs);                               \
    else                                                                                                  \
      rmsnorm_bwd_vec<XT, WT, OT, NV, WAVES, false><<<grid, block, 0, st>>>(                              \
          gp, xp, wp, rstd, dxp, ws, rows, hidden, dys, xs, dxs, drp, drs);                               \
  } while (0)
    // Measured per shape (same box, 128 Mi elements): up to two vectors per thread a row spreads over more waves
    // rather than more vectors per thread - 16 waves for rows beyond 1024 vectors (hidden 16384 in bf16: 178 -> 151 us
    // against four waves of eight vectors), eight for the fused-residual form beyond 512 (hidden 7168: 202 -> 180 us);
    // the plain form is faster with four waves of four vectors there (141 against 149 us).
    if (nvec <= 64) TP_RMS_BWD(1, 1);
    else if (nvec <= 128) TP_RMS_BWD(2, 1);
    else if (nvec <= 192) TP_RMS_BWD(3, 1);
    else if (nvec <= 256) TP_RMS_BWD(1, 4);
    else if (nvec <= 512) TP_RMS_BWD(2, 4);
    else if (nvec <= 1024) { if (drp) TP_RMS_BWD(2, 8); else TP_RMS_BWD(4, 4); }
    else TP_RMS_BWD(2, 16);
#undef TP_RMS_BWD
  } else {
    rmsnorm_bwd_dx_generic<XT, WT, OT><<<dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st>>>(gp, xp, wp, rstd, dxp, rows,
                                                                                              hidden, dys, xs, dxs, drp, drs);
    rmsnorm_bwd_dw_generic<XT, OT><<<dim3((hidden + 255) / 256, parts), dim3(256), 0, st>>>(gp, xp, rstd, ws, rows, hidden,
                                                                                          dys, xs);
  }
  rmsnorm_dw_reduce<WT><<<dim3((hidden + 15) / 16), dim3(256), 0, st>>>(ws, (WT*)dw, parts, hidden);
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
  return (size_t)rms_parts(rows, hidden) * (size_t)hidden * sizeof(float);
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

// ------------------------------------------------------------------------------------------------
// RMSNorm fused with the residual add that precedes it in a decoder layer
// ------------------------------------------------------------------------------------------------
extern "C" int tp_add_rmsnorm_fwd(const void* x, const void* residual, const void* w, void* h, void* y, float* rstd,
                                  int64_t rows, int hidden, int64_t x_row_stride, int64_t res_row_stride,
                                  int64_t h_row_stride, int64_t y_row_stride, float eps, int x_dtype, int w_dtype,
                                  void* stream) {
  TP_REQUIRE(x && residual && w && h && y && rstd, TP_ERR_BAD_ARG, "tp_add_rmsnorm_fwd: null pointer");
  TP_REQUIRE(rows >= 0 && hidden > 0, TP_ERR_BAD_ARG, "tp_add_rmsnorm_fwd: bad shape rows=%lld hidden=%d", (long long)rows, hidden);
  TP_REQUIRE(x_row_stride >= hidden && res_row_stride >= hidden && h_row_stride >= hidden && y_row_stride >= hidden,
             TP_ERR_BAD_ARG, "tp_add_rmsnorm_fwd: row stride smaller than hidden");
  if (rows == 0) return TP_OK;
  hipStream_t st = (hipStream_t)stream;
#define TP_GO(XT, WT, OT)                                                                                          \
  return fwd_typed<XT, WT, OT>(x, w, y, rstd, rows, hidden, x_row_stride, y_row_stride, eps, st, residual, h, \
                               res_row_stride, h_row_stride)
  if (x_dtype == TP_BF16 && w_dtype == TP_BF16) TP_GO(bf16_t, bf16_t, bf16_t);
  if (x_dtype == TP_BF16 && w_dtype == TP_F32) TP_GO(bf16_t, float, float);
  if (x_dtype == TP_F16 && w_dtype == TP_F16) TP_GO(f16_t, f16_t, f16_t);
  if (x_dtype == TP_F16 && w_dtype == TP_F32) TP_GO(f16_t, float, float);
  if (x_dtype == TP_F32 && w_dtype == TP_F32) TP_GO(float, float, float);
#undef TP_GO
  TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_add_rmsnorm_fwd: unsupported dtypes x=%d w=%d", x_dtype, w_dtype);
}

extern "C" int tp_add_rmsnorm_bwd(const void* dy, const void* dh, const void* h, const void* w, const float* rstd,
                                  void* dx, void* dw, float* ws, int64_t rows, int hidden, int64_t dy_row_stride,
                                  int64_t dh_row_stride, int64_t h_row_stride, int64_t dx_row_stride, int x_dtype,
                                  int w_dtype, void* stream) {
  TP_REQUIRE(dy && dh && h && w && rstd && dx && dw && ws, TP_ERR_BAD_ARG, "tp_add_rmsnorm_bwd: null pointer");
  TP_REQUIRE(rows > 0 && hidden > 0, TP_ERR_BAD_ARG, "tp_add_rmsnorm_bwd: bad shape rows=%lld hidden=%d", (long long)rows, hidden);
  TP_REQUIRE(dy_row_stride >= hidden && dh_row_stride >= hidden && h_row_stride >= hidden && dx_row_stride >= hidden,
             TP_ERR_BAD_ARG, "tp_add_rmsnorm_bwd: row stride smaller than hidden");
  hipStream_t st = (hipStream_t)stream;
#define TP_GO(XT, WT, OT)                                                                                        \
  return bwd_typed<XT, WT, OT>(dy, h, w, rstd, dx, dw, ws, rows, hidden, dy_row_stride, h_row_stride, dx_row_stride, st, \
                               dh, dh_row_stride)
  if (x_dtype == TP_BF16 && w_dtype == TP_BF16) TP_GO(bf16_t, bf16_t, bf16_t);
  if (x_dtype == TP_BF16 && w_dtype == TP_F32) TP_GO(bf16_t, float, float);
  if (x_dtype == TP_F16 && w_dtype == TP_F16) TP_GO(f16_t, f16_t, f16_t);
  if (x_dtype == TP_F16 && w_dtype == TP_F32) TP_GO(f16_t, float, float);
  if (x_dtype == TP_F32 && w_dtype == TP_F32) TP_GO(float, float, float);
#undef TP_GO
  TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_add_rmsnorm_bwd: unsupported dtypes x=%d w=%d", x_dtype, w_dtype);
}

// ------------------------------------------------------------------------------------------------
// The backward once more for callers that must not allocate (code under HIP graph capture, serving loops,
// harnesses that forbid hipMalloc): the partial-dw rows live in a file-scope device array instead of a
// caller-provided workspace.  Every GPU the library runs on holds its own copy of the array until the process
// ends.  In host code the array's name is only a stand-in for the symbol, not a device address: the address is
// looked up once per device (with that device current) and the kernels are given that pointer.
// Nothing in the array has to start at zero: every partial row that the fold reads is written in full by the
// same call first.  All calls on one GPU share the array, so calls that overlap on one GPU (two streams) race.
// ------------------------------------------------------------------------------------------------
namespace tp {
constexpr int RMS_NOALLOC_MAX_HIDDEN = 8192;
constexpr size_t RMS_NOALLOC_BYTES = (size_t)RMS_MIN_PARTS * RMS_NOALLOC_MAX_HIDDEN * sizeof(float);  // 16 MiB
static __device__ __align__(256) unsigned char scratch[RMS_NOALLOC_BYTES];

constexpr int RMS_MAX_DEVICES = 64;
static void* g_scratch_ptr[RMS_MAX_DEVICES];  // per device, filled on the first call on that device
static std::mutex g_scratch_mu;

static int scratch_for_current_device(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  TP_REQUIRE(e == hipSuccess && dev >= 0 && dev < RMS_MAX_DEVICES, TP_ERR_LAUNCH, "tp_rmsnorm_bwd_noalloc: hipGetDevice: %s",
             hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    TP_REQUIRE(e == hipSuccess && p, TP_ERR_LAUNCH, "tp_rmsnorm_bwd_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = (float*)g_scratch_ptr[dev];
  return TP_OK;
}
}  // namespace tp

extern "C" int tp_rmsnorm_bwd_noalloc(const void* dy, const void* x, const void* w, const float* rstd, void* dx, void* dw,
                                      int64_t rows, int hidden, int64_t dy_row_stride, int64_t x_row_stride,
                                      int64_t dx_row_stride, int x_dtype, int w_dtype, void* stream) {
  TP_REQUIRE(rows > 0 && hidden > 0, TP_ERR_BAD_ARG, "tp_rmsnorm_bwd_noalloc: bad shape rows=%lld hidden=%d", (long long)rows, hidden);
  const size_t need = tp_rmsnorm_bwd_workspace_bytes(rows, hidden);
  TP_REQUIRE(need <= RMS_NOALLOC_BYTES, TP_ERR_UNSUPPORTED,
             "tp_rmsnorm_bwd_noalloc: rows=%lld hidden=%d need %zu bytes of scratch, the built-in array holds %zu "
             "(hidden up to %d); use tp_rmsnorm_bwd with a caller-provided workspace",
             (long long)rows, hidden, need, (size_t)RMS_NOALLOC_BYTES, RMS_NOALLOC_MAX_HIDDEN);
  float* ws = nullptr;
  const int rc = scratch_for_current_device(&ws);
  if (rc) return rc;
  return tp_rmsnorm_bwd(dy, x, w, rstd, dx, dw, ws, rows, hidden, dy_row_stride, x_row_stride, dx_row_stride, x_dtype, w_dtype,
                        stream);
}
