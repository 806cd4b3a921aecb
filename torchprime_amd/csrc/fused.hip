// HBM-bound element-wise / row-reduction kernels either side of the attention path, for gfx950:
//
//   l2norm      Llama4TextL2Norm (torchprime/torch_xla_models/model/llama4/model.py:104-116): a weightless RMSNorm
//               over the head dim of q / k, computed in fp32 and rounded once (`.type_as(x)`).
//   scale_rows  the temperature scale of the NoPE layers (model/llama4/model.py:513-525): every head row of a
//               position is multiplied by that position's fp32 factor and rounded, `(q * attn_scales).to(q.dtype)`.
//   swiglu      act_fn(gate_proj(x)) * up_proj(x) of LlamaMLP.forward (model/llama/model.py:137-139) with
//               act_fn = SiLU: silu rounded to the activation dtype, then the product rounded, as the eager ops do.
//   cross_entropy   cross_entropy_loss (torchprime/torch_xla_models/loss.py:5-20): next-token shift, mean over the
//               labels that are not ignore_index of  logsumexp(logits) - logits[label]; one pass over the logits with
//               an online max / sum, the shift done by indexing (no contiguous copies of logits and labels).
//
// Every tensor is touched once: non-temporal 16-byte accesses, one thread = one vector.
#include "common.hpp"

namespace tp {

// ------------------------------------------------------------------------------------------------
// L2 norm over short rows (a head dim): LPR lanes share a row, 64 / LPR rows per wave
// ------------------------------------------------------------------------------------------------
template <int LPR>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int o = LPR / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

template <typename T, int LPR>
__global__ __launch_bounds__(256) void l2norm_fwd_kernel(const T* __restrict__ x, T* __restrict__ y, float* __restrict__ rstd,
                                                         int64_t rows, int dim, int64_t xs, int64_t ys, float eps) {
  constexpr int E = 16 / sizeof(T);
  const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPR;
  const int l = threadIdx.x % LPR;
  const bool valid = row < rows;
  const int64_t r = valid ? row : rows - 1;
  float v[E];
  load_f_nt<T, E>(x + r * xs + l * E, v);
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < E; e++) ss += v[e] * v[e];
  ss = group_sum<LPR>(ss);
  const float rs = rsqrtf(ss / (float)dim + eps);
  float o[E];
#pragma unroll
  for (int e = 0; e < E; e++) o[e] = v[e] * rs;
  if (valid) {
    store_f_nt<T, E>(y + r * ys + l * E, o);
    if (l == 0) rstd[r] = rs;
  }
}

// dx = rstd * (g - n * mean(g * n)),  n = x * rstd,  g = dy
template <typename T, int LPR>
__global__ __launch_bounds__(256) void l2norm_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                         const float* __restrict__ rstd, T* __restrict__ dx, int64_t rows,
                                                         int dim, int64_t dys, int64_t xs, int64_t dxs) {
  constexpr int E = 16 / sizeof(T);
  const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPR;
  const int l = threadIdx.x % LPR;
  const bool valid = row < rows;
  const int64_t r = valid ? row : rows - 1;
  float n[E], g[E];
  load_f_nt<T, E>(x + r * xs + l * E, n);
  load_f_nt<T, E>(dy + r * dys + l * E, g);
  const float rs = rstd[r];
  float c = 0.f;
#pragma unroll
  for (int e = 0; e < E; e++) {
    n[e] *= rs;
    c += g[e] * n[e];
  }
  c = group_sum<LPR>(c) / (float)dim;
  float o[E];
#pragma unroll
  for (int e = 0; e < E; e++) o[e] = rs * (g[e] - n[e] * c);
  if (valid) store_f_nt<T, E>(dx + r * dxs + l * E, o);
}

template <typename T>
static int l2norm_launch(bool backward, const void* dy, const void* x, void* out, float* rstd, int64_t rows, int dim,
                         int64_t dys, int64_t xs, int64_t os, float eps, hipStream_t st) {
  constexpr int E = 16 / sizeof(T);
  const int lpr = dim / E;
  TP_REQUIRE(dim % E == 0 && lpr >= 1 && lpr <= 64 && (lpr & (lpr - 1)) == 0, TP_ERR_UNSUPPORTED,
             "tp_l2norm: dim=%d must be %d times a power of two up to 64", dim, E);
  const bool ok = aligned16(x) && aligned16(out) && aligned16(dy) && (xs * sizeof(T)) % 16 == 0 && (os * sizeof(T)) % 16 == 0 &&
                  (dys * sizeof(T)) % 16 == 0;
  TP_REQUIRE(ok, TP_ERR_BAD_ARG, "tp_l2norm: pointers and row strides must keep rows 16-byte aligned");
  const int64_t threads = rows * lpr;
  TP_REQUIRE((threads + 255) / 256 < (1ll << 31), TP_ERR_UNSUPPORTED, "tp_l2norm: too many rows");
  const dim3 grid((unsigned)((threads + 255) / 256)), block(256);
#define TP_L2(L)                                                                                                      \
  if (lpr == L) {                                                                                                     \
    if (backward)                                                                                                     \
      l2norm_bwd_kernel<T, L><<<grid, block, 0, st>>>((const T*)dy, (const T*)x, rstd, (T*)out, rows, dim, dys, xs, os); \
    else                                                                                                              \
      l2norm_fwd_kernel<T, L><<<grid, block, 0, st>>>((const T*)x, (T*)out, rstd, rows, dim, xs, os, eps);            \
  }
  TP_L2(1) TP_L2(2) TP_L2(4) TP_L2(8) TP_L2(16) TP_L2(32) TP_L2(64)
#undef TP_L2
  return check_launch("tp_l2norm");
}

// ------------------------------------------------------------------------------------------------
// per-position scale: rows are numbered (b, s, n) and row r is multiplied by scale[(r / heads) % seq]
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void scale_rows_kernel(const T* __restrict__ x, const float* __restrict__ scale, T* __restrict__ y,
                                                         int64_t rows, int dim, int64_t xs, int64_t ys, int heads, int seq) {
  constexpr int E = 16 / sizeof(T);
  const int vpr = dim / E;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * vpr) return;
  const int64_t r = idx / vpr;
  const int c = (int)(idx - r * vpr) * E;
  const float sc = scale[(r / heads) % seq];
  float v[E];
  load_f_nt<T, E>(x + r * xs + c, v);
#pragma unroll
  for (int e = 0; e < E; e++) v[e] *= sc;
  store_f_nt<T, E>(y + r * ys + c, v);
}

// ------------------------------------------------------------------------------------------------
// SwiGLU
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float sigmoidf_fast(float x) { return 1.f / (1.f + __expf(-x)); }

template <typename T>
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const T* __restrict__ gate, const T* __restrict__ up, T* __restrict__ out,
                                                         int64_t rows, int cols, int64_t gs, int64_t us, int64_t os) {
  constexpr int E = 16 / sizeof(T);
  const int vpr = cols / E;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * vpr) return;
  const int64_t r = idx / vpr;
  const int c = (int)(idx - r * vpr) * E;
  float g[E], u[E], o[E];
  load_f_nt<T, E>(gate + r * gs + c, g);
  load_f_nt<T, E>(up + r * us + c, u);
#pragma unroll
  for (int e = 0; e < E; e++) o[e] = round_to<T>(g[e] * sigmoidf_fast(g[e])) * u[e];
  store_f_nt<T, E>(out + r * os + c, o);
}

// dgate = dout * up * d silu(gate),  dup = dout * silu(gate) (silu rounded as the forward rounded it)
template <typename T>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T* __restrict__ dout, const T* __restrict__ gate,
                                                         const T* __restrict__ up, T* __restrict__ dgate, T* __restrict__ dup,
                                                         int64_t rows, int cols, int64_t dos, int64_t gs, int64_t us,
                                                         int64_t dgs, int64_t dus) {
  constexpr int E = 16 / sizeof(T);
  const int vpr = cols / E;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * vpr) return;
  const int64_t r = idx / vpr;
  const int c = (int)(idx - r * vpr) * E;
  float d[E], g[E], u[E], dg[E], du[E];
  load_f_nt<T, E>(dout + r * dos + c, d);
  load_f_nt<T, E>(gate + r * gs + c, g);
  load_f_nt<T, E>(up + r * us + c, u);
#pragma unroll
  for (int e = 0; e < E; e++) {
    const float sg = sigmoidf_fast(g[e]);
    du[e] = d[e] * round_to<T>(g[e] * sg);
    dg[e] = round_to<T>(d[e] * u[e]) * (sg * (1.f + g[e] * (1.f - sg)));
  }
  store_f_nt<T, E>(dgate + r * dgs + c, dg);
  store_f_nt<T, E>(dup + r * dus + c, du);
}

// ------------------------------------------------------------------------------------------------
// cross entropy with the next-token shift
// ------------------------------------------------------------------------------------------------
// One block per (batch, position) row of the logits.  Row (b, s) with s < S - 1 is scored against labels[b, s + 1];
// the last position of every sequence has no target.  Online max / sum over the row, then a fixed-order fold of the
// 256 per-thread pairs.  Writes the row's logsumexp and its loss (0 where there is no target or the label is ignored).
template <typename T>
__global__ __launch_bounds__(256) void xent_fwd_kernel(const T* __restrict__ logits, const int64_t* __restrict__ labels,
                                                       float* __restrict__ lse, float* __restrict__ row_loss, int S, int V,
                                                       int64_t ls_b, int64_t ls_s, int64_t lab_b, int ignore_index) {
  constexpr int E = 16 / sizeof(T);
  __shared__ float sm[256], ss[256];
  const int row = blockIdx.x;
  const int b = row / S, s = row - b * S;
  const T* lr = logits + b * ls_b + s * ls_s;
  float m = -INFINITY, acc = 0.f;
  const int nvec = V / E;
  const bool vec = (((size_t)lr) & 15) == 0;
  if (vec) {
    for (int v = threadIdx.x; v < nvec; v += 256) {
      float x[E];
      load_f_nt<T, E>(lr + (int64_t)v * E, x);
      float mx = x[0];
#pragma unroll
      for (int e = 1; e < E; e++) mx = fmaxf(mx, x[e]);
      // (a vector of -inf logits - a masked range of the vocabulary - while the thread has seen nothing finite yet:
      // m stays -inf, and exp(x - m) would be exp(NaN); such logits add nothing)
      if (mx == -INFINITY) continue;
      if (mx > m) {
        acc *= __expf(m - mx);  // (m = -inf the first time: acc is 0 and exp(-inf) = 0)
        m = mx;
      }
#pragma unroll
      for (int e = 0; e < E; e++) acc += __expf(x[e] - m);
    }
  }
  for (int c = (vec ? nvec * E : 0) + threadIdx.x; c < V; c += 256) {
    const float x = Elem<T>::to_f(lr[c]);
    if (x == -INFINITY) continue;
    if (x > m) {
      acc *= __expf(m - x);
      m = x;
    }
    acc += __expf(x - m);
  }
  sm[threadIdx.x] = m;
  ss[threadIdx.x] = acc;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) {
      const float m1 = sm[threadIdx.x], m2 = sm[threadIdx.x + o];
      const float mm = fmaxf(m1, m2);
      const float a1 = m1 == -INFINITY ? 0.f : ss[threadIdx.x] * __expf(m1 - mm);
      const float a2 = m2 == -INFINITY ? 0.f : ss[threadIdx.x + o] * __expf(m2 - mm);
      sm[threadIdx.x] = mm;
      ss[threadIdx.x] = a1 + a2;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const float l = sm[0] + logf(ss[0]);
    lse[row] = l;
    float loss = 0.f;
    if (s < S - 1) {
      const int64_t lab = labels[b * lab_b + s + 1];
      if (lab != ignore_index && lab >= 0 && lab < V) loss = l - Elem<T>::to_f(lr[lab]);
    }
    row_loss[row] = loss;
  }
}

// loss = sum(row_loss) / count(valid targets), one block, fixed order; also stores the count for the backward
__global__ __launch_bounds__(256) void xent_mean_kernel(const float* __restrict__ row_loss, const int64_t* __restrict__ labels,
                                                        float* __restrict__ out, int B, int S, int V, int64_t lab_b,
                                                        int ignore_index) {
  __shared__ double sl[256];
  __shared__ int sc[256];
  double acc = 0.0;
  int cnt = 0;
  const int n = B * S;
  for (int i = threadIdx.x; i < n; i += 256) {
    const int b = i / S, s = i - b * S;
    acc += (double)row_loss[i];
    if (s < S - 1) {
      const int64_t lab = labels[b * lab_b + s + 1];
      cnt += (lab != ignore_index && lab >= 0 && lab < V) ? 1 : 0;
    }
  }
  sl[threadIdx.x] = acc;
  sc[threadIdx.x] = cnt;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) {
      sl[threadIdx.x] += sl[threadIdx.x + o];
      sc[threadIdx.x] += sc[threadIdx.x + o];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    out[0] = (float)(sl[0] / (double)sc[0]);  // no valid target: 0 / 0 = NaN, as CrossEntropyLoss gives
    out[1] = (float)sc[0];
  }
}

// dlogits[b, s, c] = dloss / count * (softmax(logits[b, s])[c] - [c == label]) for rows with a target, else 0
constexpr int XENT_BWD_U = 1;
template <typename T>
__global__ __launch_bounds__(256) void xent_bwd_kernel(const T* __restrict__ logits, const int64_t* __restrict__ labels,
                                                       const float* __restrict__ lse, const float* __restrict__ loss_and_count,
                                                       const float* __restrict__ dloss, T* __restrict__ dlogits, int S, int V,
                                                       int64_t ls_b, int64_t ls_s, int64_t lab_b, int64_t ds_b, int64_t ds_s,
                                                       int ignore_index, int chunks) {
  constexpr int E = 16 / sizeof(T);
  // consecutive blocks walk one row before the next: the card streams through the tensor like a flat copy
  const int row = blockIdx.x / chunks, chunk = blockIdx.x - row * chunks;
  const int b = row / S, s = row - b * S;
  const T* lr = logits + b * ls_b + s * ls_s;
  T* dr = dlogits + b * ds_b + s * ds_s;
  int64_t lab = -1;
  if (s < S - 1) {
    lab = labels[b * lab_b + s + 1];
    if (lab == ignore_index || lab < 0 || lab >= V) lab = -1;
  }
  const float scale = lab < 0 ? 0.f : dloss[0] / loss_and_count[1];
  const float l = lse[row];
  const int lab32 = (int)lab;  // labels are below V, which is an int
  constexpr float LOG2E_F = 1.4426950408889634f;
  const float nl2 = -l * LOG2E_F;
  const int nvec = V / E;
  const bool vec = ((((size_t)lr) | ((size_t)dr)) & 15) == 0;
  if (vec) {
    // XENT_BWD_U vectors per thread, all loads first, and one such step per block (`chunks` blocks per row): the card
    // sees many short blocks instead of a loop per row.  Measured at 8192 rows x 128256 fp32: a loop per row 5.1 TB/s,
    // 4 vectors per thread in short blocks 5.7 TB/s, 1 vector per thread 5.9 TB/s
    constexpr int U = XENT_BWD_U;
    for (int v0 = chunk * (256 * U) + threadIdx.x; v0 < nvec; v0 += chunks * 256 * U) {
      float x[U][E];
#pragma unroll
      for (int u = 0; u < U; u++) {
        const int v = v0 + 256 * u;
        if (lab >= 0) load_f_nt<T, E>(lr + (int64_t)(v < nvec ? v : nvec - 1) * E, x[u]);
      }
#pragma unroll
      for (int u = 0; u < U; u++) {
        const int v = v0 + 256 * u;
        if (v < nvec) {
          // two instructions per element (an fma into log2 units and the exponential); the label's one-hot term is
          // taken off in the one vector that holds it (per-element 64-bit compares cost more than the stream)
          float o[E];
#pragma unroll
          for (int e = 0; e < E; e++) o[e] = lab32 < 0 ? 0.f : scale * __builtin_amdgcn_exp2f(__builtin_fmaf(x[u][e], LOG2E_F, nl2));
          if ((unsigned)(lab32 - v * E) < (unsigned)E) {
#pragma unroll
            for (int e = 0; e < E; e++)
              if (v * E + e == lab32) o[e] -= scale;
          }
          store_f_nt<T, E>(dr + (int64_t)v * E, o);
        }
      }
    }
  }
  if (chunk != 0) return;
  for (int c = (vec ? nvec * E : 0) + threadIdx.x; c < V; c += 256) {
    const float x = lab < 0 ? 0.f : Elem<T>::to_f(lr[c]);
    dr[c] = Elem<T>::from_f(lab < 0 ? 0.f : scale * (__expf(x - l) - (c == lab ? 1.f : 0.f)));
  }
}

}  // namespace tp

using namespace tp;

extern "C" int tp_l2norm_fwd(const void* x, void* y, float* rstd, int64_t rows, int dim, int64_t x_row_stride,
                             int64_t y_row_stride, float eps, int dtype, void* stream) {
  TP_REQUIRE(x && y && rstd, TP_ERR_BAD_ARG, "tp_l2norm_fwd: null pointer");
  TP_REQUIRE(rows >= 0 && dim > 0 && x_row_stride >= dim && y_row_stride >= dim, TP_ERR_BAD_ARG, "tp_l2norm_fwd: bad shape");
  if (rows == 0) return TP_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TP_BF16) return l2norm_launch<bf16_t>(false, x, x, y, rstd, rows, dim, x_row_stride, x_row_stride, y_row_stride, eps, st);
  if (dtype == TP_F16) return l2norm_launch<f16_t>(false, x, x, y, rstd, rows, dim, x_row_stride, x_row_stride, y_row_stride, eps, st);
  if (dtype == TP_F32) return l2norm_launch<float>(false, x, x, y, rstd, rows, dim, x_row_stride, x_row_stride, y_row_stride, eps, st);
  TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_l2norm_fwd: unsupported dtype %d", dtype);
}

extern "C" int tp_l2norm_bwd(const void* dy, const void* x, const float* rstd, void* dx, int64_t rows, int dim,
                             int64_t dy_row_stride, int64_t x_row_stride, int64_t dx_row_stride, int dtype, void* stream) {
  TP_REQUIRE(dy && x && rstd && dx, TP_ERR_BAD_ARG, "tp_l2norm_bwd: null pointer");
  TP_REQUIRE(rows >= 0 && dim > 0 && dy_row_stride >= dim && x_row_stride >= dim && dx_row_stride >= dim, TP_ERR_BAD_ARG,
             "tp_l2norm_bwd: bad shape");
  if (rows == 0) return TP_OK;
  hipStream_t st = (hipStream_t)stream;
  float* r = const_cast<float*>(rstd);
  if (dtype == TP_BF16) return l2norm_launch<bf16_t>(true, dy, x, dx, r, rows, dim, dy_row_stride, x_row_stride, dx_row_stride, 0.f, st);
  if (dtype == TP_F16) return l2norm_launch<f16_t>(true, dy, x, dx, r, rows, dim, dy_row_stride, x_row_stride, dx_row_stride, 0.f, st);
  if (dtype == TP_F32) return l2norm_launch<float>(true, dy, x, dx, r, rows, dim, dy_row_stride, x_row_stride, dx_row_stride, 0.f, st);
  TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_l2norm_bwd: unsupported dtype %d", dtype);
}

template <typename T>
static int scale_rows_typed(const void* x, const float* scale, void* y, int64_t rows, int dim, int64_t xs, int64_t ys, int heads,
                            int seq, hipStream_t st) {
  constexpr int E = 16 / sizeof(T);
  TP_REQUIRE(dim % E == 0, TP_ERR_UNSUPPORTED, "tp_scale_rows: dim=%d must be a multiple of %d", dim, E);
  TP_REQUIRE(aligned16(x) && aligned16(y) && (xs * (int64_t)sizeof(T)) % 16 == 0 && (ys * (int64_t)sizeof(T)) % 16 == 0, TP_ERR_BAD_ARG,
             "tp_scale_rows: pointers and row strides must keep rows 16-byte aligned");
  const int64_t n = rows * (dim / E);
  TP_REQUIRE((n + 255) / 256 < (1ll << 31), TP_ERR_UNSUPPORTED, "tp_scale_rows: too many elements");
  scale_rows_kernel<T><<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st>>>((const T*)x, scale, (T*)y, rows, dim, xs, ys, heads, seq);
  return check_launch("tp_scale_rows");
}

extern "C" int tp_scale_rows(const void* x, const float* scale, void* y, int64_t rows, int dim, int64_t x_row_stride,
                             int64_t y_row_stride, int heads, int seq, int dtype, void* stream) {
  TP_REQUIRE(x && scale && y, TP_ERR_BAD_ARG, "tp_scale_rows: null pointer");
  TP_REQUIRE(rows >= 0 && dim > 0 && heads > 0 && seq > 0 && x_row_stride >= dim && y_row_stride >= dim, TP_ERR_BAD_ARG,
             "tp_scale_rows: bad shape");
  if (rows == 0) return TP_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TP_BF16) return scale_rows_typed<bf16_t>(x, scale, y, rows, dim, x_row_stride, y_row_stride, heads, seq, st);
  if (dtype == TP_F16) return scale_rows_typed<f16_t>(x, scale, y, rows, dim, x_row_stride, y_row_stride, heads, seq, st);
  if (dtype == TP_F32) return scale_rows_typed<float>(x, scale, y, rows, dim, x_row_stride, y_row_stride, heads, seq, st);
  TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_scale_rows: unsupported dtype %d", dtype);
}

template <typename T>
static int swiglu_typed(bool backward, const void* dout, const void* gate, const void* up, void* o1, void* o2, int64_t rows,
                        int cols, int64_t dos, int64_t gs, int64_t us, int64_t o1s, int64_t o2s, hipStream_t st) {
  constexpr int E = 16 / sizeof(T);
  TP_REQUIRE(cols % E == 0, TP_ERR_UNSUPPORTED, "tp_swiglu: cols=%d must be a multiple of %d", cols, E);
  bool ok = aligned16(gate) && aligned16(up) && aligned16(o1) && aligned16(o2) && aligned16(dout);
  for (int64_t sdv : {dos, gs, us, o1s, o2s}) ok = ok && (sdv * (int64_t)sizeof(T)) % 16 == 0;
  TP_REQUIRE(ok, TP_ERR_BAD_ARG, "tp_swiglu: pointers and row strides must keep rows 16-byte aligned");
  const int64_t n = rows * (cols / E);
  TP_REQUIRE((n + 255) / 256 < (1ll << 31), TP_ERR_UNSUPPORTED, "tp_swiglu: too many elements");
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (backward)
    swiglu_bwd_kernel<T><<<grid, block, 0, st>>>((const T*)dout, (const T*)gate, (const T*)up, (T*)o1, (T*)o2, rows, cols, dos, gs,
                                                 us, o1s, o2s);
  else
    swiglu_fwd_kernel<T><<<grid, block, 0, st>>>((const T*)gate, (const T*)up, (T*)o1, rows, cols, gs, us, o1s);
  return check_launch("tp_swiglu");
}

extern "C" int tp_swiglu_fwd(const void* gate, const void* up, void* out, int64_t rows, int cols, int64_t gate_row_stride,
                             int64_t up_row_stride, int64_t out_row_stride, int dtype, void* stream) {
  TP_REQUIRE(gate && up && out, TP_ERR_BAD_ARG, "tp_swiglu_fwd: null pointer");
  TP_REQUIRE(rows >= 0 && cols > 0 && gate_row_stride >= cols && up_row_stride >= cols && out_row_stride >= cols, TP_ERR_BAD_ARG,
             "tp_swiglu_fwd: bad shape");
  if (rows == 0) return TP_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TP_BF16) return swiglu_typed<bf16_t>(false, nullptr, gate, up, out, nullptr, rows, cols, 0, gate_row_stride, up_row_stride, out_row_stride, 0, st);
  if (dtype == TP_F16) return swiglu_typed<f16_t>(false, nullptr, gate, up, out, nullptr, rows, cols, 0, gate_row_stride, up_row_stride, out_row_stride, 0, st);
  if (dtype == TP_F32) return swiglu_typed<float>(false, nullptr, gate, up, out, nullptr, rows, cols, 0, gate_row_stride, up_row_stride, out_row_stride, 0, st);
  TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_swiglu_fwd: unsupported dtype %d", dtype);
}

extern "C" int tp_swiglu_bwd(const void* dout, const void* gate, const void* up, void* dgate, void* dup, int64_t rows, int cols,
                             int64_t dout_row_stride, int64_t gate_row_stride, int64_t up_row_stride, int64_t dgate_row_stride,
                             int64_t dup_row_stride, int dtype, void* stream) {
  TP_REQUIRE(dout && gate && up && dgate && dup, TP_ERR_BAD_ARG, "tp_swiglu_bwd: null pointer");
  TP_REQUIRE(rows >= 0 && cols > 0 && dout_row_stride >= cols && gate_row_stride >= cols && up_row_stride >= cols &&
                 dgate_row_stride >= cols && dup_row_stride >= cols,
             TP_ERR_BAD_ARG, "tp_swiglu_bwd: bad shape");
  if (rows == 0) return TP_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TP_BF16) return swiglu_typed<bf16_t>(true, dout, gate, up, dgate, dup, rows, cols, dout_row_stride, gate_row_stride, up_row_stride, dgate_row_stride, dup_row_stride, st);
  if (dtype == TP_F16) return swiglu_typed<f16_t>(true, dout, gate, up, dgate, dup, rows, cols, dout_row_stride, gate_row_stride, up_row_stride, dgate_row_stride, dup_row_stride, st);
  if (dtype == TP_F32) return swiglu_typed<float>(true, dout, gate, up, dgate, dup, rows, cols, dout_row_stride, gate_row_stride, up_row_stride, dgate_row_stride, dup_row_stride, st);
  TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_swiglu_bwd: unsupported dtype %d", dtype);
}

extern "C" int tp_cross_entropy_fwd(const void* logits, const int64_t* labels, float* lse, float* row_loss, float* loss_and_count,
                                    int B, int S, int V, int64_t logits_b_stride, int64_t logits_s_stride,
                                    int64_t labels_b_stride, int ignore_index, int dtype, void* stream) {
  TP_REQUIRE(logits && labels && lse && row_loss && loss_and_count, TP_ERR_BAD_ARG, "tp_cross_entropy_fwd: null pointer");
  TP_REQUIRE(B > 0 && S > 0 && V > 0 && (int64_t)B * S < (1ll << 31), TP_ERR_BAD_ARG, "tp_cross_entropy_fwd: bad shape");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)(B * S)), block(256);
  if (dtype == TP_F32)
    xent_fwd_kernel<float><<<grid, block, 0, st>>>((const float*)logits, labels, lse, row_loss, S, V, logits_b_stride, logits_s_stride, labels_b_stride, ignore_index);
  else if (dtype == TP_BF16)
    xent_fwd_kernel<bf16_t><<<grid, block, 0, st>>>((const bf16_t*)logits, labels, lse, row_loss, S, V, logits_b_stride, logits_s_stride, labels_b_stride, ignore_index);
  else
    TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_cross_entropy_fwd: dtype %d (fp32 and bf16 logits only)", dtype);
  xent_mean_kernel<<<dim3(1), block, 0, st>>>(row_loss, labels, loss_and_count, B, S, V, labels_b_stride, ignore_index);
  return check_launch("tp_cross_entropy_fwd");
}

extern "C" int tp_cross_entropy_bwd(const void* logits, const int64_t* labels, const float* lse, const float* loss_and_count,
                                    const float* dloss, void* dlogits, int B, int S, int V, int64_t logits_b_stride,
                                    int64_t logits_s_stride, int64_t labels_b_stride, int64_t dlogits_b_stride,
                                    int64_t dlogits_s_stride, int ignore_index, int dtype, void* stream) {
  TP_REQUIRE(logits && labels && lse && loss_and_count && dloss && dlogits, TP_ERR_BAD_ARG, "tp_cross_entropy_bwd: null pointer");
  TP_REQUIRE(B > 0 && S > 0 && V > 0 && (int64_t)B * S < (1ll << 31), TP_ERR_BAD_ARG, "tp_cross_entropy_bwd: bad shape");
  hipStream_t st = (hipStream_t)stream;
  // (vectors per row / vectors per block, for the narrower element type's vector count at most 65535 blocks along y)
  const int64_t vec_per_row = (int64_t)V / (dtype == TP_F32 ? 4 : 8);
  int64_t chunks = std::max<int64_t>((vec_per_row + 256 * XENT_BWD_U - 1) / (256 * XENT_BWD_U), 1);
  chunks = std::min<int64_t>(chunks, ((1ll << 31) - 1) / ((int64_t)B * S));  // (rows x chunks blocks in a 1-D grid)
  const dim3 grid((unsigned)((int64_t)B * S * chunks)), block(256);
  if (dtype == TP_F32)
    xent_bwd_kernel<float><<<grid, block, 0, st>>>((const float*)logits, labels, lse, loss_and_count, dloss, (float*)dlogits, S, V, logits_b_stride, logits_s_stride, labels_b_stride, dlogits_b_stride, dlogits_s_stride, ignore_index, (int)chunks);
  else if (dtype == TP_BF16)
    xent_bwd_kernel<bf16_t><<<grid, block, 0, st>>>((const bf16_t*)logits, labels, lse, loss_and_count, dloss, (bf16_t*)dlogits, S, V, logits_b_stride, logits_s_stride, labels_b_stride, dlogits_b_stride, dlogits_s_stride, ignore_index, (int)chunks);
  else
    TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_cross_entropy_bwd: dtype %d (fp32 and bf16 logits only)", dtype);
  return check_launch("tp_cross_entropy_bwd");
}
