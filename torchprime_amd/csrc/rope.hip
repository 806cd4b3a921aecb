// Rotary position embedding for gfx950: cos/sin table build and the rotate-half apply on q and k in
// one launch.  HBM-bound: one pass, 16-byte loads/stores over strided (B,H,S,D) views.
//
// Table: LlamaRotaryEmbedding.forward (torchprime/torch_xla_models/model/llama/model.py:68-88),
//        DeepseekV3RotaryEmbedding.forward (model/deepseek_v3/model.py:57-75).
// Apply: rotate_half + apply_rotary_pos_emb (model/llama/model.py:91-122), the gather variant
//        (model/mixtral/model.py:115-140), apply_rotary_pos_emb_interleave
//        (model/deepseek_v3/model.py:84-103).
//
// The eager expression `(x * cos) + (rotate_half(x) * sin)` rounds each product and the sum to the
// tensor dtype; the kernel reproduces those three roundings so bf16 results match it bit for bit.
// The file is compiled with -ffp-contract=off so the fp32 path does not fuse mul+add either.
#include <type_traits>

#include "common.hpp"

namespace tp {

template <typename T>
__global__ __launch_bounds__(256) void rope_table_kernel(const float* __restrict__ inv_freq,
                                                         const float* __restrict__ pos, T* __restrict__ cos_o,
                                                         T* __restrict__ sin_o, int64_t n_rows, int half,
                                                         float scaling) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n_rows * half) return;
  const int64_t row = idx / half;
  const int i = (int)(idx - row * half);
  const float ang = inv_freq[i] * pos[row];
  const float c = cosf(ang) * scaling, s = sinf(ang) * scaling;
  const int64_t o = row * 2 * half + i;
  cos_o[o] = Elem<T>::from_f(c);
  cos_o[o + half] = Elem<T>::from_f(c);
  sin_o[o] = Elem<T>::from_f(s);
  sin_o[o + half] = Elem<T>::from_f(s);
}

// n / d for n < 2^31 with a multiplier computed on the host: q = mulhi(n, ceil(2^(31+l) / d)) >> (l - 1),
// l = ceil(log2 d).  One quarter-rate multiply instead of the two dozen instructions of a runtime divide;
// this kernel is close enough to the VALU limit for that to show.
struct FastDiv {
  unsigned d, m, sh;
};
static inline FastDiv fast_div(unsigned d) {
  FastDiv f = {d, 0u, 0u};
  if (d > 1) {
    unsigned l = 0;
    while ((1ull << l) < d) l++;
    f.m = (unsigned)(((1ull << (31 + l)) + d - 1) / d);
    f.sh = l - 1;
  }
  return f;
}
__device__ __forceinline__ unsigned div_by(unsigned n, const FastDiv& f) {
  return f.d == 1 ? n : (__umulhi(n, f.m) >> f.sh);
}

struct RopeArgs {
  const void* x[2];
  void* y[2];
  int64_t xs[2][3];  // element strides (b, h, s)
  int64_t ys[2][3];
  int H[2];
  unsigned nblk0;    // blocks that work on x[0]; the rest work on x[1]
  FastDiv dH[2], dVH;
  const void* cos;
  const void* sin;
  const int64_t* pos;
  int64_t cs_b, cs_s, pos_b, table_rows;
  int B, S, D;
};

// One thread = one 16-byte vector of the first half and its partner in the second half (E rotation
// pairs).  A block works on one tensor (q or k) of one batch element (blockIdx.y); inside it the work
// items are numbered (s * H + h) * VH + j so a wave sweeps the heads of one token, which are contiguous
// in (B,S,H,D) memory.  Which tensor, the batch offset and all strides are wave-uniform, so they stay
// on the scalar unit; WIDE = false keeps the per-lane offsets in 32 bits (every offset inside a batch
// element below 2^31 elements, checked on the host).
// MODE 0: rotate-half on [first half | second half] (Llama, Mixtral).  MODE 1: the input is first permuted
// [x0,x1,x2,...] -> [evens | odds] and the output stays in that order (DeepSeek).  MODE 2: adjacent pairs
// (x[2i], x[2i+1]) are rotated by angle i and written back in place, using the first half of the cos/sin row for both
// members of a pair (Llama-4 apply_rotary_emb, model/llama4/model.py:364-409).
template <typename T, int MODE, bool BACKWARD, bool WIDE>
__global__ __launch_bounds__(256) void rope_apply_kernel(RopeArgs a) {
  constexpr bool LOAD_PAIRS = MODE == 1 && !BACKWARD;   // de-interleave while loading
  constexpr bool STORE_PAIRS = MODE == 1 && BACKWARD;   // re-interleave while storing
  constexpr int E = 16 / sizeof(T);
  typedef typename std::conditional<WIDE, int64_t, unsigned>::type off_t;
  const int half = a.D / 2;
  const int which = blockIdx.x >= a.nblk0 ? 1 : 0;
  const unsigned blk = blockIdx.x - (which ? a.nblk0 : 0u);
  const int b = blockIdx.y;
  const int H = a.H[which];
  const unsigned lin = blk * 256u + threadIdx.x;
  const unsigned u = div_by(lin, a.dVH);
  const int j = (int)(lin - u * a.dVH.d);
  const unsigned s = div_by(u, a.dH[which]);
  const unsigned h = u - s * (unsigned)H;
  if (s >= (unsigned)a.S) return;

  const T* xp = (const T*)a.x[which] + b * a.xs[which][0] + (off_t)h * (off_t)a.xs[which][1] + (off_t)s * (off_t)a.xs[which][2];
  T* yp = (T*)a.y[which] + b * a.ys[which][0] + (off_t)h * (off_t)a.ys[which][1] + (off_t)s * (off_t)a.ys[which][2];
  const T *cp, *sp;
  if (a.pos) {
    // (positions outside the table are clamped so that no lane reads beyond it; the host side has already
    // rejected them the way the reference's cos[position_ids] does)
    int64_t p = a.pos[b * a.pos_b + s];
    p = p < 0 ? 0 : (p >= a.table_rows ? a.table_rows - 1 : p);
    const int64_t crow = a.cs_s * p;
    cp = (const T*)a.cos + crow;
    sp = (const T*)a.sin + crow;
  } else {
    const off_t crow = (off_t)s * (off_t)a.cs_s;
    cp = (const T*)a.cos + a.cs_b * b + crow;
    sp = (const T*)a.sin + a.cs_b * b + crow;
  }

  if constexpr (MODE == 2) {
    // A 16-byte chunk holds E/2 whole pairs, so the thread's two chunks (same addresses as in the other modes)
    // are rotated independently: chunk at j*E covers pairs j*E/2.., chunk at half + j*E pairs D/4 + j*E/2..,
    // and pair p takes entry p of the cos / sin row.
    constexpr int P = E / 2;
#pragma unroll
    for (int ch = 0; ch < 2; ch++) {
      const int eoff = ch * half + j * E, poff = ch * (half / 2) + j * P;
      float v[E], c[P], sn[P], o[E];
      load_f_nt<T, E>(xp + eoff, v);
      load_f<T, P>(cp + poff, c);
      load_f<T, P>(sp + poff, sn);
#pragma unroll
      for (int e = 0; e < P; e++) {
        const float x = v[2 * e], y = v[2 * e + 1];
        if (!BACKWARD) {
          o[2 * e] = round_to<T>(round_to<T>(x * c[e]) + round_to<T>(-y * sn[e]));
          o[2 * e + 1] = round_to<T>(round_to<T>(y * c[e]) + round_to<T>(x * sn[e]));
        } else {
          o[2 * e] = round_to<T>(x * c[e]) + round_to<T>(y * sn[e]);
          o[2 * e + 1] = round_to<T>(y * c[e]) + round_to<T>(-x * sn[e]);
        }
      }
      store_f_nt<T, E>(yp + eoff, o);
    }
    return;
  }
  float c1[E], c2[E], s1[E], s2[E];
  load_f<T, E>(cp + j * E, c1);
  load_f<T, E>(cp + half + j * E, c2);
  load_f<T, E>(sp + j * E, s1);
  load_f<T, E>(sp + half + j * E, s2);

  float x1[E], x2[E], o1[E], o2[E];
  if (!LOAD_PAIRS) {
    load_f_nt<T, E>(xp + j * E, x1);
    load_f_nt<T, E>(xp + half + j * E, x2);
  } else {
    // permuted input: first-half element i is x[2i], second-half element i is x[2i+1]
    float lo[E], hi[E];
    load_f_nt<T, E>(xp + 2 * j * E, lo);
    load_f_nt<T, E>(xp + 2 * j * E + E, hi);
#pragma unroll
    for (int e = 0; e < E / 2; e++) {
      x1[e] = lo[2 * e];
      x2[e] = lo[2 * e + 1];
      x1[E / 2 + e] = hi[2 * e];
      x2[E / 2 + e] = hi[2 * e + 1];
    }
  }
#pragma unroll
  for (int e = 0; e < E; e++) {
    if (!BACKWARD) {
      // out[i] = x[i] cos[i] + (-x[i+h]) sin[i];  out[i+h] = x[i+h] cos[i+h] + x[i] sin[i+h]
      o1[e] = round_to<T>(round_to<T>(x1[e] * c1[e]) + round_to<T>(-x2[e] * s1[e]));
      o2[e] = round_to<T>(round_to<T>(x2[e] * c2[e]) + round_to<T>(x1[e] * s2[e]));
    } else {
      // dx[i] = g[i] cos[i] + g[i+h] sin[i+h];  dx[i+h] = g[i+h] cos[i+h] - g[i] sin[i]
      // (autograd forms the two products and their sum in the tensor dtype as well)
      o1[e] = round_to<T>(x1[e] * c1[e]) + round_to<T>(x2[e] * s2[e]);
      o2[e] = round_to<T>(x2[e] * c2[e]) + round_to<T>(-x1[e] * s1[e]);
    }
  }
  if (!STORE_PAIRS) {
    store_f_nt<T, E>(yp + j * E, o1);
    store_f_nt<T, E>(yp + half + j * E, o2);
  } else {
    // inverse permutation: dx[2i] = d_first[i], dx[2i+1] = d_second[i]
    float lo[E], hi[E];
#pragma unroll
    for (int e = 0; e < E / 2; e++) {
      lo[2 * e] = o1[e];
      lo[2 * e + 1] = o2[e];
      hi[2 * e] = o1[E / 2 + e];
      hi[2 * e + 1] = o2[E / 2 + e];
    }
    store_f_nt<T, E>(yp + 2 * j * E, lo);
    store_f_nt<T, E>(yp + 2 * j * E + E, hi);
  }
}

template <typename T, bool WIDE>
static void rope_launch(const RopeArgs& a, int interleaved, int backward, dim3 grid, hipStream_t st) {
  const dim3 block(256);
  if (interleaved == 0 && !backward) rope_apply_kernel<T, 0, false, WIDE><<<grid, block, 0, st>>>(a);
  else if (interleaved == 0 && backward) rope_apply_kernel<T, 0, true, WIDE><<<grid, block, 0, st>>>(a);
  else if (interleaved == 1 && !backward) rope_apply_kernel<T, 1, false, WIDE><<<grid, block, 0, st>>>(a);
  else if (interleaved == 1 && backward) rope_apply_kernel<T, 1, true, WIDE><<<grid, block, 0, st>>>(a);
  else if (!backward) rope_apply_kernel<T, 2, false, WIDE><<<grid, block, 0, st>>>(a);
  else rope_apply_kernel<T, 2, true, WIDE><<<grid, block, 0, st>>>(a);
}

template <typename T>
static int rope_typed(RopeArgs& a, int interleaved, int backward, hipStream_t st) {
  constexpr int E = 16 / sizeof(T);
  const int VH = a.D / 2 / E;
  if (a.B == 0 || a.S == 0) return TP_OK;
  const int64_t lim = 1ll << 31;
  const int64_t items0 = (int64_t)a.S * a.H[0] * VH, items1 = (int64_t)a.S * a.H[1] * VH;
  TP_REQUIRE(items0 < lim - 256 && items1 < lim - 256 && a.B <= 65535, TP_ERR_UNSUPPORTED,
             "tp_rope_apply: more than 2^31 16-byte vectors per batch element, or batch > 65535");
  const unsigned nb0 = (unsigned)((items0 + 255) / 256), nb1 = (unsigned)((items1 + 255) / 256);
  a.nblk0 = nb0;
  a.dVH = fast_div((unsigned)VH);
  a.dH[0] = fast_div((unsigned)a.H[0]);
  a.dH[1] = fast_div((unsigned)(a.H[1] > 0 ? a.H[1] : 1));
  // 32-bit per-lane offsets when every offset inside one batch element stays below 2^31 elements
  bool narrow = a.cs_s >= 0 && (int64_t)a.S * a.cs_s < lim;
  for (int w = 0; w < 2; w++)
    for (int i = 1; i < 3; i++) narrow = narrow && a.xs[w][i] >= 0 && a.ys[w][i] >= 0;
  for (int w = 0; w < 2 && narrow; w++)
    narrow = a.H[w] * a.xs[w][1] + a.S * a.xs[w][2] < lim && a.H[w] * a.ys[w][1] + a.S * a.ys[w][2] < lim;
  const dim3 grid(nb0 + nb1, (unsigned)a.B);
  if (narrow) rope_launch<T, false>(a, interleaved, backward, grid, st);
  else rope_launch<T, true>(a, interleaved, backward, grid, st);
  return check_launch("tp_rope_apply");
}

}  // namespace tp

using namespace tp;

extern "C" int tp_rope_table(const float* inv_freq, const float* position_ids, void* cos, void* sin, int Bp, int S,
                             int half, float attention_scaling, int dtype, void* stream) {
  TP_REQUIRE(inv_freq && position_ids && cos && sin, TP_ERR_BAD_ARG, "tp_rope_table: null pointer");
  TP_REQUIRE(Bp >= 0 && S >= 0 && half > 0, TP_ERR_BAD_ARG, "tp_rope_table: bad shape Bp=%d S=%d half=%d", Bp, S, half);
  const int64_t rows = (int64_t)Bp * S;
  if (rows == 0) return TP_OK;
  const dim3 grid((unsigned)((rows * half + 255) / 256)), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TP_BF16) rope_table_kernel<bf16_t><<<grid, block, 0, st>>>(inv_freq, position_ids, (bf16_t*)cos, (bf16_t*)sin, rows, half, attention_scaling);
  else if (dtype == TP_F16) rope_table_kernel<f16_t><<<grid, block, 0, st>>>(inv_freq, position_ids, (f16_t*)cos, (f16_t*)sin, rows, half, attention_scaling);
  else if (dtype == TP_F32) rope_table_kernel<float><<<grid, block, 0, st>>>(inv_freq, position_ids, (float*)cos, (float*)sin, rows, half, attention_scaling);
  else TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_rope_table: unsupported dtype %d", dtype);
  return check_launch("tp_rope_table");
}

extern "C" int tp_rope_apply(const void* q, const void* k, const void* cos, const void* sin, const int64_t* pos,
                             void* q_out, void* k_out, int B, int Hq, int Hkv, int S, int D, const int64_t q_strides[3],
                             const int64_t k_strides[3], const int64_t qo_strides[3], const int64_t ko_strides[3],
                             int64_t cs_b_stride, int64_t cs_s_stride, int64_t pos_b_stride, int64_t table_rows,
                             int interleaved, int backward, int dtype, void* stream) {
  TP_REQUIRE(q && q_out && cos && sin && q_strides && qo_strides, TP_ERR_BAD_ARG, "tp_rope_apply: null pointer");
  TP_REQUIRE((k == nullptr) == (Hkv == 0), TP_ERR_BAD_ARG, "tp_rope_apply: k must be NULL exactly when Hkv == 0");
  TP_REQUIRE(Hkv == 0 || (k_out && k_strides && ko_strides), TP_ERR_BAD_ARG, "tp_rope_apply: null k output/strides");
  TP_REQUIRE(B >= 0 && Hq > 0 && Hkv >= 0 && S >= 0 && D > 0, TP_ERR_BAD_ARG, "tp_rope_apply: bad shape");
  TP_REQUIRE(interleaved >= 0 && interleaved <= 2, TP_ERR_BAD_ARG, "tp_rope_apply: interleaved must be 0, 1 or 2");
  TP_REQUIRE(!pos || table_rows > 0, TP_ERR_BAD_ARG, "tp_rope_apply: a position gather needs the table's row count");
  const int esz = dtype == TP_F32 ? 4 : 2;
  TP_REQUIRE(dtype == TP_BF16 || dtype == TP_F16 || dtype == TP_F32, TP_ERR_UNSUPPORTED, "tp_rope_apply: unsupported dtype %d", dtype);
  const int E = 16 / esz;
  TP_REQUIRE(D % (2 * E) == 0, TP_ERR_UNSUPPORTED, "tp_rope_apply: D=%d must be a multiple of %d", D, 2 * E);
  RopeArgs a;
  a.x[0] = q; a.x[1] = k; a.y[0] = q_out; a.y[1] = k_out;
  a.H[0] = Hq; a.H[1] = Hkv;
  bool ok = aligned16(q) && aligned16(q_out) && aligned16(cos) && aligned16(sin) && aligned16(k) && aligned16(k_out);
  for (int i = 0; i < 3; i++) {
    a.xs[0][i] = q_strides[i]; a.ys[0][i] = qo_strides[i];
    a.xs[1][i] = Hkv ? k_strides[i] : 0; a.ys[1][i] = Hkv ? ko_strides[i] : 0;
    ok = ok && (a.xs[0][i] * esz) % 16 == 0 && (a.ys[0][i] * esz) % 16 == 0 && (a.xs[1][i] * esz) % 16 == 0 &&
         (a.ys[1][i] * esz) % 16 == 0;
  }
  ok = ok && (cs_b_stride * esz) % 16 == 0 && (cs_s_stride * esz) % 16 == 0;
  TP_REQUIRE(ok, TP_ERR_BAD_ARG, "tp_rope_apply: pointers and strides must keep rows 16-byte aligned");
  a.cos = cos; a.sin = sin; a.pos = pos;
  a.cs_b = cs_b_stride; a.cs_s = cs_s_stride; a.pos_b = pos_b_stride; a.table_rows = table_rows;
  a.B = B; a.S = S; a.D = D;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TP_BF16) return rope_typed<bf16_t>(a, interleaved, backward, st);
  if (dtype == TP_F16) return rope_typed<f16_t>(a, interleaved, backward, st);
  return rope_typed<float>(a, interleaved, backward, st);
}
