// Attention backward in fp32 for gfx950: fp32 operands and accumulation on v_mfma_f32_32x32x2_f32.
//
// The counterpart of attn_fwd_f32.hip: autograd through the reference's eager branch on fp32 tensors
// (torchprime/torch_xla_models/attention.py:151-170) without any 16-bit rounding.  Same split as the 16-bit backward
// (attn_bwd.hip): delta = rowsum(dO o O), then a dQ kernel (one workgroup per 128 query rows of a head) and a
// dK/dV kernel (one workgroup per 128 kv rows of a kv head, looping over the query heads of its group), no atomics.
// Causal / full, segment ids, GQA, explicit scale.  Sized for correctness at small shapes, not tuned.
//
// v_mfma_f32_32x32x2_f32 (wave64; ln = lane % 32, g = lane / 32):
//   A (32 x 2): lane holds row ln, k = g        B (2 x 32): lane holds column ln, k = g
//   C (32 x 32): lane holds column ln, rows r(v) = 8*(v/4) + 4*g + v%4 for v = 0..15
// Two kinds of products, as in the forward:
//   "row" products  C[m][n] = sum_d X[m][d] Y[n][d]: lane group g takes head-dim half g, step st pairs X[ln][g*HD+st]
//                   with Y[ln][g*HD+st] (X from LDS, Y in registers);
//   "C-fed" products C2[d][n] += sum_m X[m][d] C[m][n] with C straight from the accumulator layout: step v pairs
//                   X[r(v)][d-block*32 + ln] (from LDS) with the lane's value v of C.
#include "attn_common.hpp"

namespace tp {

struct BwdArgs32 {
  const float* q;
  const float* k;
  const float* v;
  const float* out;
  const float* dout;
  const float* lse;
  const int32_t* seg;
  float* dq;
  float* dk;
  float* dv;
  float* delta;
  int B, Hq, Hkv, Sq, Skv, n_rep;
  int64_t qs[3], ks[3], vs[3], os[3], dos[3], dqs[3], dks[3], dvs[3];
  float scale_log2, sm_scale;
  int causal;
  MaskExt mx;   // as in the forward
  float cap2;
};

// delta[b, h, q] = sum_d dO[q][d] * O[q][d]
template <int D>
__global__ __launch_bounds__(256) void attn_delta_f32_kernel(const BwdArgs32 a) {
  const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t rows = (int64_t)a.B * a.Hq * a.Sq;
  if (row >= rows) return;
  const int q = (int)(row % a.Sq);
  const int64_t bh = row / a.Sq;
  const int h = (int)(bh % a.Hq), b = (int)(bh / a.Hq);
  const float* o = a.out + b * a.os[0] + h * a.os[1] + (int64_t)q * a.os[2];
  const float* d = a.dout + b * a.dos[0] + h * a.dos[1] + (int64_t)q * a.dos[2];
  float acc = 0.f;
#pragma unroll 4
  for (int c = 0; c < D; c += 4) {
    const f32x4 x = *(const f32x4*)(o + c), y = *(const f32x4*)(d + c);
    acc += x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3];
  }
  a.delta[row] = acc;
}

// stage rows r0 .. r0+31 of a (rows, D) matrix with row stride `stride` into LDS rows of STRIDE floats (zeros past n)
template <int D, int STRIDE>
__device__ __forceinline__ void stage32(float* dst, const float* src, int64_t stride, int r0, int n, int tid) {
  for (int c = tid; c < 32 * (D / 4); c += 256) {
    const int r = c / (D / 4), cc = (c % (D / 4)) * 4;
    f32x4 x = {0.f, 0.f, 0.f, 0.f};
    if (r0 + r < n) x = *(const f32x4*)(src + (int64_t)(r0 + r) * stride + cc);
    *(f32x4*)(dst + r * STRIDE + cc) = x;
  }
}

template <int D>
__global__ __launch_bounds__(256) void attn_bwd_dq_f32_kernel(const BwdArgs32 a) {
  constexpr int BN = 32, BM = 128, DB = D / 32, HD = D / 2, STRIDE = D + 4;
  __shared__ __align__(16) float ksm[BN * STRIDE];
  __shared__ __align__(16) float vsm[BN * STRIDE];
  __shared__ int ssm[BN];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, ln = lane & 31;
  const int n_qt = (a.Sq + BM - 1) / BM;
  const int qt = blockIdx.x % n_qt, bh = blockIdx.x / n_qt;
  const int h = bh % a.Hq, b = bh / a.Hq, hk = h / a.n_rep;
  const int q0 = qt * BM, wq0 = q0 + wave * 32;
  const int Sq = a.Sq, Skv = a.Skv;
  const int qrow = wq0 + ln, qrow_c = min(qrow, Sq - 1);
  const float* kb = a.k + b * a.ks[0] + hk * a.ks[1];
  const float* vb = a.v + b * a.vs[0] + hk * a.vs[1];
  const int32_t* segb = a.seg ? a.seg + (int64_t)b * Skv : nullptr;
  const int segq = segb ? segb[qrow_c] : 0;
  // Q (pre-multiplied by the scale in log2 units) and dO fragments of this lane's query row, head-dim half g
  float qf[HD], dof[HD];
  {
    const float* qp = a.q + b * a.qs[0] + h * a.qs[1] + (int64_t)qrow_c * a.qs[2] + g * HD;
    const float* dp = a.dout + b * a.dos[0] + h * a.dos[1] + (int64_t)qrow_c * a.dos[2] + g * HD;
#pragma unroll
    for (int s = 0; s < HD; s += 4) {
      const f32x4 t = *(const f32x4*)(qp + s), u = *(const f32x4*)(dp + s);
#pragma unroll
      for (int e = 0; e < 4; e++) { qf[s + e] = t[e] * a.scale_log2; dof[s + e] = u[e]; }
    }
  }
  const int64_t ro = ((int64_t)b * a.Hq + h) * Sq + qrow_c;
  const float lraw = a.lse[ro];
  const float lse2 = (lraw == -INFINITY) ? INFINITY : lraw * LOG2E;  // rows without an allowed key: P = 0
  const float delta = a.delta[ro];
  f32x16 dqacc[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int v = 0; v < 16; v++) dqacc[d][v] = 0.f;

  const int qp = a.mx.on ? (a.mx.qpos ? a.mx.qpos[qrow_c] : qrow_c) : 0;
  const int band_lo = a.mx.on ? qp - a.mx.lo_off : -BAND_INF, band_hi = a.mx.on ? qp + a.mx.hi_off : BAND_INF;
  const float* bias_row = a.mx.bias ? a.mx.bias + b * a.mx.bias_s[0] + h * a.mx.bias_s[1] + (int64_t)qrow_c * a.mx.bias_s[2] : nullptr;
  const int kv_end = a.causal ? min(Skv, q0 + BM) : Skv;
  const int ntiles = (kv_end + BN - 1) / BN;
  for (int t = 0; t < ntiles; t++) {
    const int kv0 = t * BN;
    __syncthreads();
    stage32<D, STRIDE>(ksm, kb, a.ks[2], kv0, Skv, tid);
    stage32<D, STRIDE>(vsm, vb, a.vs[2], kv0, Skv, tid);
    if (segb && tid < BN) ssm[tid] = segb[min(kv0 + tid, Skv - 1)];
    __syncthreads();
    if (a.causal && kv0 > wq0 + 31) continue;  // (uniform per wave; the barriers above are outside)
    // S^T = K Q^T and dP^T = V dO^T: rows = kv, column = this lane's query
    f32x16 s, dp;
#pragma unroll
    for (int v = 0; v < 16; v++) { s[v] = 0.f; dp[v] = 0.f; }
    const float* kr = ksm + ln * STRIDE + g * HD;
    const float* vr = vsm + ln * STRIDE + g * HD;
#pragma unroll
    for (int st = 0; st < HD; st += 4) {
      const f32x4 k4 = *(const f32x4*)(kr + st), v4 = *(const f32x4*)(vr + st);
#pragma unroll
      for (int e = 0; e < 4; e++) {
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(k4[e], qf[st + e], s, 0, 0, 0);
        dp = __builtin_amdgcn_mfma_f32_32x32x2f32(v4[e], dof[st + e], dp, 0, 0, 0);
      }
    }
    // dS^T = P o (dP^T - delta), P = exp2(S^T - LSE) on allowed pairs
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int kvl = 8 * (v / 4) + 4 * g + (v % 4), kv = kv0 + kvl;
      const bool ok = kv < Skv && (!a.causal || kv <= qrow) && (!segb || ssm[kvl] == segq) && kv >= band_lo && kv <= band_hi;
      float sv = s[v], fac = 1.f;
      if (a.cap2 != 0.f) {
        const float th = tanhf(sv / a.cap2);
        sv = a.cap2 * th;
        fac = 1.f - th * th;  // derivative of the capped score with respect to the raw one
      }
      if (bias_row) sv += LOG2E * bias_row[min(kv, Skv - 1)];  // additive mask (-inf stays -inf)
      const float p = ok ? exp2f(sv - lse2) : 0.f;
      s[v] = p * (dp[v] - delta) * fac;
    }
    // dQ^T += K^T dS^T
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int kvl = 8 * (v / 4) + 4 * g + (v % 4);
#pragma unroll
      for (int d = 0; d < DB; d++) dqacc[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(ksm[kvl * STRIDE + d * 32 + ln], s[v], dqacc[d], 0, 0, 0);
    }
  }
  if (qrow < Sq) {
    float* dqp = a.dq + b * a.dqs[0] + h * a.dqs[1] + (int64_t)qrow * a.dqs[2];
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int vq = 0; vq < 4; vq++) {
        const f32x16& o = dqacc[d];
        *(f32x4*)(dqp + d * 32 + 8 * vq + 4 * g) =
            f32x4{o[4 * vq] * a.sm_scale, o[4 * vq + 1] * a.sm_scale, o[4 * vq + 2] * a.sm_scale, o[4 * vq + 3] * a.sm_scale};
      }
  }
}

template <int D>
__global__ __launch_bounds__(256) void attn_bwd_dkdv_f32_kernel(const BwdArgs32 a) {
  constexpr int BMQ = 32, BNK = 128, DB = D / 32, HD = D / 2, STRIDE = D + 4;
  __shared__ __align__(16) float qsm[BMQ * STRIDE];
  __shared__ __align__(16) float dosm[BMQ * STRIDE];
  __shared__ float lsm[BMQ], dsm[BMQ];
  __shared__ int ssm[BMQ], psm[BMQ];  // segment ids and key-order positions of the tile's query rows
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, ln = lane & 31;
  const int n_kt = (a.Skv + BNK - 1) / BNK;
  const int kt = blockIdx.x % n_kt, bg = blockIdx.x / n_kt;
  const int hk = bg % a.Hkv, b = bg / a.Hkv;
  const int kv0 = kt * BNK, wkv0 = kv0 + wave * 32;
  const int Sq = a.Sq, Skv = a.Skv;
  const int kvcol = wkv0 + ln, kvcol_c = min(kvcol, Skv - 1);
  const int32_t* segb = a.seg ? a.seg + (int64_t)b * Skv : nullptr;
  const int segk = segb ? segb[kvcol_c] : 0;
  // K (pre-multiplied by the scale in log2 units) and V fragments of this lane's kv row, head-dim half g
  float kf[HD], vf[HD];
  {
    const float* kp = a.k + b * a.ks[0] + hk * a.ks[1] + (int64_t)kvcol_c * a.ks[2] + g * HD;
    const float* vp = a.v + b * a.vs[0] + hk * a.vs[1] + (int64_t)kvcol_c * a.vs[2] + g * HD;
#pragma unroll
    for (int s = 0; s < HD; s += 4) {
      const f32x4 t = *(const f32x4*)(kp + s), u = *(const f32x4*)(vp + s);
#pragma unroll
      for (int e = 0; e < 4; e++) { kf[s + e] = t[e] * a.scale_log2; vf[s + e] = u[e]; }
    }
  }
  f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int v = 0; v < 16; v++) { dkacc[d][v] = 0.f; dvacc[d][v] = 0.f; }

  const int nqt = (Sq + BMQ - 1) / BMQ;
  const int qt_first = a.causal ? min(kv0 / BMQ, nqt) : 0;
  for (int hl = 0; hl < a.n_rep; hl++) {
    const int h = hk * a.n_rep + hl;
    const float* qb = a.q + b * a.qs[0] + h * a.qs[1];
    const float* dob = a.dout + b * a.dos[0] + h * a.dos[1];
    const int64_t ro = ((int64_t)b * a.Hq + h) * Sq;
    const float* bias_head = a.mx.bias ? a.mx.bias + b * a.mx.bias_s[0] + h * a.mx.bias_s[1] : nullptr;
    for (int qt = qt_first; qt < nqt; qt++) {
      const int qi0 = qt * BMQ;
      __syncthreads();
      stage32<D, STRIDE>(qsm, qb, a.qs[2], qi0, Sq, tid);
      stage32<D, STRIDE>(dosm, dob, a.dos[2], qi0, Sq, tid);
      if (tid < BMQ) {
        const int qr = min(qi0 + tid, Sq - 1);
        const float lraw = a.lse[ro + qr];
        lsm[tid] = (lraw == -INFINITY) ? INFINITY : lraw * LOG2E;
        dsm[tid] = a.delta[ro + qr];
        ssm[tid] = segb ? segb[qr] : 0;
        psm[tid] = a.mx.qpos ? a.mx.qpos[qr] : qr;
      }
      __syncthreads();
      if ((a.causal && qi0 + BMQ - 1 < wkv0) || wkv0 >= Skv) continue;  // (uniform per wave)
      // S = Q K^T and dP = dO V^T: rows = queries, column = this lane's kv row
      f32x16 s, dp;
#pragma unroll
      for (int v = 0; v < 16; v++) { s[v] = 0.f; dp[v] = 0.f; }
      const float* qr_ = qsm + ln * STRIDE + g * HD;
      const float* dr_ = dosm + ln * STRIDE + g * HD;
#pragma unroll
      for (int st = 0; st < HD; st += 4) {
        const f32x4 q4 = *(const f32x4*)(qr_ + st), d4 = *(const f32x4*)(dr_ + st);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          s = __builtin_amdgcn_mfma_f32_32x32x2f32(q4[e], kf[st + e], s, 0, 0, 0);
          dp = __builtin_amdgcn_mfma_f32_32x32x2f32(d4[e], vf[st + e], dp, 0, 0, 0);
        }
      }
      // P and dS = P o (dP - delta); rows of the C tile are queries
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int r = 8 * (v / 4) + 4 * g + (v % 4), qrow = qi0 + r;
        bool ok = qrow < Sq && kvcol < Skv && (!a.causal || kvcol <= qrow) && (!segb || ssm[r] == segk);
        if (a.mx.on) ok = ok && kvcol >= psm[r] - a.mx.lo_off && kvcol <= psm[r] + a.mx.hi_off;
        float sv = s[v], fac = 1.f;
        if (a.cap2 != 0.f) {
          const float th = tanhf(sv / a.cap2);
          sv = a.cap2 * th;
          fac = 1.f - th * th;
        }
        if (bias_head) sv += LOG2E * bias_head[(int64_t)min(qrow, Sq - 1) * a.mx.bias_s[2] + min(kvcol, Skv - 1)];  // additive mask
        const float p = ok ? exp2f(sv - lsm[r]) : 0.f;
        s[v] = p;
        dp[v] = p * (dp[v] - dsm[r]) * fac;
      }
      // dV^T += dO^T P,  dK^T += Q^T dS
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int r = 8 * (v / 4) + 4 * g + (v % 4);
#pragma unroll
        for (int d = 0; d < DB; d++) {
          dvacc[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(dosm[r * STRIDE + d * 32 + ln], s[v], dvacc[d], 0, 0, 0);
          dkacc[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(qsm[r * STRIDE + d * 32 + ln], dp[v], dkacc[d], 0, 0, 0);
        }
      }
    }
  }
  if (kvcol < Skv) {
    float* dkp = a.dk + b * a.dks[0] + hk * a.dks[1] + (int64_t)kvcol * a.dks[2];
    float* dvp = a.dv + b * a.dvs[0] + hk * a.dvs[1] + (int64_t)kvcol * a.dvs[2];
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int vq = 0; vq < 4; vq++) {
        const f32x16& x = dkacc[d];
        const f32x16& y = dvacc[d];
        *(f32x4*)(dkp + d * 32 + 8 * vq + 4 * g) =
            f32x4{x[4 * vq] * a.sm_scale, x[4 * vq + 1] * a.sm_scale, x[4 * vq + 2] * a.sm_scale, x[4 * vq + 3] * a.sm_scale};
        *(f32x4*)(dvp + d * 32 + 8 * vq + 4 * g) = f32x4{y[4 * vq], y[4 * vq + 1], y[4 * vq + 2], y[4 * vq + 3]};
      }
  }
}

template <int D>
static int launch_bwd_f32(const BwdArgs32& a, hipStream_t st) {
  const int64_t rows = (int64_t)a.B * a.Hq * a.Sq;
  attn_delta_f32_kernel<D><<<dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, st>>>(a);
  int rc = check_launch("tp_attn_bwd(fp32 delta)");
  if (rc) return rc;
  attn_bwd_dkdv_f32_kernel<D><<<dim3((unsigned)((int64_t)a.B * a.Hkv * ((a.Skv + 127) / 128))), dim3(256), 0, st>>>(a);
  rc = check_launch("tp_attn_bwd(fp32 dkdv)");
  if (rc) return rc;
  attn_bwd_dq_f32_kernel<D><<<dim3((unsigned)((int64_t)a.B * a.Hq * ((a.Sq + 127) / 128))), dim3(256), 0, st>>>(a);
  return check_launch("tp_attn_bwd(fp32 dq)");
}

// called by tp_attn_bwd for TP_F32 inputs (pointers, sizes and Hq % Hkv already validated there)
int attn_bwd_f32(const void* dout, const void* q, const void* k, const void* v, const void* out, const float* lse,
                 const int32_t* seg, void* dq, void* dk, void* dv, float* ws, int B, int Hq, int Hkv, int Sq, int Skv, int Dqk,
                 int Dv, const int64_t* dos, const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                 const int64_t* dqs, const int64_t* dks, const int64_t* dvs, float sm_scale, int causal, hipStream_t st,
                 const MaskExt& mx) {
  TP_REQUIRE(Dqk == Dv && (Dqk == 64 || Dqk == 128), TP_ERR_UNSUPPORTED,
             "tp_attn_bwd: fp32 attention is built for head dims 64 and 128 (got qk=%d, v=%d)", Dqk, Dv);
  BwdArgs32 a;
  a.q = (const float*)q; a.k = (const float*)k; a.v = (const float*)v; a.out = (const float*)out; a.dout = (const float*)dout;
  a.lse = lse; a.seg = seg; a.dq = (float*)dq; a.dk = (float*)dk; a.dv = (float*)dv; a.delta = ws;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.Sq = Sq; a.Skv = Skv; a.n_rep = Hq / Hkv;
  bool ok = aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out) && aligned16(dout) && aligned16(dq) && aligned16(dk) && aligned16(dv);
  for (int i = 0; i < 3; i++) {
    a.qs[i] = qs[i]; a.ks[i] = ks[i]; a.vs[i] = vs[i]; a.os[i] = os[i]; a.dos[i] = dos[i]; a.dqs[i] = dqs[i]; a.dks[i] = dks[i]; a.dvs[i] = dvs[i];
    ok = ok && qs[i] % 4 == 0 && ks[i] % 4 == 0 && vs[i] % 4 == 0 && os[i] % 4 == 0 && dos[i] % 4 == 0 && dqs[i] % 4 == 0 &&
         dks[i] % 4 == 0 && dvs[i] % 4 == 0;
  }
  TP_REQUIRE(ok, TP_ERR_BAD_ARG, "tp_attn_bwd: fp32 pointers and strides must keep rows 16-byte aligned");
  TP_REQUIRE((int64_t)B * Hq * ((Sq + 127) / 128) < (1ll << 31) && ((int64_t)B * Hq * Sq + 255) / 256 < (1ll << 31), TP_ERR_UNSUPPORTED,
             "tp_attn_bwd: too many workgroups");
  a.scale_log2 = sm_scale * LOG2E;
  a.sm_scale = sm_scale;
  a.causal = mx.on ? 0 : causal;
  a.mx = mx;
  a.cap2 = mx.cap_in != 0.f ? mx.cap_out * sm_scale * LOG2E : 0.f;
  return Dqk == 64 ? launch_bwd_f32<64>(a, st) : launch_bwd_f32<128>(a, st);
}

}  // namespace tp
