// Attention forward in fp32 for gfx950: fp32 operands and accumulation on v_mfma_f32_32x32x2_f32.
//
// The reference's eager branch on fp32 tensors (torchprime/torch_xla_models/attention.py:151-170: fp32 matmuls, fp32
// softmax) is what its own CPU tests run the small configurations in
// (torchprime/torch_xla_models/tests/test_llama.py:143-188); the 16-bit kernels cannot meet those tolerances.  This
// kernel is the same algorithm as attn_fwd.hip without any 16-bit rounding: causal / full, segment ids, GQA, explicit
// scale, LSE out.  It is sized for correctness at small shapes, not tuned like the 16-bit kernels.
//
// v_mfma_f32_32x32x2_f32 (wave64; ln = lane % 32, g = lane / 32):
//   A (32 x 2): lane holds row ln, k = g        B (2 x 32): lane holds column ln, k = g
//   C (32 x 32): lane holds column ln, rows 8*(v/4) + 4*g + v%4 for v = 0..15
// As in the 16-bit kernel the scores are computed transposed, S^T = K Q^T, so a lane owns one query column: row
// max / sum are per-lane scalars and exp(S^T) is directly the B operand of O^T += V^T P^T.  The hardware pairs A and
// B per k index, so the order of the contraction index is free as long as both operands agree: lane group g takes
// head-dim element g*D/2 + step for S^T (contiguous per lane, 16-byte LDS reads), and kv row 8*(v/4) + 4*g + v%4 at
// step v for P V (exactly the C layout of P^T).
#include "attn_common.hpp"

namespace tp {

struct FwdArgs32 {
  const float* q;
  const float* k;
  const float* v;
  const int32_t* seg;
  float* out;
  float* lse;
  int B, Hq, Hkv, Sq, Skv, n_rep;
  int64_t qs[3], ks[3], vs[3], os[3];
  float scale_log2;
  int causal;
  MaskExt mx;   // window / query positions / causal offset as a band of key positions per query row; soft cap
  float cap2;   // the soft cap in the scores' log2 units (0: none)
};

typedef float f32x1 __attribute__((ext_vector_type(1)));

template <int D>
__global__ __launch_bounds__(256) void attn_fwd_f32_kernel(const FwdArgs32 a) {
  constexpr int BN = 32, BM = 128, DB = D / 32, HD = D / 2;
  constexpr int KSTRIDE = D + 4;  // floats per LDS row of K: 16-byte aligned rows, consecutive rows 4 banks apart
  constexpr int VSTRIDE = D + 1;
  __shared__ __align__(16) float ksm[BN * KSTRIDE];
  __shared__ float vsm[BN * VSTRIDE];
  __shared__ int ssm[BN];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, ln = lane & 31;
  const int n_qt = (a.Sq + BM - 1) / BM;
  const int qt = blockIdx.x % n_qt;
  const int bh = blockIdx.x / n_qt;
  const int h = bh % a.Hq, b = bh / a.Hq, hk = h / a.n_rep;
  const int q0 = qt * BM, wq0 = q0 + wave * 32;
  const int Sq = a.Sq, Skv = a.Skv;
  const int qrow = wq0 + ln;
  const float* qb = a.q + b * a.qs[0] + h * a.qs[1];
  const float* kb = a.k + b * a.ks[0] + hk * a.ks[1];
  const float* vb = a.v + b * a.vs[0] + hk * a.vs[1];
  const int32_t* segb = a.seg ? a.seg + (int64_t)b * Skv : nullptr;
  const int segq = segb ? segb[min(qrow, Sq - 1)] : 0;
  // mask extensions: this lane's query row may see key positions qp - lo_off .. qp + hi_off (causality is part of
  // the band then, and a.causal is off)
  const int qp = a.mx.on ? (a.mx.qpos ? a.mx.qpos[min(qrow, Sq - 1)] : qrow) : 0;
  const int band_lo = a.mx.on ? qp - a.mx.lo_off : -BAND_INF, band_hi = a.mx.on ? qp + a.mx.hi_off : BAND_INF;
  const float* bias_row =
      a.mx.bias ? a.mx.bias + b * a.mx.bias_s[0] + h * a.mx.bias_s[1] + (int64_t)min(qrow, Sq - 1) * a.mx.bias_s[2] : nullptr;

  // Q^T fragments: lane (query column ln, group g) holds Q[q][g*HD + s] for s = 0..HD-1, pre-multiplied by the
  // scale in log2 units (an fp32 product: no precision is lost that the fp32 reference keeps)
  float qf[HD];
  {
    const float* qp = qb + (int64_t)min(qrow, Sq - 1) * a.qs[2] + g * HD;
#pragma unroll
    for (int s = 0; s < HD; s += 4) {
      const f32x4 t = *(const f32x4*)(qp + s);
      qf[s] = t[0] * a.scale_log2; qf[s + 1] = t[1] * a.scale_log2; qf[s + 2] = t[2] * a.scale_log2; qf[s + 3] = t[3] * a.scale_log2;
    }
  }

  f32x16 oacc[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int v = 0; v < 16; v++) oacc[d][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const int kv_end = a.causal ? min(Skv, q0 + BM) : Skv;
  const int ntiles = (kv_end + BN - 1) / BN;
  for (int t = 0; t < ntiles; t++) {
    const int kv0 = t * BN;
    __syncthreads();  // everyone is done with the previous tile
    // stage K and V rows kv0 .. kv0+31 (rows past Skv as zeros): 16-byte chunks, thread -> (row, chunk)
    for (int c = tid; c < BN * (D / 4); c += 256) {
      const int r = c / (D / 4), cc = (c % (D / 4)) * 4;
      f32x4 kvv = {0.f, 0.f, 0.f, 0.f}, vvv = {0.f, 0.f, 0.f, 0.f};
      if (kv0 + r < Skv) {
        kvv = *(const f32x4*)(kb + (int64_t)(kv0 + r) * a.ks[2] + cc);
        vvv = *(const f32x4*)(vb + (int64_t)(kv0 + r) * a.vs[2] + cc);
      }
      *(f32x4*)(ksm + r * KSTRIDE + cc) = kvv;
      vsm[r * VSTRIDE + cc] = vvv[0]; vsm[r * VSTRIDE + cc + 1] = vvv[1]; vsm[r * VSTRIDE + cc + 2] = vvv[2]; vsm[r * VSTRIDE + cc + 3] = vvv[3];
    }
    if (segb && tid < BN) ssm[tid] = segb[min(kv0 + tid, Skv - 1)];
    __syncthreads();
    if (a.causal && kv0 > wq0 + 31) continue;  // the whole tile lies above this wave's diagonal (uniform per wave)

    // S^T = K Q^T: row = kv (ln of the A operand), column = query
    f32x16 s;
#pragma unroll
    for (int v = 0; v < 16; v++) s[v] = 0.f;
    const float* kr = ksm + ln * KSTRIDE + g * HD;
#pragma unroll
    for (int st = 0; st < HD; st += 4) {
      const f32x4 k4 = *(const f32x4*)(kr + st);
#pragma unroll
      for (int e = 0; e < 4; e++) s = __builtin_amdgcn_mfma_f32_32x32x2f32(k4[e], qf[st + e], s, 0, 0, 0);
    }
    // mask, online softmax (log2 units)
    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int kvl = 8 * (v / 4) + 4 * g + (v % 4);
      const int kv = kv0 + kvl;
      const bool ok = kv < Skv && (!a.causal || kv <= qrow) && (!segb || ssm[kvl] == segq) && kv >= band_lo && kv <= band_hi;
      if (a.cap2 != 0.f) s[v] = a.cap2 * tanhf(s[v] / a.cap2);  // cap * tanh(score / cap), in log2 units
      if (bias_row) s[v] += LOG2E * bias_row[min(kv, Skv - 1)];  // additive mask (-inf stays -inf)
      s[v] = ok ? s[v] : -INFINITY;
      mx = fmaxf(mx, s[v]);
    }
    mx = half_max(mx);
    const float m_new = fmaxf(m_run, mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = (m_run == -INFINITY) ? 0.f : exp2f(m_run - m_use);
    float rs = 0.f;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      s[v] = exp2f(s[v] - m_use);
      rs += s[v];
    }
    l_run = l_run * alpha + rs;
    m_run = m_new;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int v = 0; v < 16; v++) oacc[d][v] *= alpha;
    // O^T += V^T P^T: step v pairs kv row 8*(v/4) + 4*g + v%4 of V with the lane's value v of P^T
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int kvl = 8 * (v / 4) + 4 * g + (v % 4);
#pragma unroll
      for (int d = 0; d < DB; d++) oacc[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(vsm[kvl * VSTRIDE + d * 32 + ln], s[v], oacc[d], 0, 0, 0);
    }
  }

  // epilogue: lane = query, value v of block d is output column d*32 + 8*(v/4) + 4*g + v%4
  const float l = half_sum(l_run);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  if (qrow < Sq) {
    if (g == 0) a.lse[((int64_t)b * a.Hq + h) * Sq + qrow] = l > 0.f ? (m_run + log2f(l)) * LN2 : -INFINITY;
    float* op = a.out + b * a.os[0] + h * a.os[1] + (int64_t)qrow * a.os[2];
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int vq = 0; vq < 4; vq++) {
        const f32x16& o = oacc[d];
        *(f32x4*)(op + d * 32 + 8 * vq + 4 * g) = f32x4{o[4 * vq] * inv, o[4 * vq + 1] * inv, o[4 * vq + 2] * inv, o[4 * vq + 3] * inv};
      }
  }
}

// called by tp_attn_fwd for TP_F32 inputs (arguments already validated there)
int attn_fwd_f32(const void* q, const void* k, const void* v, const int32_t* seg, void* out, float* lse, int B, int Hq, int Hkv,
                 int Sq, int Skv, int Dqk, int Dv, const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                 float sm_scale, int causal, hipStream_t st, const MaskExt& mx) {
  TP_REQUIRE(Dqk == Dv && (Dqk == 64 || Dqk == 128), TP_ERR_UNSUPPORTED,
             "tp_attn_fwd: fp32 attention is built for head dims 64 and 128 (got qk=%d, v=%d)", Dqk, Dv);
  FwdArgs32 a;
  a.q = (const float*)q; a.k = (const float*)k; a.v = (const float*)v; a.seg = seg; a.out = (float*)out; a.lse = lse;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.Sq = Sq; a.Skv = Skv; a.n_rep = Hq / Hkv;
  bool ok = aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out);
  for (int i = 0; i < 3; i++) {
    a.qs[i] = qs[i]; a.ks[i] = ks[i]; a.vs[i] = vs[i]; a.os[i] = os[i];
    ok = ok && qs[i] % 4 == 0 && ks[i] % 4 == 0 && vs[i] % 4 == 0 && os[i] % 4 == 0;
  }
  TP_REQUIRE(ok, TP_ERR_BAD_ARG, "tp_attn_fwd: fp32 pointers and strides must keep rows 16-byte aligned");
  a.scale_log2 = sm_scale * LOG2E;
  a.causal = mx.on ? 0 : causal;
  a.mx = mx;
  a.cap2 = mx.cap_in != 0.f ? mx.cap_out * sm_scale * LOG2E : 0.f;
  const int64_t blocks = (int64_t)B * Hq * ((Sq + 127) / 128);
  TP_REQUIRE(blocks < (1ll << 31), TP_ERR_UNSUPPORTED, "tp_attn_fwd: too many workgroups");
  if (Dqk == 64) attn_fwd_f32_kernel<64><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a);
  else attn_fwd_f32_kernel<128><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a);
  return check_launch("tp_attn_fwd(fp32)");
}

}  // namespace tp
