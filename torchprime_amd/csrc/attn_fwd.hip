// Attention forward for gfx950: causal / segment-masked GQA, bf16 or fp16 in, fp32 accumulate.
//
// Replaces AttentionModule.forward's three branches (torchprime/torch_xla_models/attention.py:70-170)
// and the segment-id path of torchprime/utils/kernel_utils.py:215-220, 259-263.
//
// Structure (one workgroup = 4 waves = 128*MR query rows of one (batch, head); KV tiles of 64):
//   * the scores are computed TRANSPOSED, S^T = K Q^T, so that in the MFMA result layout a lane owns
//     one query column and 16 key rows per 32x32 block: row max / sum / rescale are per-lane scalars
//     (one half-wave exchange per tile), and exp(S^T) converted to 16 bit is already the B operand of
//     O^T += V^T P^T - P never goes through LDS;
//   * Q fragments stay in registers for the whole KV loop; K tiles are staged row-major in LDS, V tiles
//     are transposed while being written to LDS so both are read with conflict-free 16-byte loads;
//   * the next K/V tile is fetched from HBM into registers while the current one is being multiplied
//     (LDS double buffer, one barrier per tile);
//   * causal: the KV loop ends at the diagonal, element masks only on tiles that straddle it;
//     segments: per-tile [min,max] of the ids is computed once per workgroup, tiles whose id range
//     misses the query rows' range are skipped, element compares only where ranges are not one id.
#include "attn_common.hpp"

namespace tp {

struct FwdArgs {
  const void* q;
  const void* k;
  const void* v;
  const int32_t* seg;
  void* out;
  float* lse;
  int Hq, Hkv, Sq, Skv, n_rep;
  int64_t qs[3], ks[3], vs[3], os[3];
  float scale_log2;  // sm_scale * log2(e)
};

template <typename T, int DQK, int DV, int MR, bool CAUSAL, bool SEG>
__global__ __launch_bounds__(256) void attn_fwd_kernel(const FwdArgs a) {
  typedef typename MT<T>::v8 v8;
  constexpr int BN = 64;              // kv rows per tile
  constexpr int BM = 128 * MR;        // q rows per workgroup
  constexpr int NB = BN / 32;         // 32-row kv blocks per tile
  constexpr int KSTEPS = DQK / 16;    // MFMA k-steps over the qk head dim
  constexpr int DVB = DV / 32;        // 32-column blocks of the v head dim
  typedef RowTile<DQK> KT;
  constexpr int K_BYTES = BN * KT::STRIDE;
  constexpr int V_BYTES = DV * TrTile64::ROW_BYTES;
  constexpr int SEG_BYTES = SEG ? BN * 4 : 0;
  constexpr int BUF_BYTES = K_BYTES + V_BYTES + SEG_BYTES;
  constexpr int KCH = DQK / 8;                      // 16-byte chunks per K row
  constexpr int K_ITEMS = BN * KCH / 256;           // chunks per thread
  constexpr int V_TOT = (DV / 8) * (BN / 4);        // 4x8 blocks of the V tile
  constexpr int V_ITEMS = (V_TOT + 255) / 256;
  static_assert(BN * KCH % 256 == 0, "K tile must split evenly over 256 threads");

  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, ln = lane & 31;
  const int qt = gridDim.x - 1 - blockIdx.x;  // longest (latest) query tiles are scheduled first
  const int h = blockIdx.y, b = blockIdx.z, hk = h / a.n_rep;
  const int q0 = qt * BM;
  const int wq0 = q0 + wave * 32 * MR;
  const int Sq = a.Sq, Skv = a.Skv;

  const T* qb = (const T*)a.q + b * a.qs[0] + h * a.qs[1];
  const T* kb = (const T*)a.k + b * a.ks[0] + hk * a.ks[1];
  const T* vb = (const T*)a.v + b * a.vs[0] + hk * a.vs[1];
  const int32_t* segb = SEG ? a.seg + (int64_t)b * Skv : nullptr;

  const int kv_end = CAUSAL ? min(Skv, q0 + BM) : Skv;
  const int ntiles = (kv_end + BN - 1) / BN;

  // ---- Q fragments (B operand of S^T = K Q^T): lane = query column, 8 head-dim values per k-step
  v8 qf[MR][KSTEPS];
  int segq[MR];
#pragma unroll
  for (int mr = 0; mr < MR; mr++) {
    const int row = min(wq0 + mr * 32 + ln, Sq - 1);
    const T* qp = qb + row * a.qs[2] + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) qf[mr][ks] = *(const v8*)(qp + 16 * ks);
    segq[mr] = SEG ? segb[row] : 0;
  }

  // ---- segment bookkeeping: per-tile id ranges, list of tiles that can contain an allowed pair
  int* kvmin = (int*)(smem + 2 * BUF_BYTES);
  int* kvmax = kvmin + ntiles;
  int* active = kvmax + ntiles;
  int* bq = active + ntiles;  // 8 ints: per-wave (min,max) of the query rows' ids
  int nact = ntiles;
  int wqmin = 0, wqmax = 0;
  if (SEG) {
    wqmin = segq[0]; wqmax = segq[0];
#pragma unroll
    for (int mr = 1; mr < MR; mr++) { wqmin = min(wqmin, segq[mr]); wqmax = max(wqmax, segq[mr]); }
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) {
      wqmin = min(wqmin, __shfl_xor(wqmin, o, 64));
      wqmax = max(wqmax, __shfl_xor(wqmax, o, 64));
    }
    if (lane == 0) { bq[2 * wave] = wqmin; bq[2 * wave + 1] = wqmax; }
    for (int t = wave; t < ntiles; t += 4) {
      const int idx = min(t * BN + lane, Skv - 1);
      int lo = segb[idx], hi = lo;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        lo = min(lo, __shfl_xor(lo, o, 64));
        hi = max(hi, __shfl_xor(hi, o, 64));
      }
      if (lane == 0) { kvmin[t] = lo; kvmax[t] = hi; }
    }
    __syncthreads();
    const int bqmin = min(min(bq[0], bq[2]), min(bq[4], bq[6]));
    const int bqmax = max(max(bq[1], bq[3]), max(bq[5], bq[7]));
    // every wave builds the same list redundantly (no second barrier needed for the count)
    int cnt = 0;
    for (int base = 0; base < ntiles; base += 64) {
      const int t = base + lane;
      const bool act = t < ntiles && !(kvmax[t] < bqmin || kvmin[t] > bqmax);
      const unsigned long long m = __ballot(act);
      if (act && wave == 0) active[cnt + __popcll(m & ((1ull << lane) - 1ull))] = t;
      cnt += __popcll(m);
    }
    nact = cnt;
    __syncthreads();
  }

  // ---- global -> register staging of one K/V tile (buffer loads, rows past Skv read as zero)
  const rsrc_t krs = make_rsrc(kb, span_bytes(Skv, a.ks[2], DQK));
  const rsrc_t vrs = make_rsrc(vb, span_bytes(Skv, a.vs[2], DV));
  const unsigned k_tile_bytes = (unsigned)(BN * a.ks[2] * 2), v_tile_bytes = (unsigned)(BN * a.vs[2] * 2);
  unsigned kvo[K_ITEMS], vvo[V_ITEMS][4];
#pragma unroll
  for (int i = 0; i < K_ITEMS; i++) {
    const int item = tid + 256 * i;
    kvo[i] = (unsigned)(((item / KCH) * a.ks[2] + (item % KCH) * 8) * 2);
  }
#pragma unroll
  for (int i = 0; i < V_ITEMS; i++) {
    const int item = tid + 256 * i;
    const int c8 = item % (DV / 8), rq = item / (DV / 8);
#pragma unroll
    for (int ii = 0; ii < 4; ii++) vvo[i][ii] = (unsigned)(((4 * rq + ii) * a.vs[2] + c8 * 8) * 2);
  }
  u32x4 kreg[K_ITEMS];
  u32x4 vreg[V_ITEMS][4];
  int sreg = 0;
  auto load_tile = [&](int t) {
    const unsigned kso = (unsigned)t * k_tile_bytes, vso = (unsigned)t * v_tile_bytes;
#pragma unroll
    for (int i = 0; i < K_ITEMS; i++) kreg[i] = buf_load16(krs, kvo[i], kso);
#pragma unroll
    for (int i = 0; i < V_ITEMS; i++) {
      if (tid + 256 * i < V_TOT) {
#pragma unroll
        for (int ii = 0; ii < 4; ii++) vreg[i][ii] = buf_load16(vrs, vvo[i][ii], vso);
      }
    }
    if (SEG && tid < BN) sreg = segb[min(t * BN + tid, Skv - 1)];
  };
  auto store_tile = [&](int buf) {
    unsigned char* kl = smem + buf * BUF_BYTES;
    unsigned char* vl = kl + K_BYTES;
#pragma unroll
    for (int i = 0; i < K_ITEMS; i++) {
      const int item = tid + 256 * i;
      *(u32x4*)(kl + KT::off(item / KCH, (item % KCH) * 8)) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < V_ITEMS; i++) {
      const int item = tid + 256 * i;
      if (item < V_TOT) {
        const int c8 = item % (DV / 8), rq = item / (DV / 8);
#pragma unroll
        for (int j = 0; j < 8; j++) *(u32x2*)(vl + TrTile64::quad_off(c8 * 8 + j, rq)) = transpose_col(vreg[i], j);
      }
    }
    if (SEG && tid < BN) ((int*)(vl + V_BYTES))[tid] = sreg;
  };

  // ---- accumulators: O^T blocks [DVB][MR], running max (log2 units) and per-lane partial row sums
  f32x16 oacc[DVB][MR];
  float m_run[MR], l_run[MR];
#pragma unroll
  for (int mr = 0; mr < MR; mr++) {
    m_run[mr] = -INFINITY;
    l_run[mr] = 0.f;
#pragma unroll
    for (int d = 0; d < DVB; d++)
#pragma unroll
      for (int v = 0; v < 16; v++) oacc[d][mr][v] = 0.f;
  }
  const float c = a.scale_log2;
  const int wq_last = wq0 + 32 * MR - 1;

  if (nact > 0) {
    load_tile(SEG ? active[0] : 0);
    store_tile(0);
  }
  // Everything loaded so far (the Q fragments above all) has landed before the loop starts.  Without
  // this the compiler must assume those loads may still be in flight at the loop head and, the vector
  // memory counter being in-order, makes the first MFMA of EVERY iteration wait for that iteration's
  // own prefetch loads.
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();

  for (int it = 0; it < nact; it++) {
    const int t = SEG ? active[it] : it;
    const int kv0 = t * BN;
    const int buf = it & 1;
    if (it + 1 < nact) load_tile(SEG ? active[it + 1] : it + 1);

    const unsigned char* kl = smem + buf * BUF_BYTES;
    const unsigned char* vl = kl + K_BYTES;
    const int* sl = (const int*)(vl + V_BYTES);

    bool skip = CAUSAL && kv0 > wq_last;
    bool need_mask = (kv0 + BN > Skv) || (CAUSAL && kv0 + BN - 1 > wq0);
    if (SEG) {
      const int lo = kvmin[t], hi = kvmax[t];
      skip = skip || hi < wqmin || lo > wqmax;
      need_mask = need_mask || !(lo == hi && wqmin == wqmax && lo == wqmin);
    }
    if (!skip) {
      // ---- S^T = K Q^T
      f32x16 sacc[NB][MR];
#pragma unroll
      for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int mr = 0; mr < MR; mr++)
#pragma unroll
          for (int v = 0; v < 16; v++) sacc[nb][mr][v] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
          const v8 kf = *(const v8*)(kl + KT::off(nb * 32 + ln, 16 * ks + 8 * g));
#pragma unroll
          for (int mr = 0; mr < MR; mr++) sacc[nb][mr] = MT<T>::mfma32(kf, qf[mr][ks], sacc[nb][mr]);
        }
      }
      // ---- mask (only tiles that straddle the diagonal, the tail, or a segment boundary)
      if (need_mask) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
#pragma unroll
          for (int v = 0; v < 16; v++) {
            const int kvl = nb * 32 + 8 * (v / 4) + 4 * g + (v % 4);
            const int kv = kv0 + kvl;
            const int sk = SEG ? sl[kvl] : 0;
#pragma unroll
            for (int mr = 0; mr < MR; mr++) {
              const int qrow = wq0 + mr * 32 + ln;
              const bool ok = kv < Skv && (!CAUSAL || kv <= qrow) && (!SEG || sk == segq[mr]);
              sacc[nb][mr][v] = ok ? sacc[nb][mr][v] : -INFINITY;
            }
          }
        }
      }
      // ---- online softmax, per lane = per query column
      v8 pf[MR][BN / 16];
#pragma unroll
      for (int mr = 0; mr < MR; mr++) {
        float mx = -INFINITY;
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
          for (int v = 0; v < 16; v++) mx = fmaxf(mx, sacc[nb][mr][v]);
        mx = half_max(mx);
        // Lazy rescale: the running max only moves when the tile max exceeds it by more than 2^8, so
        // p stays <= 256 (harmless in fp32 sums and in the 16-bit P operand) and on most tiles no lane of
        // the wave needs its accumulators rescaled.  O and l always share the same reference max.
        const float mxs = mx * c;
        const bool grow = mxs > m_run[mr] + 8.0f;
        const float m_new = grow ? mxs : m_run[mr];
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = grow ? fast_exp2(m_run[mr] - m_use) : 1.0f;
        m_run[mr] = m_new;
        float rs = 0.f;
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
          for (int v = 0; v < 16; v++) {
            const float p = fast_exp2(__builtin_fmaf(sacc[nb][mr][v], c, -m_use));
            sacc[nb][mr][v] = p;
            rs += p;
          }
        l_run[mr] = l_run[mr] * alpha + rs;
        if (__builtin_amdgcn_ballot_w64(grow) != 0) {
#pragma unroll
          for (int d = 0; d < DVB; d++)
#pragma unroll
            for (int v = 0; v < 16; v++) oacc[d][mr][v] *= alpha;
        }
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
          for (int hh = 0; hh < 2; hh++) {
            const f32x16& s = sacc[nb][mr];
            pf[mr][nb * 2 + hh] = pack8<T>(s[8 * hh + 0], s[8 * hh + 1], s[8 * hh + 2], s[8 * hh + 3], s[8 * hh + 4],
                                           s[8 * hh + 5], s[8 * hh + 6], s[8 * hh + 7]);
          }
      }
      // ---- O^T += V^T P^T
#pragma unroll
      for (int ks = 0; ks < BN / 16; ks++) {
#pragma unroll
        for (int d = 0; d < DVB; d++) {
          const v8 vf = *(const v8*)(vl + TrTile64::chunk_off(d * 32 + ln, ks, g));
#pragma unroll
          for (int mr = 0; mr < MR; mr++) oacc[d][mr] = MT<T>::mfma32(vf, pf[mr][ks], oacc[d][mr]);
        }
      }
    }
    if (it + 1 < nact) store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: normalise, write O (row = query, 4 consecutive v-dims per store) and LSE
  T* ob = (T*)a.out + b * a.os[0] + h * a.os[1];
  float* lb = a.lse + ((int64_t)b * a.Hq + h) * Sq;
#pragma unroll
  for (int mr = 0; mr < MR; mr++) {
    const int row = wq0 + mr * 32 + ln;
    const float l = half_sum(l_run[mr]);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    if (row < Sq) {
      if (g == 0) lb[row] = l > 0.f ? (m_run[mr] + log2f(l)) * LN2 : -INFINITY;
      T* op = ob + row * a.os[2];
#pragma unroll
      for (int d = 0; d < DVB; d++)
#pragma unroll
        for (int vq = 0; vq < 4; vq++) {
          const f32x16& o = oacc[d][mr];
          *(u32x2*)(op + d * 32 + 8 * vq + 4 * g) =
              pack4<T>(o[4 * vq] * inv, o[4 * vq + 1] * inv, o[4 * vq + 2] * inv, o[4 * vq + 3] * inv);
        }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------------------
template <typename T, int DQK, int DV, int MR, bool CAUSAL, bool SEG>
static int launch_fwd(const FwdArgs& a, int B, hipStream_t st) {
  constexpr int BN = 64, BM = 128 * MR;
  constexpr int BUF = BN * RowTile<DQK>::STRIDE + DV * TrTile64::ROW_BYTES + (SEG ? BN * 4 : 0);
  const int ntiles_max = (a.Skv + BN - 1) / BN;
  const size_t smem = 2 * (size_t)BUF + (SEG ? (size_t)(3 * ntiles_max + 8) * 4 : 0);
  TP_REQUIRE(smem <= 160 * 1024, TP_ERR_UNSUPPORTED, "tp_attn_fwd: Skv=%d needs %zu bytes of LDS (max 163840)", a.Skv, smem);
  auto kern = attn_fwd_kernel<T, DQK, DV, MR, CAUSAL, SEG>;
  static bool attr_set = false;  // benign race: every thread sets the same value
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    TP_REQUIRE(e == hipSuccess, TP_ERR_LAUNCH, "tp_attn_fwd: hipFuncSetAttribute failed: %s", hipGetErrorString(e));
    attr_set = true;
  }
  const dim3 grid((a.Sq + BM - 1) / BM, a.Hq, B), block(256);
  kern<<<grid, block, smem, st>>>(a);
  return check_launch("tp_attn_fwd");
}

template <typename T, int DQK, int DV>
static int dispatch_fwd(const FwdArgs& a, int B, int causal, hipStream_t st) {
  constexpr int MR = 1;
  if (causal) {
    if (a.seg) return launch_fwd<T, DQK, DV, MR, true, true>(a, B, st);
    return launch_fwd<T, DQK, DV, MR, true, false>(a, B, st);
  }
  if (a.seg) return launch_fwd<T, DQK, DV, MR, false, true>(a, B, st);
  return launch_fwd<T, DQK, DV, MR, false, false>(a, B, st);
}

}  // namespace tp

using namespace tp;

extern "C" int tp_attn_fwd(const void* q, const void* k, const void* v, const int32_t* seg, void* out, float* lse,
                           int B, int Hq, int Hkv, int Sq, int Skv, int Dqk, int Dv, const int64_t q_strides[3],
                           const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3],
                           float sm_scale, int causal, int dtype, void* stream) {
  TP_REQUIRE(q && k && v && out && lse && q_strides && k_strides && v_strides && o_strides, TP_ERR_BAD_ARG,
             "tp_attn_fwd: null pointer");
  TP_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Sq > 0 && Skv > 0, TP_ERR_BAD_ARG, "tp_attn_fwd: non-positive size");
  TP_REQUIRE(Hq % Hkv == 0, TP_ERR_BAD_ARG, "tp_attn_fwd: Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  TP_REQUIRE(!seg || Sq == Skv, TP_ERR_BAD_ARG, "tp_attn_fwd: segment ids need Sq == Skv (got %d, %d)", Sq, Skv);
  TP_REQUIRE(sm_scale > 0.f, TP_ERR_BAD_ARG, "tp_attn_fwd: sm_scale must be positive");
  TP_REQUIRE(dtype == TP_BF16 || dtype == TP_F16, TP_ERR_UNSUPPORTED, "tp_attn_fwd: dtype %d (bf16 and fp16 only)", dtype);
  TP_REQUIRE(B <= 65535 && Hq <= 65535, TP_ERR_UNSUPPORTED, "tp_attn_fwd: batch and heads are limited to 65535");
  FwdArgs a;
  a.q = q; a.k = k; a.v = v; a.seg = seg; a.out = out; a.lse = lse;
  a.Hq = Hq; a.Hkv = Hkv; a.Sq = Sq; a.Skv = Skv; a.n_rep = Hq / Hkv;
  bool ok = aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out);
  for (int i = 0; i < 3; i++) {
    a.qs[i] = q_strides[i]; a.ks[i] = k_strides[i]; a.vs[i] = v_strides[i]; a.os[i] = o_strides[i];
    ok = ok && q_strides[i] % 8 == 0 && k_strides[i] % 8 == 0 && v_strides[i] % 8 == 0 && o_strides[i] % 4 == 0;
  }
  TP_REQUIRE(ok, TP_ERR_BAD_ARG, "tp_attn_fwd: pointers and strides must keep rows 16-byte aligned");
  // tiles are addressed with 32-bit byte offsets inside one (batch, head) slice
  TP_REQUIRE(((int64_t)Skv * k_strides[2] + Dqk) * 2 < (1ll << 31) && ((int64_t)Skv * v_strides[2] + Dv) * 2 < (1ll << 31) &&
                 k_strides[2] > 0 && v_strides[2] > 0,
             TP_ERR_UNSUPPORTED, "tp_attn_fwd: one (batch, head) slice of k or v spans 2 GiB or more");
  a.scale_log2 = sm_scale * LOG2E;
  hipStream_t st = (hipStream_t)stream;
#define TP_FWD(T, DQ, DVV) return dispatch_fwd<T, DQ, DVV>(a, B, causal, st)
  if (dtype == TP_BF16) {
    if (Dqk == 128 && Dv == 128) TP_FWD(bf16_t, 128, 128);
    if (Dqk == 64 && Dv == 64) TP_FWD(bf16_t, 64, 64);
    if (Dqk == 192 && Dv == 128) TP_FWD(bf16_t, 192, 128);
  } else {
    if (Dqk == 128 && Dv == 128) TP_FWD(f16_t, 128, 128);
    if (Dqk == 64 && Dv == 64) TP_FWD(f16_t, 64, 64);
    if (Dqk == 192 && Dv == 128) TP_FWD(f16_t, 192, 128);
  }
#undef TP_FWD
  TP_REQUIRE(false, TP_ERR_UNSUPPORTED, "tp_attn_fwd: head dims (qk=%d, v=%d) not built", Dqk, Dv);
}
