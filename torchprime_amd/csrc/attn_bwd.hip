// Attention backward for gfx950: recompute P from LSE, no atomics, bitwise reproducible.
//
// The reference obtains these gradients from autograd through the eager expression
// (torchprime/torch_xla_models/attention.py:151-170) or from the Pallas backward kernels behind
// attention.py:121-123 / 144-150.  With P = exp(sm_scale*QK^T - LSE), delta = rowsum(dO o O):
//     dV = P^T dO;  dS = P o (dO V^T - delta);  dQ = sm_scale dS K;  dK = sm_scale dS^T Q
// and dK, dV summed over the n_rep query heads that share a KV head.
//
// Kernels:
//   attn_delta_kernel     -delta[b,h,i] = -sum_d dO*O, and the LSE in log2 units      (HBM-bound; only where the
//                         general dQ kernel runs: the lean dQ kernel computes both itself and runs first)
//   attn_bwd_dkdv_kernel  one workgroup = 128 KV rows of one (batch, kv head); K and V fragments stay
//                         in registers, row-major Q / dO tiles of every query head of the group stream through
//                         three LDS buffers (fragment reads for S = QK^T and dP = dO V^T, transposing reads
//                         for dV^T += dO^T P and dK^T += Q^T dS).  S is computed un-transposed here so
//                         that a lane owns one KV column: P and dS converted to 16 bit are directly the
//                         B operands of the two accumulating products.
//   attn_bwd_dq_plain_kernel  dQ without mask extensions (plain, causal, causal with segment ids): one workgroup =
//                         128 query rows of one (batch, head); Q and dO fragments in registers, row-major K and V
//                         tiles stream through two LDS buffers; S^T, dP^T are computed transposed (a lane owns one
//                         query column, so LSE and delta are per-lane scalars) and dS^T feeds dQ^T += K^T dS^T,
//                         whose K^T operand comes out of transposing reads.
//   attn_bwd_dq_kernel    the general dQ kernel (mask extensions, segment ids without causality): 4 or 8 waves,
//                         K (row-major + transposed copy) and V tiles staged through registers.
// Splitting dQ from dK/dV recomputes S and dP once more but needs no atomics: fp32 atomic adds reach
// about 1.3 TB/s on this part, an order of magnitude short of what accumulating dQ tiles would need.
#include <type_traits>

#include "attn_common.hpp"

namespace tp {

// position j of a sequence that alternates the steps of two accumulation chains of lengths n0 and n1
struct AbSlot {
  int kind, k;
};
__host__ __device__ constexpr AbSlot ab_slot(int j, int n0, int n1) {
  int n = 0;
  for (int k = 0; k < (n0 > n1 ? n0 : n1); k++) {
    if (k < n0) {
      if (n == j) return AbSlot{0, k};
      n++;
    }
    if (k < n1) {
      if (n == j) return AbSlot{1, k};
      n++;
    }
  }
  return AbSlot{0, 0};
}

struct BwdArgs {
  const void* q;
  const void* k;
  const void* v;
  const void* out;
  const void* dout;
  const float* lse;
  const int32_t* seg;
  void* dq;
  void* dk;
  void* dv;
  float* delta;
  int B, Hq, Hkv, Sq, Skv, n_rep;
  int64_t qs[3], ks[3], vs[3], os[3], dos[3], dqs[3], dks[3], dvs[3];
  float scale_log2;  // sm_scale * log2(e)
  float sm_scale;
  // the causal kernels' band: query row i sees keys i - band_lo .. i + band_hi (plain causality: no lower bound, 0).
  // Sliding windows and causal offsets without the other mask extensions run through these kernels.
  int band_lo, band_hi;
  MaskExt mx;
};

// ------------------------------------------------------------------------------------------------
// delta = rowsum(dO o O)
// ------------------------------------------------------------------------------------------------
template <typename T, int DV>
__global__ __launch_bounds__(256) void attn_delta_kernel(const BwdArgs a) {
  constexpr int TPR = DV / 8;  // threads per row, one 16-byte chunk each
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t total = (int64_t)a.B * a.Hq * a.Sq;
  int64_t rowid = idx / TPR;
  const int ch = (int)(idx % TPR);
  const bool valid = rowid < total;
  if (!valid) rowid = total - 1;
  const int s = (int)(rowid % a.Sq);
  const int64_t bh = rowid / a.Sq;
  const int h = (int)(bh % a.Hq), b = (int)(bh / a.Hq);
  float o[8], g[8];
  // (streamed once here: non-temporal loads, as in the other HBM-bound kernels)
  load_f_nt<T, 8>((const T*)a.out + b * a.os[0] + h * a.os[1] + s * a.os[2] + ch * 8, o);
  load_f_nt<T, 8>((const T*)a.dout + b * a.dos[0] + h * a.dos[1] + s * a.dos[2] + ch * 8, g);
  float acc = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e++) acc += o[e] * g[e];
#pragma unroll
  for (int off = TPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (valid && ch == 0) {
    a.delta[rowid] = -acc;  // stored negated: the dK/dV kernel starts its dP accumulators from it
    // second half of the workspace: minus the LSE in log2 units, which the dK/dV kernel starts its S
    // accumulators from; a row with no allowed key (LSE = -inf) gets -inf so that its P = exp2(-inf) = 0
    const float l = a.lse[rowid];
    a.delta[total + rowid] = (l == -INFINITY) ? -INFINITY : -l * LOG2E;
  }
}

// ------------------------------------------------------------------------------------------------
// staging helpers: a tile of 64 rows x D 16-bit elements, each thread owning 4-row x 8-column blocks
// so that one set of global loads serves both the row-major and the transposed LDS copy
// ------------------------------------------------------------------------------------------------
template <int D>
struct Stage64 {
  static constexpr int TOT = (D / 8) * 16;       // 4x8 blocks in the tile
  static constexpr int ITEMS = (TOT + 255) / 256;
  u32x4 r[ITEMS][4];
  unsigned vo[ITEMS][4];  // byte offsets of this thread's 16-byte pieces inside a tile

  // block (column chunk c8, row quad rq) of work item `item`.  Row quads are dealt so that the 32 lanes
  // whose transposed 8-byte stores are served together fall into 32 different bank pairs.
  static __device__ __forceinline__ int c8_of(int item) { return item % (D / 8); }
  static __device__ __forceinline__ int rq_of(int item) {
    const int rqi = item / (D / 8);
    return (rqi & ~3) | ((rqi & 1) << 1) | ((rqi >> 1) & 1);
  }
  __device__ __forceinline__ void init(int64_t row_stride, int tid) {
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
      const int item = tid + 256 * i;
      const int c8 = c8_of(item), rq = rq_of(item);
#pragma unroll
      for (int ii = 0; ii < 4; ii++) vo[i][ii] = (unsigned)(((4 * rq + ii) * row_stride + c8 * 8) * 2);
    }
  }
  // rows past the end of the tensor (offset >= the resource's size) read as zero
  __device__ __forceinline__ void load(rsrc_t rs, unsigned tile_byte_offset, int tid) {
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
      if (tid + 256 * i < TOT) {
#pragma unroll
        for (int ii = 0; ii < 4; ii++) r[i][ii] = buf_load16(rs, vo[i][ii], tile_byte_offset);
      }
    }
  }
  __device__ __forceinline__ void store_rowmajor(unsigned char* dst, int tid) const {
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
      const int item = tid + 256 * i;
      if (item < TOT) {
        const int c8 = c8_of(item), rq = rq_of(item);
#pragma unroll
        for (int ii = 0; ii < 4; ii++) *(u32x4*)(dst + RowTile<D>::off(4 * rq + ii, c8 * 8)) = r[i][ii];
      }
    }
  }
  // column pair member J (0..7) of the transposed copy, for tiles with one block per thread
  template <int J>
  __device__ __forceinline__ void store_transposed_step(unsigned char* dst, int tid) const {
    static_assert(ITEMS == 1, "one block per thread");
    if (tid < TOT) {
      const int c8 = c8_of(tid), rq = rq_of(tid), flip = c8 & 1;
      const unsigned sel = ((J & 1) ^ flip) ? 0x07060302u : 0x05040100u;
      constexpr int w = J >> 1;
      u32x2 o;
      o.x = __builtin_amdgcn_perm(r[0][1][w], r[0][0][w], sel);
      o.y = __builtin_amdgcn_perm(r[0][3][w], r[0][2][w], sel);
      *(u32x2*)(dst + TrTile64::quad_off(c8 * 8 + (J ^ flip), rq)) = o;
    }
  }
  __device__ __forceinline__ void store_transposed(unsigned char* dst, int tid) const {
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
      const int item = tid + 256 * i;
      if (item < TOT) {
        const int c8 = c8_of(item), rq = rq_of(item);
        // odd column chunks take their columns in the order 1,0,3,2,...: at every step half the lanes
        // write even LDS rows and half odd ones
        const int flip = c8 & 1;
        const unsigned sel_even = flip ? 0x07060302u : 0x05040100u, sel_odd = flip ? 0x05040100u : 0x07060302u;
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const unsigned sel = (j & 1) ? sel_odd : sel_even;
          const int w = j >> 1;
          u32x2 o;
          o.x = __builtin_amdgcn_perm(r[i][1][w], r[i][0][w], sel);
          o.y = __builtin_amdgcn_perm(r[i][3][w], r[i][2][w], sel);
          *(u32x2*)(dst + TrTile64::quad_off(c8 * 8 + (j ^ flip), rq)) = o;
        }
      }
    }
  }
};

// 4 bytes per lane straight into LDS at dst + 4 * lane (a 64-entry row vector per instruction)
__device__ __forceinline__ void dma_dword(u32x4 rs, unsigned byte_offset, unsigned char* dst, int lane) {
  const unsigned d = __builtin_amdgcn_readfirstlane((unsigned)(size_t)dst);
  byte_offset = __builtin_amdgcn_readfirstlane(byte_offset);
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, %3 offen lds"
               :: "s"(d), "v"((unsigned)lane * 4u), "s"(rs), "s"(byte_offset) : "memory", "m0");
}
__device__ __forceinline__ void dma_dword_at(u32x4 rs, unsigned byte_offset, unsigned dst, int lane) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, %3 offen lds"
               :: "s"(dst), "v"((unsigned)lane * 4u), "s"(rs), "s"(byte_offset) : "memory", "m0");
}
// ------------------------------------------------------------------------------------------------
// dK / dV
// ------------------------------------------------------------------------------------------------
template <typename T, int DQK, int DV, int NBUF, bool CAUSAL, bool SEG>
__global__ __launch_bounds__(256) void attn_bwd_dkdv_kernel(const BwdArgs a) {
  typedef typename MT<T>::v8 v8;
  constexpr int BMQ = 64;   // query rows per streamed tile
  constexpr int BNK = 128;  // kv rows per workgroup, 32 per wave
  constexpr int KS_QK = DQK / 16, KS_DV = DV / 16;
  constexpr int DKB = DQK / 32, DVB = DV / 32;
  // Three row-major buffers of Q and dO tiles, no transposed copies: the operands of the two accumulating products
  // are read from the row-major tiles with transposing LDS reads.
  static_assert(NBUF == 3, "the tile loop rotates three buffers");
  typedef DmaTile<DQK, true> QT;
  typedef DmaTile<DV, true> OT;
  constexpr int Q_BYTES = QT::BYTES, DO_BYTES = OT::BYTES;
  constexpr int ROW_BYTES = BMQ * 4 * 4;  // lse (log2 units), delta, segment id, position per query row
  constexpr int BUF_BYTES = Q_BYTES + DO_BYTES;
  // LDS layout: the NBUF copies of each kind of tile lie side by side (Q.. dO.., then the row vectors), so that with
  // the buffer index a constant every fragment address is a loop-invariant per-lane offset plus an immediate
  constexpr int Q_AT = 0, DO_AT = NBUF * Q_BYTES;

  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, ln = lane & 31;
  int tile, inner, group;
  if (!xcd_map((a.Skv + BNK - 1) / BNK, 1, a.B * a.Hkv, tile, inner, group)) return;
  const int b = group / a.Hkv, hk = group - b * a.Hkv;
  const int kv0 = tile * BNK;  // low kv tiles see the most queries: they start first
  const int wkv0 = kv0 + wave * 32;
  const int Sq = a.Sq, Skv = a.Skv;
  // GEN: the instantiation that also evaluates the mask extensions (and then may run without segment ids)
  constexpr bool GEN = !CAUSAL && SEG;
  const bool has_seg = SEG && (!GEN || a.seg != nullptr);
  const bool ext = GEN && a.mx.on;
  const bool capped = GEN && a.mx.cap_in != 0.f;
  const bool biased = GEN && a.mx.bias != nullptr;
  const bool has_pos = ext && a.mx.qpos != nullptr;
  const int32_t* segb = has_seg ? a.seg + (int64_t)b * Skv : nullptr;

  // ---- K, V fragments of this wave's 32 kv rows (B operands: lane = kv column)
  v8 kf[KS_QK], vf[KS_DV];
  const int kvrow = min(wkv0 + ln, Skv - 1);
  {
    const T* kp = (const T*)a.k + b * a.ks[0] + hk * a.ks[1] + kvrow * a.ks[2] + 8 * g;
    const T* vp = (const T*)a.v + b * a.vs[0] + hk * a.vs[1] + kvrow * a.vs[2] + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS_QK; ks++) kf[ks] = *(const v8*)(kp + 16 * ks);
#pragma unroll
    for (int ks = 0; ks < KS_DV; ks++) vf[ks] = *(const v8*)(vp + 16 * ks);
  }
  const int segk = has_seg ? segb[kvrow] : 0;

  // ---- query tiles to visit: causal => tiles that reach the first kv row; segments => id ranges overlap
  // (band: row i sees keys i - band_lo .. i + band_hi, so key j is seen by rows j - band_hi .. j + band_lo)
  const int band_lo = CAUSAL ? a.band_lo : BAND_INF, band_hi = CAUSAL ? a.band_hi : BAND_INF;
  const int nqt_tot = (Sq + BMQ - 1) / BMQ;
  const int nqt_all = CAUSAL ? min((kv0 + BNK - 1 + band_lo) / BMQ + 1, nqt_tot) : nqt_tot;  // one past the last tile in reach
  const int qt_first = CAUSAL ? min(max(kv0 - band_hi, 0) / BMQ, nqt_all) : 0;
  const int nqt = nqt_all - qt_first;
  // id ranges of all query tiles and the list of those to visit: only needed until the control entries below are
  // built, so they borrow the tile buffers, which nothing has been loaded into yet
  int* qmin = (int*)smem;
  int* qmax = qmin + nqt;
  int* active = qmax + nqt;
  int* bk = (int*)(smem + NBUF * BUF_BYTES + 3 * ROW_BYTES);  // 8 ints: per-wave (min,max) of kv ids
  int* pmin = bk + 8;      // per query tile: (min,max) of the rows' positions in the key order (mask extensions)
  int* pmax = pmin + nqt;
  // per visited tile, in visiting order: (query tile, min id, max id, index into the position ranges), 16 bytes that
  // one LDS read fetches a whole tile ahead of their use (the tile loop would otherwise start every tile by waiting
  // out a chain of dependent LDS reads: list entry -> its ranges -> which body to run)
  // (its address is formed as an offset from the LDS array: rounded through an integer the pointer loses its address
  // space, every read of an entry becomes a flat load, and waiting for a flat load waits, the vector-memory counter
  // being in-order, for the tile loads issued before it)
  const unsigned ctl_off = ((unsigned)((const unsigned char*)(pmax + nqt) - smem) + 15u) & ~15u;
  int* ctl = (int*)(smem + ctl_off);
  int nact = nqt;
  int wkmin = 0, wkmax = 0;
  if (SEG) {
    wkmin = segk; wkmax = segk;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) {
      wkmin = min(wkmin, __shfl_xor(wkmin, o, 64));
      wkmax = max(wkmax, __shfl_xor(wkmax, o, 64));
    }
    wkmin = __builtin_amdgcn_readfirstlane(wkmin);
    wkmax = __builtin_amdgcn_readfirstlane(wkmax);
    if (lane == 0) { bk[2 * wave] = wkmin; bk[2 * wave + 1] = wkmax; }
    if (has_seg) {
      seg_tile_ranges(segb, Sq, qt_first, nqt_all, qmin, qmax, tid, 256);
    } else {
      for (int t = tid; t < nqt; t += 256) { qmin[t] = 0; qmax[t] = 0; }
    }
    if (ext) {
      if (has_pos) {
        seg_tile_ranges(a.mx.qpos, Sq, qt_first, nqt_all, pmin, pmax, tid, 256);
      } else {
        for (int t = tid; t < nqt; t += 256) { pmin[t] = (qt_first + t) * BMQ; pmax[t] = min((qt_first + t) * BMQ + BMQ - 1, Sq - 1); }
      }
    }
    __syncthreads();
    const int bkmin = min(min(bk[0], bk[2]), min(bk[4], bk[6]));
    const int bkmax = max(max(bk[1], bk[3]), max(bk[5], bk[7]));
    int cnt = 0;
    for (int base = 0; base < nqt; base += 64) {
      const int t = base + lane;
      bool act = t < nqt && !(qmax[t] < bkmin || qmin[t] > bkmax);
      // (band: some row of the tile must reach into this workgroup's 128 kv rows)
      if (ext && act) act = kv0 <= pmax[t] + a.mx.hi_off && kv0 + BNK - 1 >= pmin[t] - a.mx.lo_off;
      const unsigned long long m = __ballot(act);
      if (act && wave == 0) active[cnt + __popcll(m & ((1ull << lane) - 1ull))] = t;
      cnt += __popcll(m);
    }
    nact = cnt;
    __syncthreads();
    for (int i = tid; i < nact; i += 256) {
      const int t = active[nact - 1 - i];  // visiting order: last query tile first (see qtile_of)
      *(i32x4*)(ctl + 4 * i) = i32x4{qt_first + t, qmin[t], qmax[t], t};
    }
    __syncthreads();
  }
  const int n_iter = nact * a.n_rep;

  // ---- staging: every piece of a query tile (Q, dO row-major; log2-scaled LSE, delta, segment ids of its
  // rows) is written into LDS by the loads themselves; the transposed copies are made LDS-to-LDS
  QT qdma;
  OT dodma;
  qdma.init(a.qs[2], wave, lane);
  dodma.init(a.dos[2], wave, lane);
  const unsigned q_span = span_bytes(Sq, a.qs[2], DQK), do_span = span_bytes(Sq, a.dos[2], DV);
  const unsigned q_tile_bytes = (unsigned)(BMQ * a.qs[2] * 2), do_tile_bytes = (unsigned)(BMQ * a.dos[2] * 2);
  const float* lse2 = a.delta + (int64_t)a.B * a.Hq * Sq;  // second half of the workspace (written by the kernel before this one)
  unsigned char* const rows_base = smem + NBUF * BUF_BYTES;
  // Query tiles are visited from the last one down.  The workgroups of a (batch, kv head) run side by side on one XCD
  // and all stream the same Q / dO tiles; each needs the tiles from its own kv rows on, so counting up they would start
  // at different tiles and never meet in the L2 (every tile fetched from memory once per workgroup); counting down
  // they start together at the last tile and stay within an L2's reach of each other.
  auto qtile_of = [&](int idx) { return SEG ? ctl[4 * idx] : nqt_all - 1 - idx; };
  auto issue_tile = [&](int hl, int idx, int buf, int rslot) {
    const int hq = hk * a.n_rep + hl;
    const int qt = qtile_of(idx);
    qdma.issue(make_rsrc_words((const T*)a.q + b * a.qs[0] + hq * a.qs[1], q_span), (unsigned)qt * q_tile_bytes,
               smem + Q_AT + buf * Q_BYTES, wave);
    dodma.issue(make_rsrc_words((const T*)a.dout + b * a.dos[0] + hq * a.dos[1], do_span), (unsigned)qt * do_tile_bytes,
                smem + DO_AT + buf * DO_BYTES, wave);
    // waves 0..2 fetch one 64-entry row vector each: 4 bytes per lane, rows past Sq arrive as zeros
    const int64_t ro = ((int64_t)b * a.Hq + hq) * Sq;
    const void* src = wave == 0 ? (const void*)(lse2 + ro) : wave == 1 ? (const void*)(a.delta + ro)
                    : wave == 2 ? (const void*)segb : (const void*)a.mx.qpos;
    if (wave < 2 || (wave == 2 && has_seg) || (wave == 3 && has_pos))
      dma_dword(make_rsrc_words(src, (unsigned)Sq * 4u), (unsigned)(qt * BMQ) * 4u, rows_base + rslot * ROW_BYTES + wave * BMQ * 4, lane);
  };

  // per-lane byte offsets of the MFMA fragments inside a tile (the swizzles are resolved once, here)
  unsigned faq[KS_QK], fao[KS_DV];
#pragma unroll
  for (int ks = 0; ks < KS_QK; ks++) faq[ks] = (unsigned)QT::off(ln, 2 * ks + g);
#pragma unroll
  for (int ks = 0; ks < KS_DV; ks++) fao[ks] = (unsigned)OT::off(ln, 2 * ks + g);

  f32x16 dkacc[DKB], dvacc[DVB];
  {
    // whole-vector values from the start: element-wise initialisation makes the compiler track 16 scalars per
    // accumulator across the loop and reassemble the tuple around every accumulating MFMA
    f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int d = 0; d < DKB; d++) {
      asm volatile("" : "+a"(zero16));
      dkacc[d] = zero16;
    }
#pragma unroll
    for (int d = 0; d < DVB; d++) {
      asm volatile("" : "+a"(zero16));
      dvacc[d] = zero16;
    }
  }
  const float c = a.scale_log2;

  // wave-level decisions for a query tile (uniform): skip if every query row precedes every kv row
  // (lo, hi: id range of the query tile; t: its index into the position ranges)
  // (The decisions are taken on the wave's first kv row as it arrives, in a vector register.  With a scalar copy the
  // compiler turns the choice of the tile body into scalar branches and copies the pinned accumulators between them,
  // right behind the MFMAs that write them: the build's hazard check rejects that code.  The same change in the
  // forward and the lean dQ kernel passed the check and ran 45 % and 64 % slower.)
  auto tile_mode_of = [&](int lo, int hi, int t, int qi0) {  // 0 = nothing to compute, 1 = no masking needed, 2 = masked
    bool skip = (CAUSAL && (qi0 + BMQ - 1 + band_hi < wkv0 || qi0 - band_lo > wkv0 + 31)) || wkv0 >= Skv;
    bool need_mask = (qi0 + BMQ > Sq) || (wkv0 + 32 > Skv) ||
                     (CAUSAL && (qi0 + band_hi < wkv0 + 31 || qi0 + BMQ - 1 - band_lo > wkv0));
    if (SEG) {
      skip = skip || hi < wkmin || lo > wkmax;
      need_mask = need_mask || !(lo == hi && wkmin == wkmax && lo == wkmin);
    }
    if (ext) {
      const int plo = pmin[t], phi = pmax[t];
      skip = skip || wkv0 > phi + a.mx.hi_off || wkv0 + 31 < plo - a.mx.lo_off;
      need_mask = need_mask || capped || biased || !(wkv0 >= phi - a.mx.lo_off && wkv0 + 31 <= plo + a.mx.hi_off);
    }
    return skip ? 0 : (need_mask ? 2 : 1);
  };
  auto tile_mode = [&](int idx, int qi0) {
    const int* e = ctl + 4 * idx;
    return tile_mode_of(SEG ? e[1] : 0, SEG ? e[2] : 0, SEG ? e[3] : 0, qi0);
  };
  // iteration -> (query head of the group, query tile): heads outer, tiles inner, no division in the loop.  (Tiles
  // outer would keep the group's workgroups on the same tile for the whole launch and cut the fetches from memory to
  // 1.8 GB at the benchmark's shape, against 6.5 GB this way - and ran 4 % slower: 32 CUs asking one L2 for the same
  // lines at the same time, and the descriptors rebuilt every tile.)
  auto advance = [&](int& hl, int& idx) {
    if (++idx == nact) { idx = 0; hl++; }
  };

  {
    // Software pipeline over query tiles t, three row-major buffers and three row-vector slots (tile t lives in
    // buffer and slot t % 3), one barrier per tile:
    //   part 1 (S, dP: fragment reads of buffer t % 3)
    //   wait for this wave's share of tile t+1 (issued a whole tile earlier), barrier
    //                                  -> tile t+1 has landed for everybody, everybody is done with tile t-1
    //   part 2 (dV, dK: transposing reads of buffer t % 3), with the loads of tile t+2 issued between its MFMAs
    //   into the buffer tile t-1 used
    int c_hl = 0, c_idx = 0, n_hl = 0, n_idx = 0;  // tile being computed, tile whose loads are issued next
    // Per-lane LDS byte addresses of the operands inside a tile (base of the workgroup's LDS included), each an
    // opaque register: every read below is such a register plus an immediate.  (Formed from the `smem` symbol, the
    // same addresses cost an add per read whenever the constant part happens to be zero, and the compiler
    // recomputes what it could have kept.)  Addresses into the dO tiles carry O_BIAS: constants there would
    // otherwise exceed the reach of an instruction offset.
    //   aq / ao   fragment reads of the row-major tiles (S, dP): row ln, chunk 2 ks + g
    //   trq / tro transposing reads (dK, dV): head-dim block d (32 columns), half h2 (rows +8); the query block and
    //             the k-step are immediates (multiples of 16 rows leave the swizzle alone)
    constexpr int O_BIAS = DO_AT;
    const unsigned lb = (unsigned)(size_t)smem;
    unsigned aq[KS_QK], ao[KS_DV], trq[DKB][2], tro[DVB][2];
#pragma unroll
    for (int ks = 0; ks < KS_QK; ks++) { aq[ks] = faq[ks] + lb; asm volatile("" : "+v"(aq[ks])); }
#pragma unroll
    for (int ks = 0; ks < KS_DV; ks++) { ao[ks] = fao[ks] + lb + (unsigned)O_BIAS; asm volatile("" : "+v"(ao[ks])); }
#pragma unroll
    for (int d = 0; d < DKB; d++)
#pragma unroll
      for (int h2 = 0; h2 < 2; h2++) {
        trq[d][h2] = (unsigned)QT::tr_off(8 * h2 + 4 * g, 2 * d + ((lane >> 4) & 1), lane & 15) + lb;
        asm volatile("" : "+v"(trq[d][h2]));
      }
#pragma unroll
    for (int d = 0; d < DVB; d++)
#pragma unroll
      for (int h2 = 0; h2 < 2; h2++) {
        tro[d][h2] = (unsigned)OT::tr_off(8 * h2 + 4 * g, 2 * d + ((lane >> 4) & 1), lane & 15) + lb + (unsigned)O_BIAS;
        asm volatile("" : "+v"(tro[d][h2]));
      }
    auto ld16 = [](unsigned addr) { return *(const __attribute__((address_space(3))) v8*)addr; };
    auto ldtr = [](unsigned a0, unsigned a1) {
      return tr_read8<v8>((const __attribute__((address_space(3))) unsigned char*)a0, (const __attribute__((address_space(3))) unsigned char*)a1);
    };
    if (n_iter > 0) { issue_tile(n_hl, n_idx, 0, 0); advance(n_hl, n_idx); }
    if (n_iter > 1) { issue_tile(n_hl, n_idx, 1, 1); advance(n_hl, n_idx); }
    // the control entry of the tile being computed and the query tile whose loads are issued next, as scalars; their
    // successors are read at the top of a tile and taken over at its end
    auto entry = [&](int idx) {
      if constexpr (SEG) return *(const i32x4*)(ctl + 4 * min(idx, max(nact - 1, 0)));
      else return i32x4{nqt_all - 1 - idx, 0, 0, 0};
    };
    auto scalar4 = [&](i32x4 v) {
      return i32x4{__builtin_amdgcn_readfirstlane(v[0]), __builtin_amdgcn_readfirstlane(v[1]),
                   __builtin_amdgcn_readfirstlane(v[2]), __builtin_amdgcn_readfirstlane(v[3])};
    };
    i32x4 cur = scalar4(entry(0));
    int nq_cur = __builtin_amdgcn_readfirstlane(entry(n_idx)[0]);
    // all earlier loads (the K/V fragments, the first tiles) have landed
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    // fragment ring: slot i's LDS fragment is requested AHEAD slots earlier and kept in fr[i % NF]; the
    // first AHEAD fragments of a tile are requested at the end of the tile before it (its row-major
    // tiles are complete by then), so that the LDS round trip and the scalar bookkeeping at the top of
    // the loop overlap
    constexpr int AHEAD = KS_QK >= 8 ? 5 : 3, NF = AHEAD + 1;
    v8 fr[NF];
    static_for<0, AHEAD>([&](auto I) {
      constexpr int i = decltype(I)::value;
      static_assert(AHEAD <= KS_QK, "the carried fragments all belong to S of the first query block");
      fr[i % NF] = ld16(aq[i] + Q_AT);
    });
    struct { u32x4 rq, ro, rr; unsigned offq, offo, offr; } nx;
    const unsigned lds_base = __builtin_amdgcn_readfirstlane((unsigned)(size_t)smem);
    const unsigned wave_q = __builtin_amdgcn_readfirstlane((unsigned)(wave * QT::PER_WAVE * 1024));
    const unsigned wave_o = __builtin_amdgcn_readfirstlane((unsigned)(wave * OT::PER_WAVE * 1024));
    const unsigned wave_r = __builtin_amdgcn_readfirstlane((unsigned)(wave * BMQ * 4));
    // one query tile; the buffer index is a constant (the loop below rotates three copies of this)
    auto iteration = [&](auto BUFc, const int it) {
      constexpr int buf = decltype(BUFc)::value;
      const int qi0 = cur[0] * BMQ;
      const int mode = tile_mode_of(cur[1], cur[2], cur[3], qi0);
      const bool issue_next = it + 2 < n_iter;
      // successors of the two cursors (read now, used when this tile is done)
      int c_hl2 = c_hl, c_idx2 = c_idx, n_hl2 = n_hl, n_idx2 = n_idx;
      advance(c_hl2, c_idx2);
      if (issue_next) advance(n_hl2, n_idx2);
      const i32x4 cur_next = entry(c_idx2);
      const int nq_next = entry(n_idx2)[0];
      constexpr int buf1 = (buf + 1) % 3, buf2 = (buf + 2) % 3;  // tile t+1 (read first in the next iteration), tile t+2
      constexpr unsigned ql = Q_AT + buf * Q_BYTES;                // + aq[] / trq[]
      constexpr unsigned dol = DO_AT + buf * DO_BYTES - O_BIAS;    // + ao[] / tro[]
      constexpr unsigned nxq = Q_AT + buf1 * Q_BYTES;
      const float* lsel = (const float*)(rows_base + buf * ROW_BYTES);
      const float* deltal = lsel + BMQ;
      const int* segl = (const int*)(deltal + BMQ);
      const int* posl = segl + BMQ;  // query positions of the tile's rows (mask extensions)
      const float* bias_head = biased ? a.mx.bias + b * a.mx.bias_s[0] + (hk * a.n_rep + c_hl) * a.mx.bias_s[1] : nullptr;
      // LDS destinations of this wave's loads of tile t+2 (scalar byte addresses)
      const unsigned dma_q = lds_base + (unsigned)(Q_AT + buf2 * Q_BYTES) + wave_q;
      const unsigned dma_o = lds_base + (unsigned)(DO_AT + buf2 * DO_BYTES) + wave_o;
      const unsigned dma_r = lds_base + (unsigned)(NBUF * BUF_BYTES + buf2 * ROW_BYTES) + wave_r;
      // descriptors of tile t+2's loads (wave-uniform), issued piecewise in part 2.  The bases change with
      // the query head only; they are rebuilt when a new head starts (and when the tiles run out: size 0).
      if (it == 0 || n_idx == 0 || !issue_next) {
        const int hq = hk * a.n_rep + (issue_next ? n_hl : 0);
        nx.rq = make_rsrc_words((const T*)a.q + b * a.qs[0] + hq * a.qs[1], issue_next ? q_span : 0u);
        nx.ro = make_rsrc_words((const T*)a.dout + b * a.dos[0] + hq * a.dos[1], issue_next ? do_span : 0u);
        const int64_t ro = ((int64_t)b * a.Hq + hq) * Sq;
        const void* src = wave == 0 ? (const void*)(lse2 + ro) : wave == 1 ? (const void*)(a.delta + ro)
                        : wave == 2 ? (const void*)segb : (const void*)a.mx.qpos;
        // a wave with no row vector to fetch (wave 2 without segment ids, wave 3 without query positions): size 0
        nx.rr = make_rsrc_words(src, (issue_next && (wave < 2 || (wave == 2 && has_seg) || (wave == 3 && has_pos))) ? (unsigned)Sq * 4u : 0u);
      }
      {
        const int qt = issue_next ? nq_cur : 0;
        nx.offq = __builtin_amdgcn_readfirstlane((unsigned)qt * q_tile_bytes);
        nx.offo = __builtin_amdgcn_readfirstlane((unsigned)qt * do_tile_bytes);
        nx.offr = __builtin_amdgcn_readfirstlane((unsigned)(qt * BMQ) * 4u);
      }

      // The tile body is laid out by hand as a sequence of slots, one MFMA each, with a scheduling barrier
      // after every slot: the LDS fragment a slot needs was requested AHEAD slots earlier, and the
      // exponentials / products that turn S, dP into the 16-bit operands P, dS are spread over the slots
      // under the MFMAs of the other query block.  (Left to itself the compiler reads each fragment right
      // before its MFMA and the matrix unit waits out every LDS round trip.)
      //   slots   part 1: S0 = Q0 K^T, S1 = Q1 K^T, dP0 = dO0 V^T, dP1 = dO1 V^T
      //           part 2: dV^T += dO0^T P0, dK^T += Q0^T dS0, dV^T += dO1^T P1, dK^T += Q1^T dS1
      //   VALU    P0 from S1 on, P1 from dP0 on, dS0 from dP1 on, dS1 from part 2 on
      auto body = [&](auto mode_c) {
        constexpr int MODE = decltype(mode_c)::value;
        constexpr bool COMPUTE = MODE != 0, MASKED = MODE == 2;
        // part 1: S0, S1, dP0, dP1 (the exponentials can start as soon as S0 is complete and are over
        // before part 2, which carries the transposition of the next tile);
        // part 2: dV0, dK0, dV1, dK1 (four accumulators each, used round robin)
        // (K1 / K2 k-steps per S / dP product; CLV / CLK slots per query block of dV / dK)
        constexpr int K1 = KS_QK, K2 = KS_DV, CLV = 2 * DVB, CLK = 2 * DKB;
        constexpr int S1_AT = K1, D0_AT = 2 * K1, D1_AT = 2 * K1 + K2, C0 = 2 * (K1 + K2);
        constexpr int V0_AT = C0, K0_AT = V0_AT + CLV, V1_AT = K0_AT + CLK, K1_AT = V1_AT + CLV, NS = K1_AT + CLK;
        // VALU groups of VL slots each: P of a block starts when its S is complete, dS when its dP is; each
        // group is over before the MFMAs that consume its packed operand
        constexpr int EPS = K2 >= 8 ? 1 : 2, VL = 16 / EPS;
        constexpr int VP0 = S1_AT, VP1 = D0_AT, VS0 = D1_AT, VS1 = C0;
        static_assert(VP0 + VL <= V0_AT && VS0 + VL <= K0_AT && VP1 + VL <= V1_AT && VS1 + VL <= K1_AT, "operands not ready");
        constexpr int N_DMA = QT::PER_WAVE + OT::PER_WAVE + 1, DMA_EVERY = (NS - C0) / N_DMA;
        static_assert(DMA_EVERY >= 1, "second half too short for the loads");
        const int kvcol = wkv0 + ln;
        f32x16 s[2], dp[2];
        v8 pf[2][2], df[2][2];
        // -LSE (log2 units) and -delta of the 16 rows a lane holds of either query block.  LDS reads return in
        // order, so each group is requested a ring depth or more before its first use: waiting for it then waits
        // for no fragment that is not due anyway
        f32x4 nl0[4], nl1[4], nd0[4], nd1[4];
        float fc[2][16];  // soft cap: 1 - tanh^2 of every score, kept from P to dS
        // Masked tiles without the mask extensions: which of the tile's 64 query rows this lane's kv column may see,
        // as one bit per row, built once per tile (bounds and causality are a bit range; the rows of each id present
        // among the wave's columns come from a ballot over the tile's id vector).  An element then costs a bit-field
        // extract and an AND instead of four compares.  rowbits[qb] is shifted so that value v of the lane's 16 is
        // bit 8 (v / 4) + v % 4.
        unsigned rowbits[2] = {0u, 0u};
        const bool by_bits = MASKED && !(GEN && ext);
        if (MASKED && by_bits) {
          const int lo_r = CAUSAL ? max(kvcol - band_hi - qi0, 0) : 0;
          int hi_r = kvcol < Skv ? min(Sq - qi0, BMQ) : 0;
          if (CAUSAL) hi_r = min(hi_r, kvcol + band_lo - qi0 + 1);
          unsigned long long m = 0ull;
          if (hi_r > lo_r) m = (~0ull << lo_r) & (~0ull >> (64 - hi_r));
          if (SEG && has_seg) {
            const int rowseg = segl[lane];  // lane l: id of the tile's query row l
            unsigned long long ms = 0ull, todo = ~0ull;
            while (todo) {
              const int x = __builtin_amdgcn_readlane(segk, (int)__builtin_ctzll(todo));
              const unsigned long long rows = __ballot(rowseg == x);
              const bool mine = segk == x;
              ms = mine ? rows : ms;
              todo &= ~__ballot(mine);
            }
            m &= ms;
          }
          rowbits[0] = (unsigned)m >> (4 * g);
          rowbits[1] = (unsigned)(m >> 32) >> (4 * g);
        }

        auto frag = [&](auto I) -> v8 {
          constexpr int i = decltype(I)::value;
          if constexpr (i < D0_AT) {
            constexpr int qb = i / K1, ks = i % K1;
            return ld16(aq[ks] + (ql + qb * 32 * QT::ROWB));
          } else if constexpr (i < C0) {
            constexpr int qb = (i - D0_AT) / K2, ks = (i - D0_AT) % K2;
            return ld16(ao[ks] + (dol + qb * 32 * OT::ROWB));
          } else {
            // operand of an accumulating product: rows = head-dim block d, contraction over query rows
            // 32 qb + 16 hh + {4g..4g+3, 8+4g..8+4g+3} (the order in which P / dS hold them), read transposed
            constexpr int qb = i >= V1_AT ? 1 : 0, base = qb ? V1_AT : V0_AT;
            if constexpr (i - base < CLV) {
              constexpr int j = i - base, hh = j / DVB, d = j % DVB;
              constexpr int rows = (32 * qb + 16 * hh) * OT::ROWB;
              return ldtr(tro[d][0] + (dol + rows), tro[d][1] + (dol + rows));
            } else {
              constexpr int j = i - base - CLV, hh = j / DKB, d = j % DKB;
              constexpr int rows = (32 * qb + 16 * hh) * QT::ROWB;
              return ldtr(trq[d][0] + (ql + rows), trq[d][1] + (ql + rows));
            }
          }
        };
        auto mma = [&](auto I, const v8& f) {
          constexpr int i = decltype(I)::value;
          const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          if constexpr (i < D0_AT) {
            constexpr int qb = i / K1, ks = i % K1;
            s[qb] = MT<T>::mfma32(f, kf[ks], ks == 0 ? zero : s[qb]);
          } else if constexpr (i < C0) {
            constexpr int qb = (i - D0_AT) / K2, ks = (i - D0_AT) % K2;
            if constexpr (ks == 0) {
              // dP starts from -delta of its rows (C layout: value v belongs to row 8 (v/4) + 4 g + v%4), so
              // that dS = P o dP needs no subtraction
              const f32x4 (&nd)[4] = qb == 0 ? nd0 : nd1;
              const f32x16 init = {nd[0][0], nd[0][1], nd[0][2], nd[0][3], nd[1][0], nd[1][1], nd[1][2], nd[1][3],
                                   nd[2][0], nd[2][1], nd[2][2], nd[2][3], nd[3][0], nd[3][1], nd[3][2], nd[3][3]};
              dp[qb] = MT<T>::mfma32(f, vf[ks], init);
            } else {
              dp[qb] = MT<T>::mfma32(f, vf[ks], dp[qb]);
            }
          } else {
            constexpr int qb = i >= V1_AT ? 1 : 0, base = qb ? V1_AT : V0_AT;
            if constexpr (i - base < CLV) {
              constexpr int j = i - base, hh = j / DVB, d = j % DVB;
              MT<T>::mfma32_acc(dvacc[d], f, pf[qb][hh]);
            } else {
              constexpr int j = i - base - CLV, hh = j / DKB, d = j % DKB;
              MT<T>::mfma32_acc(dkacc[d], f, df[qb][hh]);
            }
          }
        };
        // VALU group of query block QB starting at slot START: EPS elements per slot for VL slots.
        // IS_P: s <- exp2(s c - lse) (masked), else dp <- s (dp - delta); the 16-bit operands are packed as
        // soon as the eight values of a half are done.
        auto valu = [&](auto I, auto START, auto QBc, auto IS_Pc) {
          constexpr int i = decltype(I)::value, st = decltype(START)::value, qb = decltype(QBc)::value;
          constexpr bool IS_P = decltype(IS_Pc)::value;
          constexpr int QS = 4 / EPS;  // slots per quad of rows
          if constexpr (i >= st && i < st + VL) {
            constexpr int k = i - st, vq = k / QS;
#pragma unroll
            for (int e2 = 0; e2 < EPS; e2++) {
              const int e = EPS * (k % QS) + e2, v = 4 * vq + e;
              if constexpr (IS_P) {
                const f32x4 (&nl)[4] = qb == 0 ? nl0 : nl1;
                float sval = s[qb][v];
                if (GEN && MASKED) {
                  if (capped) {
                    const float th = fast_tanh(sval * a.mx.cap_in);
                    fc[qb][v] = 1.f - th * th;
                    sval = a.mx.cap_out * th;
                  }
                  if (biased) {  // additive mask, in units of the raw score (-inf stays -inf)
                    const int qrow_b = min(qi0 + qb * 32 + 8 * vq + 4 * g + e, Sq - 1);
                    sval += a.mx.bias_mul * bias_head[(int64_t)qrow_b * a.mx.bias_s[2] + min(kvcol, Skv - 1)];
                  }
                }
                float pv = fast_exp2(__builtin_fmaf(sval, c, nl[vq][e]));
                if (MASKED) {
                  if (by_bits) {
                    pv = __builtin_bit_cast(float, __builtin_bit_cast(int, pv) & __builtin_amdgcn_sbfe((int)rowbits[qb], 8 * vq + e, 1));
                  } else {
                    const int r = qb * 32 + 8 * vq + 4 * g + e;
                    const int qrow = qi0 + r;
                    bool ok = qrow < Sq && kvcol < Skv && (!CAUSAL || kvcol <= qrow) && (!SEG || !has_seg || segl[r] == segk);
                    if (GEN) {
                      if (ext) {
                        const int qp = has_pos ? posl[r] : qrow;
                        ok = ok && kvcol >= qp - a.mx.lo_off && kvcol <= qp + a.mx.hi_off;
                      }
                    }
                    pv = ok ? pv : 0.f;
                  }
                }
                asm volatile("" : "+v"(pv));  // anchors the computation in this slot (it would sink past the barrier)
                s[qb][v] = pv;
              } else {
                float dsv = s[qb][v] * dp[qb][v];
                if (GEN && MASKED) {
                  if (capped) dsv *= fc[qb][v];  // derivative of the capped score with respect to the raw one
                }
                asm volatile("" : "+v"(dsv));
                dp[qb][v] = dsv;
              }
            }
            if constexpr (((k + 1) * EPS) % 8 == 0) {
              constexpr int hh = (k + 1) * EPS / 8 - 1;
              const f32x16& x = IS_P ? s[qb] : dp[qb];
              const v8 packed = pack8<T>(x[8 * hh + 0], x[8 * hh + 1], x[8 * hh + 2], x[8 * hh + 3], x[8 * hh + 4],
                                         x[8 * hh + 5], x[8 * hh + 6], x[8 * hh + 7]);
              if constexpr (IS_P) pf[qb][hh] = packed;
              else df[qb][hh] = packed;
            }
          }
        };
        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, 1> I1;
        static_for<0, NS>([&](auto I) {
          constexpr int i = decltype(I)::value;
          if constexpr (i == C0) {
            // this wave's loads of tile t+1 were issued a tile ago (vmcnt only: fragment reads stay in flight)
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
          }
          // the loads of tile t+2, one instruction every few slots: the texture path takes a kilobyte in
          // some 25 cycles for the whole CU, and a wave that issues them back to back sits out the queue
          if constexpr (i >= C0 && (i - C0) % DMA_EVERY == 0 && (i - C0) / DMA_EVERY < N_DMA) {
            constexpr int m = (i - C0) / DMA_EVERY;
            // (no branch here: past the last tile the descriptors have size 0 and the loads deliver zeros
            // into buffers nobody reads any more)
            if constexpr (m < QT::PER_WAVE) qdma.template issue_one_at<m>(nx.rq, nx.offq, dma_q);
            else if constexpr (m < QT::PER_WAVE + OT::PER_WAVE) dodma.template issue_one_at<m - QT::PER_WAVE>(nx.ro, nx.offo, dma_o);
            else dma_dword_at(nx.rr, nx.offr, dma_r, lane);
          }
          if constexpr (COMPUTE) {
            // row vectors, a quad of rows at a time: -LSE of query block qb LEAD slots before the exponentials of that
            // quad (VP0 / VP1 + QS vq), -delta two slots before the first dP MFMA of the block (2K, 3K)
            constexpr int QS = 4 / EPS, LEAD = 3;
            static_for<0, 4>([&](auto VQ) {
              constexpr int vq = decltype(VQ)::value;
              constexpr int r0 = VP0 + QS * vq - LEAD, r1 = VP1 + QS * vq - LEAD;
              if constexpr (i == (r0 < 0 ? 0 : r0)) nl0[vq] = *(const f32x4*)(lsel + 8 * vq + 4 * g);
              if constexpr (i == (r1 < 0 ? 0 : r1)) nl1[vq] = *(const f32x4*)(lsel + 32 + 8 * vq + 4 * g);
            });
            if constexpr (i == D0_AT - 2) {
#pragma unroll
              for (int vq = 0; vq < 4; vq++) nd0[vq] = *(const f32x4*)(deltal + 8 * vq + 4 * g);
            }
            if constexpr (i == D1_AT - 2) {
#pragma unroll
              for (int vq = 0; vq < 4; vq++) nd1[vq] = *(const f32x4*)(deltal + 32 + 8 * vq + 4 * g);
            }
            if constexpr (i + AHEAD < NS) fr[(i + AHEAD) % NF] = frag(std::integral_constant<int, i + AHEAD>{});
            mma(I, fr[i % NF]);
            valu(I, std::integral_constant<int, VP0>{}, I0{}, std::true_type{});
            valu(I, std::integral_constant<int, VP1>{}, I1{}, std::true_type{});
            valu(I, std::integral_constant<int, VS0>{}, I0{}, std::false_type{});
            valu(I, std::integral_constant<int, VS1>{}, I1{}, std::false_type{});
          }
          __builtin_amdgcn_sched_barrier(0);
        });
        static_for<0, AHEAD>([&](auto I) {
          constexpr int i = decltype(I)::value;
          fr[i % NF] = ld16(aq[i] + nxq);
        });
      };
      if (mode == 1) body(std::integral_constant<int, 1>{});
      else if (mode == 2) body(std::integral_constant<int, 2>{});
      else body(std::integral_constant<int, 0>{});
      n_hl = n_hl2; n_idx = n_idx2;
      c_hl = c_hl2; c_idx = c_idx2;
      cur = scalar4(cur_next);
      nq_cur = __builtin_amdgcn_readfirstlane(nq_next);
    };
    for (int it = 0; it < n_iter; it += 3) {
      iteration(std::integral_constant<int, 0>{}, it);
      if (it + 1 < n_iter) iteration(std::integral_constant<int, 1>{}, it + 1);
      if (it + 2 < n_iter) iteration(std::integral_constant<int, 2>{}, it + 2);
    }
  }

  // every LDS-writing load of this wave has landed before it leaves (the last ones write zeros nobody reads,
  // but they must not outlive the workgroup's LDS allocation)
  __builtin_amdgcn_s_waitcnt(0);
  // The accumulating MFMAs are opaque assembly (mfma32_acc): the compiler does not know that dkacc / dvacc come
  // out of a 16-pass matrix instruction and inserts no wait states before reading them.  Make the distance
  // explicit (the longest MFMA-write -> VALU-read hazard is 18 wait states).
  // (the accumulators are operands of the statement, so that no read of them can be scheduled ahead of it)
  static_assert(DKB <= 6 && DVB <= 4, "operand lists below");
  asm volatile("s_nop 15\n\ts_nop 3" : "+a"(dkacc[0]), "+a"(dkacc[1]), "+a"(dvacc[0]), "+a"(dvacc[1]) :: "memory");
  if constexpr (DKB > 2) asm volatile("" : "+a"(dkacc[2]), "+a"(dkacc[3]));
  if constexpr (DKB > 4) asm volatile("" : "+a"(dkacc[4]), "+a"(dkacc[5]));
  if constexpr (DVB > 2) asm volatile("" : "+a"(dvacc[2]), "+a"(dvacc[3]));
  // ---- epilogue: lane = kv row, 4 consecutive head-dim values per store
  const int row = wkv0 + ln;
  if (row < Skv) {
    T* dkp = (T*)a.dk + b * a.dks[0] + hk * a.dks[1] + row * a.dks[2];
    T* dvp = (T*)a.dv + b * a.dvs[0] + hk * a.dvs[1] + row * a.dvs[2];
    const float sc = a.sm_scale;
#pragma unroll
    for (int d = 0; d < DKB; d++)
#pragma unroll
      for (int vq = 0; vq < 4; vq++) {
        const f32x16& o = dkacc[d];
        *(u32x2*)(dkp + d * 32 + 8 * vq + 4 * g) =
            pack4<T>(o[4 * vq] * sc, o[4 * vq + 1] * sc, o[4 * vq + 2] * sc, o[4 * vq + 3] * sc);
      }
#pragma unroll
    for (int d = 0; d < DVB; d++)
#pragma unroll
      for (int vq = 0; vq < 4; vq++) {
        const f32x16& o = dvacc[d];
        *(u32x2*)(dvp + d * 32 + 8 * vq + 4 * g) = pack4<T>(o[4 * vq], o[4 * vq + 1], o[4 * vq + 2], o[4 * vq + 3]);
      }
  }
}

// ------------------------------------------------------------------------------------------------
// dQ
// ------------------------------------------------------------------------------------------------
// NW = waves per workgroup.  With 8 (head dims up to 128) two waves share a SIMD, 256 registers each: a wave
// issues at most one instruction every four cycles, and at ~600 instructions for 48 MFMAs per tile a single
// wave per SIMD leaves the matrix unit idle most of the time, whatever the order of its instructions.
template <typename T, int DQK, int DV, int NW, bool CAUSAL, bool SEG>
__global__ __launch_bounds__(64 * NW) void attn_bwd_dq_kernel(const BwdArgs a) {
  typedef typename MT<T>::v8 v8;
  constexpr int BN = 64, BM = 32 * NW;
  static_assert(NW == 4 || (NW == 8 && DQK == DV && DQK <= 128), "8 waves: equal head dims up to 128");
  constexpr int KS_QK = DQK / 16, KS_DV = DV / 16, DKB = DQK / 32;
  typedef RowTile<DQK> KT;
  typedef RowTile<DV> VT;
  constexpr int K_BYTES = BN * KT::STRIDE, V_BYTES = BN * VT::STRIDE, KTR_BYTES = DQK * TrTile64::ROW_BYTES;
  // LDS: two row-major K/V buffers, NKTR transposed K tiles (three with 8 waves: the dQ MFMAs of a tile's
  // second kv block run in the next iteration), two segment-id rows, then the per-tile id ranges
  constexpr int NKTR = NW == 8 ? 3 : 2;
  constexpr int KV_BYTES = K_BYTES + V_BYTES;
  constexpr int KTR_AT = 2 * KV_BYTES, SEG_AT = KTR_AT + NKTR * KTR_BYTES, META_AT = SEG_AT + 2 * BN * 4;

  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, ln = lane & 31;
  const int n_qt = (a.Sq + BM - 1) / BM;
  int tile, inner, group;
  if (!xcd_map(n_qt, a.n_rep, a.B * a.Hkv, tile, inner, group)) return;
  const int qt = n_qt - 1 - tile;
  const int b = group / a.Hkv, hk = group - b * a.Hkv, h = hk * a.n_rep + inner;
  const int q0 = qt * BM, wq0 = q0 + wave * 32;
  const int Sq = a.Sq, Skv = a.Skv;
  const T* kb = (const T*)a.k + b * a.ks[0] + hk * a.ks[1];
  const T* vb = (const T*)a.v + b * a.vs[0] + hk * a.vs[1];
  constexpr bool GEN = !CAUSAL && SEG;  // also evaluates the mask extensions (and may then run without segment ids)
  const bool has_seg = SEG && (!GEN || a.seg != nullptr);
  const bool ext = GEN && a.mx.on;
  const bool capped = GEN && a.mx.cap_in != 0.f;
  const bool biased = GEN && a.mx.bias != nullptr;
  const int32_t* segb = has_seg ? a.seg + (int64_t)b * Skv : nullptr;

  const int kv_end = CAUSAL ? min(Skv, q0 + BM) : Skv;
  const int ntiles = (kv_end + BN - 1) / BN;

  // ---- Q, dO fragments (B operands: lane = query column), per-lane LSE / delta
  const int qrow_c = min(wq0 + ln, Sq - 1);
  v8 qf[KS_QK], dof[KS_DV];
  {
    const T* qp = (const T*)a.q + b * a.qs[0] + h * a.qs[1] + qrow_c * a.qs[2] + 8 * g;
    const T* dp = (const T*)a.dout + b * a.dos[0] + h * a.dos[1] + qrow_c * a.dos[2] + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS_QK; ks++) qf[ks] = *(const v8*)(qp + 16 * ks);
#pragma unroll
    for (int ks = 0; ks < KS_DV; ks++) dof[ks] = *(const v8*)(dp + 16 * ks);
  }
  const int64_t ro = ((int64_t)b * a.Hq + h) * Sq + qrow_c;
  const float lraw = a.lse[ro];
  const float lse_s = (lraw == -INFINITY) ? INFINITY : lraw * LOG2E;
  const float ndelta_s = a.delta[ro];  // -rowsum(dO o O)
  const int segq = has_seg ? segb[qrow_c] : 0;
  // additive mask: this lane's query row of it
  const float* bias_row = biased ? a.mx.bias + b * a.mx.bias_s[0] + h * a.mx.bias_s[1] + (int64_t)qrow_c * a.mx.bias_s[2] : nullptr;
  // band of allowed keys of this lane's query row, and the positions' extent over the wave
  int lo_q = -BAND_INF, hi_q = BAND_INF, wpmin = 0, wpmax = 0;
  if (ext) {
    const int qp = a.mx.qpos ? a.mx.qpos[qrow_c] : qrow_c;
    lo_q = qp - a.mx.lo_off;
    hi_q = qp + a.mx.hi_off;
    wpmin = qp; wpmax = qp;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) {
      wpmin = min(wpmin, __shfl_xor(wpmin, o, 64));
      wpmax = max(wpmax, __shfl_xor(wpmax, o, 64));
    }
    wpmin = __builtin_amdgcn_readfirstlane(wpmin);
    wpmax = __builtin_amdgcn_readfirstlane(wpmax);
  }

  int* kvmin = (int*)(smem + META_AT);
  int* kvmax = kvmin + ntiles;
  int* active = kvmax + ntiles;
  int* bq = active + ntiles;
  int nact = ntiles;
  int wqmin = 0, wqmax = 0;
  if (SEG) {
    wqmin = segq; wqmax = segq;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) {
      wqmin = min(wqmin, __shfl_xor(wqmin, o, 64));
      wqmax = max(wqmax, __shfl_xor(wqmax, o, 64));
    }
    wqmin = __builtin_amdgcn_readfirstlane(wqmin);
    wqmax = __builtin_amdgcn_readfirstlane(wqmax);
    if (lane == 0) { bq[2 * wave] = wqmin; bq[2 * wave + 1] = wqmax; bq[2 * NW + 2 * wave] = wpmin; bq[2 * NW + 2 * wave + 1] = wpmax; }
    if (has_seg) {
      seg_tile_ranges(segb, Skv, 0, ntiles, kvmin, kvmax, tid, 64 * NW);
    } else {
      for (int t = tid; t < ntiles; t += 64 * NW) { kvmin[t] = 0; kvmax[t] = 0; }
    }
    __syncthreads();
    int bqmin = bq[0], bqmax = bq[1], bpmin = bq[2 * NW], bpmax = bq[2 * NW + 1];
#pragma unroll
    for (int w = 1; w < NW; w++) {
      bqmin = min(bqmin, bq[2 * w]); bqmax = max(bqmax, bq[2 * w + 1]);
      bpmin = min(bpmin, bq[2 * NW + 2 * w]); bpmax = max(bpmax, bq[2 * NW + 2 * w + 1]);
    }
    const int b_lo = ext ? bpmin - a.mx.lo_off : -BAND_INF, b_hi = ext ? bpmax + a.mx.hi_off : BAND_INF;
    int cnt = 0;
    for (int base = 0; base < ntiles; base += 64) {
      const int t = base + lane;
      const bool act = t < ntiles && !(kvmax[t] < bqmin || kvmin[t] > bqmax) && t * BN <= b_hi && t * BN + BN - 1 >= b_lo;
      const unsigned long long m = __ballot(act);
      if (act && wave == 0) active[cnt + __popcll(m & ((1ull << lane) - 1ull))] = t;
      cnt += __popcll(m);
    }
    nact = cnt;
    __syncthreads();
    // One word per visited tile, in visiting order: the kv tile in the low half, above it two bits per wave (its rows'
    // ids miss the tile's range / the ranges are not one shared id).  The tile loop reads the word a tile ahead of
    // its use; it would otherwise start every tile by waiting out a chain of dependent LDS reads (list entry ->
    // ranges -> which body to run).
    for (int i = tid; i < nact; i += 64 * NW) {
      const int t = active[i], lo = kvmin[t], hi = kvmax[t];
      unsigned bits = 0;
#pragma unroll
      for (int w = 0; w < NW; w++) {
        const int wmin = bq[2 * w], wmax = bq[2 * w + 1];
        const unsigned sk = (hi < wmin || lo > wmax) ? 1u : 0u, nm = (lo == hi && wmin == wmax && lo == wmin) ? 0u : 2u;
        bits |= (sk | nm) << (2 * w);
      }
      active[i] = (int)((unsigned)t | (bits << 16));  // (thread i owns entry i: read above, replaced here)
    }
    __syncthreads();
  }
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);

  // ---- staging of one K/V tile through registers.  Every thread owns one 4-row x 8-column block of K and
  // (4 waves) one of V; with 8 waves the first four stage K, the last four V.
  const int stid = tid & 255;
  const rsrc_t krs = make_rsrc(kb, span_bytes(Skv, a.ks[2], DQK));
  const rsrc_t vrs = make_rsrc(vb, span_bytes(Skv, a.vs[2], DV));
  const unsigned k_tile_bytes = (unsigned)(BN * a.ks[2] * 2), v_tile_bytes = (unsigned)(BN * a.vs[2] * 2);
  Stage64<DQK> kst;
  Stage64<DV> vst;
  kst.init((NW == 4 || wave < 4) ? a.ks[2] : a.vs[2], stid);  // 8 waves: one set of offsets, the role's
  if (NW == 4) vst.init(a.vs[2], stid);
  int sreg = 0;
  // 8 waves: waves 0..3 stage K (and its transposed copy), waves 4..7 stage V, in the same registers
  auto stages_k = [&](int) { return NW == 4 || wave < 4; };
  auto load_tile = [&](int t, int it) {
    if (NW == 4) {
      kst.load(krs, (unsigned)t * k_tile_bytes, stid);
      vst.load(vrs, (unsigned)t * v_tile_bytes, stid);
    } else {
      // same registers for either role (the offsets and the resource are picked, not the code path)
      // (a scalar choice: with the descriptor in vector registers every load would sit in a loop over its
      // distinct values)
      const bool sk = __builtin_amdgcn_readfirstlane((int)stages_k(it)) != 0;
      const rsrc_t rs = sk ? krs : vrs;
      const unsigned off = sk ? (unsigned)t * k_tile_bytes : (unsigned)t * v_tile_bytes;
#pragma unroll
      for (int ii = 0; ii < 4; ii++) kst.r[0][ii] = buf_load16(rs, kst.vo[0][ii], off);
    }
    if (has_seg && tid < BN) sreg = segb[min(t * BN + tid, Skv - 1)];
  };
  // (kslot: which transposed tile; the row-major buffer is buf)
  auto store_tile = [&](int buf, int kslot, int it) {
    unsigned char* base = smem + buf * KV_BYTES;
    unsigned char* ktr = smem + KTR_AT + kslot * KTR_BYTES;
    if (NW == 4) {
      kst.store_rowmajor(base, stid);
      vst.store_rowmajor(base + K_BYTES, stid);
      kst.store_transposed(ktr, stid);
    } else if (stages_k(it)) {
      kst.store_rowmajor(base, stid);
      kst.store_transposed(ktr, stid);
    } else {
      kst.store_rowmajor(base + K_BYTES, stid);  // K and V tiles have the same shape here
    }
    if (SEG && tid < BN) ((int*)(smem + SEG_AT + buf * BN * 4))[tid] = sreg;
  };

  unsigned ta[4];  // per-lane byte offsets of the K^T fragments (swizzle resolved once)
#pragma unroll
  for (int m = 0; m < 4; m++) ta[m] = (unsigned)TrTile64::chunk_off(ln, m, g);

  // Wide heads, causal (four waves, one per SIMD, 512 registers each): the dQ accumulators are pinned to the
  // accumulation registers like dK / dV in the other kernel.  Not the other four-wave variants: there the branches
  // of the tile loop end with the accumulators in different registers and the compiler copies them right behind the
  // MFMAs, which it does not know to be MFMAs (the build's assembly scan rejects that).  Eight waves have 256
  // registers in all and keep the compiler's MFMA form.
  constexpr bool ACC_PINNED = NW == 4 && CAUSAL && DQK > 128;
  f32x16 dqacc[DKB];
  {
    f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int d = 0; d < DKB; d++) {
      if constexpr (ACC_PINNED) asm volatile("" : "+a"(zero16));
      dqacc[d] = zero16;
    }
  }
  const float c = a.scale_log2;
  const int wq_last = wq0 + 31;
  const int qrow = wq0 + ln;

  // i-th kv tile to visit, as a scalar (a tile offset in vector registers would put every staging load into a
  // loop over its distinct values)
  auto entry = [&](int i) { return SEG ? active[min(i, max(nact - 1, 0))] : i; };
  // entries of the tile being computed and of the one after it (whose loads are issued at the top of this one)
  int cur = __builtin_amdgcn_readfirstlane(entry(0)), nxt = __builtin_amdgcn_readfirstlane(entry(1));
  // Masked tiles: which of the tile's 64 kv rows this lane's query row may see, one bit per row, built once per tile
  // (bounds, causality and the band of the mask extensions are a bit range; the rows of each id present among the
  // wave's query rows come from a ballot over the tile's id vector).  An element then costs a bit-field extract and
  // an AND instead of its compares.  kbits[nb] is shifted so that value v of the lane's 16 is bit 8 (v / 4) + v % 4.
  unsigned kbits[2] = {0u, 0u};
  auto make_key_bits = [&](int kv0, const int* sl) {
    int lo = 0, hi = min(Skv - kv0, BN);
    if (CAUSAL) hi = min(hi, wq0 + ln - kv0 + 1);
    if (GEN) {
      lo = max(lo_q - kv0, 0);
      hi = min(hi, hi_q - kv0 + 1);
    }
    unsigned long long m = 0ull;
    if (hi > lo) m = (~0ull << lo) & (~0ull >> (64 - hi));
    if (SEG && has_seg) {
      const int rowseg = sl[lane];  // lane l: id of the tile's kv row l
      unsigned long long ms = 0ull, todo = ~0ull;
      while (todo) {
        const int x = __builtin_amdgcn_readlane(segq, (int)__builtin_ctzll(todo));
        const unsigned long long rows = __ballot(rowseg == x);
        const bool mine = segq == x;
        ms = mine ? rows : ms;
        todo &= ~__ballot(mine);
      }
      m &= ms;
    }
    kbits[0] = (unsigned)m >> (4 * g);
    kbits[1] = (unsigned)(m >> 32) >> (4 * g);
  };
  if (nact > 0) {
    load_tile(cur & 0xffff, 0);
    store_tile(0, 0, 0);
  }
  __builtin_amdgcn_s_waitcnt(0);  // Q / dO fragments, LSE and delta have landed (see the dK/dV kernel)
  __syncthreads();

  if constexpr (NW == 8) {
    // Eight waves (two per SIMD).  A wave's VALU work runs beside its own MFMAs only when the two are mixed
    // finely: a run of back-to-back MFMAs holds up the vector issue port of the SIMD, the other wave's
    // included.  So the element-wise work is cut into pieces of a few instructions, one per slot, and the
    // slots are ordered so that every piece has its inputs a slot or more before it runs:
    //   slots   S0 = K0 Q^T | dQ += K1'^T dS1' | dP0 = V0 dO^T | S1 = K1 Q^T | dQ += K0^T dS0 | dP1 = V1 dO^T
    //   VALU    dS1'        | P0 ..............................| dS0         | P1 ...........................
    // (primed: second kv block of the tile before, whose P and dP are carried over in s[1], dp[1]; its
    // transposed K tile is still in LDS, which is why there are three of them).  A wave that skips a tile,
    // and the end of the loop, finish the carried block on their own (drain).
    constexpr int A2 = 2 * DKB;
    constexpr int P1 = KS_QK, P2 = P1 + A2, P3 = P2 + KS_DV, P4 = P3 + KS_QK, P5 = P4 + A2, NS = P5 + KS_DV;
    constexpr int LEN_P = A2 + KS_DV - 1;  // slots of a P group (starts one slot after its S is complete)
    constexpr int AHEAD = 3, NF = 4;
    f32x16 s[2], dp[2];
#pragma unroll
    for (int v = 0; v < 16; v++) { s[1][v] = 0.f; dp[1][v] = 0.f; }
    // the first tile's carried block is all zeros: its K^T operand must be finite
    for (int o = tid * 16; o < KTR_BYTES; o += 64 * NW * 16) *(u32x4*)(smem + KTR_AT + 2 * KTR_BYTES + o) = u32x4{0u, 0u, 0u, 0u};
    __syncthreads();

    // dS of elements [LO, HI) of a block: d <- p (d - delta); a half is packed once its eight values are there
    auto ds_chunk = [&](auto LOc, auto HIc, const f32x16& p, f32x16& d, v8* dfb) {
      constexpr int lo = decltype(LOc)::value, hi = decltype(HIc)::value;
#pragma unroll
      for (int v = lo; v < hi; v++) {
        float dsv = p[v] * (d[v] + ndelta_s);
        asm volatile("" : "+v"(dsv));  // keeps the computation in its slot
        d[v] = dsv;
      }
      static_for<0, 2>([&](auto H) {
        constexpr int hh = decltype(H)::value;
        if constexpr (8 * hh + 8 > lo && 8 * hh + 8 <= hi)
          dfb[hh] = pack8<T>(d[8 * hh + 0], d[8 * hh + 1], d[8 * hh + 2], d[8 * hh + 3], d[8 * hh + 4], d[8 * hh + 5],
                             d[8 * hh + 6], d[8 * hh + 7]);
      });
    };
    // finishes the carried block without a tile around it
    auto drain = [&](const unsigned char* ktp) {
      v8 d1[2];
      ds_chunk(std::integral_constant<int, 0>{}, std::integral_constant<int, 16>{}, s[1], dp[1], d1);
#pragma unroll
      for (int j = 0; j < A2; j++) {
        const int hh = j / DKB, d = j % DKB;
        const v8 f = *(const v8*)(ktp + ta[(2 + hh) ^ (d & 3)] + d * 32 * TrTile64::ROW_BYTES);
        dqacc[d] = MT<T>::mfma32(f, d1[hh], dqacc[d]);
      }
#pragma unroll
      for (int v = 0; v < 16; v++) { s[1][v] = 0.f; dp[1][v] = 0.f; }
    };

    bool pending = false;
    int kslot = 0;
    for (int it = 0; it < nact; it++) {
      const int t = cur & 0xffff;
      const int kv0 = t * BN;
      const int buf = it & 1;
      if (it + 1 < nact) load_tile(nxt & 0xffff, it);
      const int after = entry(it + 2);  // read now, taken over at the end of the tile
      const int kprev = kslot == 0 ? 2 : kslot - 1, knext = kslot == 2 ? 0 : kslot + 1;
      const unsigned char* kl = smem + buf * KV_BYTES;
      const unsigned char* vl = kl + K_BYTES;
      const unsigned char* ktl = smem + KTR_AT + kslot * KTR_BYTES;
      const unsigned char* ktp = smem + KTR_AT + kprev * KTR_BYTES;
      const int* sl = (const int*)(smem + SEG_AT + buf * BN * 4);

      bool skip = CAUSAL && kv0 > wq_last;
      bool need_mask = (kv0 + BN > Skv) || (CAUSAL && kv0 + BN - 1 > wq0);
      if (SEG) {
        const unsigned my = ((unsigned)cur >> (16 + 2 * wave_s)) & 3u;
        skip = skip || (my & 1u);
        need_mask = need_mask || (my & 2u);
      }
      if (ext) {
        skip = skip || kv0 > wpmax + a.mx.hi_off || kv0 + BN - 1 < wpmin - a.mx.lo_off;
        need_mask = need_mask || capped || biased || !(kv0 >= wpmax - a.mx.lo_off && kv0 + BN - 1 <= wpmin + a.mx.hi_off);
      }
      if (need_mask && !skip) make_key_bits(kv0, sl);
      auto body = [&](auto masked_c) {
        constexpr bool MASKED = decltype(masked_c)::value;
        v8 fr[NF];
        v8 df0[2], df1[2];
        auto frag = [&](auto I) -> v8 {
          constexpr int i = decltype(I)::value;
          if constexpr (i < P1) return *(const v8*)(kl + KT::off(ln, 16 * i + 8 * g));
          else if constexpr (i < P2) {
            constexpr int j = i - P1, hh = j / DKB, d = j % DKB;
            return *(const v8*)(ktp + ta[(2 + hh) ^ (d & 3)] + d * 32 * TrTile64::ROW_BYTES);
          } else if constexpr (i < P3) return *(const v8*)(vl + VT::off(ln, 16 * (i - P2) + 8 * g));
          else if constexpr (i < P4) return *(const v8*)(kl + KT::off(32 + ln, 16 * (i - P3) + 8 * g));
          else if constexpr (i < P5) {
            constexpr int j = i - P4, hh = j / DKB, d = j % DKB;
            return *(const v8*)(ktl + ta[hh ^ (d & 3)] + d * 32 * TrTile64::ROW_BYTES);
          } else return *(const v8*)(vl + VT::off(32 + ln, 16 * (i - P5) + 8 * g));
        };
        auto mma = [&](auto I, const v8& f) {
          constexpr int i = decltype(I)::value;
          const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          if constexpr (i < P1) s[0] = MT<T>::mfma32(f, qf[i], i == 0 ? zero : s[0]);
          else if constexpr (i < P2) dqacc[(i - P1) % DKB] = MT<T>::mfma32(f, df1[(i - P1) / DKB], dqacc[(i - P1) % DKB]);
          else if constexpr (i < P3) dp[0] = MT<T>::mfma32(f, dof[i - P2], i == P2 ? zero : dp[0]);
          else if constexpr (i < P4) s[1] = MT<T>::mfma32(f, qf[i - P3], i == P3 ? zero : s[1]);
          else if constexpr (i < P5) dqacc[(i - P4) % DKB] = MT<T>::mfma32(f, df0[(i - P4) / DKB], dqacc[(i - P4) % DKB]);
          else dp[1] = MT<T>::mfma32(f, dof[i - P5], i == P5 ? zero : dp[1]);
        };
        // piece K of LEN of a 16-element group
        auto ds_piece = [&](auto I, auto STARTc, const f32x16& p, f32x16& d, v8* dfb) {
          constexpr int i = decltype(I)::value, st = decltype(STARTc)::value, len = KS_QK;
          if constexpr (i >= st && i < st + len) {
            constexpr int k = i - st, lo = (k * 16 + len - 1) / len, hi = ((k + 1) * 16 + len - 1) / len;
            ds_chunk(std::integral_constant<int, lo>{}, std::integral_constant<int, hi>{}, p, d, dfb);
          }
        };
        auto p_piece = [&](auto I, auto STARTc, auto NBc, f32x16& sv) {
          constexpr int i = decltype(I)::value, st = decltype(STARTc)::value, nb = decltype(NBc)::value, len = LEN_P;
          if constexpr (i >= st && i < st + len) {
            constexpr int k = i - st, lo = (k * 16 + len - 1) / len, hi = ((k + 1) * 16 + len - 1) / len;
#pragma unroll
            for (int v = lo; v < hi; v++) {
              float sval = sv[v], dcap = 1.f;
              if (GEN && MASKED) {
                if (capped) {
                  const float th = fast_tanh(sval * a.mx.cap_in);
                  dcap = 1.f - th * th;  // derivative of the capped score; P only feeds dS here, so it rides on P
                  sval = a.mx.cap_out * th;
                }
                // additive mask, in units of the raw score (-inf stays -inf)
                if (biased) sval += a.mx.bias_mul * bias_row[min(kv0 + nb * 32 + 8 * (v / 4) + 4 * g + (v % 4), Skv - 1)];
              }
              float pv = fast_exp2(__builtin_fmaf(sval, c, -lse_s));
              if (MASKED) {
                if (GEN) pv *= dcap;
                pv = __builtin_bit_cast(float, __builtin_bit_cast(int, pv) & __builtin_amdgcn_sbfe((int)kbits[nb], 8 * (v / 4) + (v % 4), 1));
              }
              asm volatile("" : "+v"(pv));
              sv[v] = pv;
            }
          }
        };
        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, 1> I1;
        static_for<0, AHEAD>([&](auto I) { fr[decltype(I)::value % NF] = frag(I); });
        static_for<0, NS>([&](auto I) {
          constexpr int i = decltype(I)::value;
          if constexpr (i + AHEAD < NS) fr[(i + AHEAD) % NF] = frag(std::integral_constant<int, i + AHEAD>{});
          mma(I, fr[i % NF]);
          ds_piece(I, std::integral_constant<int, 1>{}, s[1], dp[1], df1);
          p_piece(I, std::integral_constant<int, P1 + 1>{}, I0{}, s[0]);
          ds_piece(I, std::integral_constant<int, P3 + 1>{}, s[0], dp[0], df0);
          p_piece(I, std::integral_constant<int, P4 + 1>{}, I1{}, s[1]);
          // the next tile (requested at the top of this one) goes to LDS under the last MFMAs; after the last
          // tile this stores stale registers nobody reads
          constexpr int ST0 = NS - 12;
          if constexpr (i == ST0) kst.store_rowmajor(smem + (buf ^ 1) * KV_BYTES + (wave < 4 ? 0 : K_BYTES), stid);
          if constexpr (i >= ST0 + 2 && i < ST0 + 10) {
            if (wave < 4) kst.template store_transposed_step<i - ST0 - 2>(smem + KTR_AT + knext * KTR_BYTES, stid);
          }
          __builtin_amdgcn_sched_barrier(0);
        });
      };
      if (!skip) {
        if (need_mask) body(std::true_type{});
        else body(std::false_type{});
        pending = true;
        if (SEG && tid < BN) ((int*)(smem + SEG_AT + (buf ^ 1) * BN * 4))[tid] = sreg;
      } else {
        if (pending) { drain(ktp); pending = false; }
        if (it + 1 < nact) store_tile(buf ^ 1, knext, it);
      }
      __syncthreads();
      kslot = knext;
      cur = nxt;
      nxt = __builtin_amdgcn_readfirstlane(after);
    }
    if (pending) drain(smem + KTR_AT + (kslot == 0 ? 2 : kslot - 1) * KTR_BYTES);
  } else {
  for (int it = 0; it < nact; it++) {
      const int t = cur & 0xffff;
      const int kv0 = t * BN;
      const int buf = it & 1;
      if (it + 1 < nact) load_tile(nxt & 0xffff, it);
      const int after = entry(it + 2);  // read now, taken over at the end of the tile
  
      const unsigned char* kl = smem + buf * KV_BYTES;
      const unsigned char* vl = kl + K_BYTES;
      const unsigned char* ktl = smem + KTR_AT + buf * KTR_BYTES;
      const int* sl = (const int*)(smem + SEG_AT + buf * BN * 4);
  
      bool skip = CAUSAL && kv0 > wq_last;
      bool need_mask = (kv0 + BN > Skv) || (CAUSAL && kv0 + BN - 1 > wq0);
      if (SEG) {
        const unsigned my = ((unsigned)cur >> (16 + 2 * wave_s)) & 3u;
        skip = skip || (my & 1u);
        need_mask = need_mask || (my & 2u);
      }
      if (ext) {
        skip = skip || kv0 > wpmax + a.mx.hi_off || kv0 + BN - 1 < wpmin - a.mx.lo_off;
        need_mask = need_mask || capped || biased || !(kv0 >= wpmax - a.mx.lo_off && kv0 + BN - 1 <= wpmin + a.mx.hi_off);
      }
      // The tile body is laid out slot by slot (one MFMA each, a scheduling barrier after every slot): the
      // LDS fragment of a slot is requested AHEAD slots earlier, and the element-wise work that turns
      // S^T, dP^T into the 16-bit operand dS^T is spread under the MFMAs of the following slots.
      //   slots   S0^T = K0 Q^T alternating with dP0^T = V0 dO^T;  S1^T with dP1^T;
      //           dQ^T += K0^T dS0^T;  dQ^T += K1^T dS1^T (first the half whose operand is ready first)
      //   VALU    dS0^T under S1^T/dP1^T; dS1^T under the dQ^T slots that do not need it yet
      if (need_mask && !skip) make_key_bits(kv0, sl);
      auto body = [&](auto masked_c) {
        constexpr bool MASKED = decltype(masked_c)::value;
        // 4 waves: S/dP of both kv blocks first, so that dS of block 0 has the MFMAs of block 1 next to it.
        // 8 waves: block by block (S/dP, dS, dQ), which keeps one pair of 32x32 tiles live; the other wave on
        // the SIMD supplies the overlap.
        constexpr bool STAG = NW == 4;
        constexpr int L1 = KS_QK + KS_DV, A2 = 2 * DKB, NS = 2 * L1 + 2 * A2;
        constexpr int AB1 = STAG ? L1 : L1 + A2;          // first slot of S1/dP1
        constexpr int ACC0 = STAG ? 2 * L1 : L1;          // first slot of dQ += K0^T dS0
        constexpr int ACC1 = 2 * L1 + A2;                 // first slot of dQ += K1^T dS1
        constexpr int AHEAD = 3, NF = 4;
        v8 fr[NF];
        f32x16 s[2], dp[2];
        v8 df[2][2];
        auto frag = [&](auto I) -> v8 {
          constexpr int i = decltype(I)::value;
          constexpr bool is_acc = (i >= ACC0 && i < ACC0 + A2) || i >= ACC1;
          if constexpr (!is_acc) {
            constexpr int nb = i >= AB1 ? 1 : 0;
            constexpr AbSlot sl = ab_slot(nb ? i - AB1 : i, KS_QK, KS_DV);
            if constexpr (sl.kind == 0) return *(const v8*)(kl + KT::off(nb * 32 + ln, 16 * sl.k + 8 * g));
            else return *(const v8*)(vl + VT::off(nb * 32 + ln, 16 * sl.k + 8 * g));
          } else {
            constexpr int nb = i >= ACC1 ? 1 : 0, j = nb ? i - ACC1 : i - ACC0, hh = j / DKB, d = j % DKB;
            return *(const v8*)(ktl + ta[(2 * nb + hh) ^ (d & 3)] + d * 32 * TrTile64::ROW_BYTES);
          }
        };
        auto mma = [&](auto I, const v8& f) {
          constexpr int i = decltype(I)::value;
          constexpr bool is_acc = (i >= ACC0 && i < ACC0 + A2) || i >= ACC1;
          const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          if constexpr (!is_acc) {
            constexpr int nb = i >= AB1 ? 1 : 0;
            constexpr AbSlot sl = ab_slot(nb ? i - AB1 : i, KS_QK, KS_DV);
            if constexpr (sl.kind == 0) s[nb] = MT<T>::mfma32(f, qf[sl.k], sl.k == 0 ? zero : s[nb]);
            else dp[nb] = MT<T>::mfma32(f, dof[sl.k], sl.k == 0 ? zero : dp[nb]);
          } else {
            constexpr int nb = i >= ACC1 ? 1 : 0, j = nb ? i - ACC1 : i - ACC0, hh = j / DKB, d = j % DKB;
            if constexpr (ACC_PINNED) MT<T>::mfma32_acc_guarded(dqacc[d], f, df[nb][hh]);
            else dqacc[d] = MT<T>::mfma32(f, df[nb][hh], dqacc[d]);
          }
        };
        // elements [E0, E0 + N) of block NB spread evenly over the LEN slots starting at START
        auto valu = [&](auto I, auto NBc, auto E0c, auto Nc, auto STARTc, auto LENc) {
          constexpr int i = decltype(I)::value, nb = decltype(NBc)::value, e0 = decltype(E0c)::value, n = decltype(Nc)::value,
                        st = decltype(STARTc)::value, len = decltype(LENc)::value;
          if constexpr (i >= st && i < st + len) {
            constexpr int k = i - st, lo = e0 + (k * n + len - 1) / len, hi = e0 + ((k + 1) * n + len - 1) / len;
  #pragma unroll
            for (int v = lo; v < hi; v++) {
              float sval = s[nb][v], dcap = 1.f;
              if (GEN && MASKED) {
                if (capped) {
                  const float th = fast_tanh(sval * a.mx.cap_in);
                  dcap = 1.f - th * th;
                  sval = a.mx.cap_out * th;
                }
                if (biased) sval += a.mx.bias_mul * bias_row[min(kv0 + nb * 32 + 8 * (v / 4) + 4 * g + (v % 4), Skv - 1)];
              }
              float pv = fast_exp2(__builtin_fmaf(sval, c, -lse_s));
              if (MASKED) {
                if (GEN) pv *= dcap;
                pv = __builtin_bit_cast(float, __builtin_bit_cast(int, pv) & __builtin_amdgcn_sbfe((int)kbits[nb], 8 * (v / 4) + (v % 4), 1));
              }
              float dsv = pv * (dp[nb][v] + ndelta_s);
              asm volatile("" : "+v"(dsv));  // keeps the computation in this slot
              dp[nb][v] = dsv;
            }
            static_for<0, 2>([&](auto H) {  // every half whose eighth value was produced in this slot
              constexpr int hh = decltype(H)::value;
              if constexpr (8 * hh + 8 > lo && 8 * hh + 8 <= hi) {
                const f32x16& x = dp[nb];
                df[nb][hh] = pack8<T>(x[8 * hh + 0], x[8 * hh + 1], x[8 * hh + 2], x[8 * hh + 3], x[8 * hh + 4],
                                      x[8 * hh + 5], x[8 * hh + 6], x[8 * hh + 7]);
              }
            });
          }
        };
        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, 1> I1;
        typedef std::integral_constant<int, 8> I8;
        typedef std::integral_constant<int, 16> I16;
        static_for<0, AHEAD>([&](auto I) { fr[decltype(I)::value % NF] = frag(I); });
        static_for<0, NS>([&](auto I) {
          constexpr int i = decltype(I)::value;
          if constexpr (i + AHEAD < NS) fr[(i + AHEAD) % NF] = frag(std::integral_constant<int, i + AHEAD>{});
          if constexpr (!STAG) {
            // whole dS of a block right before the dQ slots that consume it
            valu(I, I0{}, I0{}, I16{}, std::integral_constant<int, ACC0>{}, I1{});
            valu(I, I1{}, I0{}, I16{}, std::integral_constant<int, ACC1>{}, I1{});
          }
          mma(I, fr[i % NF]);
          if constexpr (!STAG) {
            // the next tile (requested at the top of this one) goes to the other buffer under the last MFMAs
            // instead of in a phase of its own; after the last tile this stores stale registers nobody reads
            constexpr int ST0 = NS - 12;
            unsigned char* nb_base = smem + (buf ^ 1) * KV_BYTES;
            if constexpr (i == ST0) kst.store_rowmajor(nb_base + (wave < 4 ? 0 : K_BYTES), stid);
            if constexpr (i >= ST0 + 2 && i < ST0 + 10) {
              if (wave < 4) kst.template store_transposed_step<i - ST0 - 2>(smem + KTR_AT + (buf ^ 1) * KTR_BYTES, stid);
            }
          }
          if constexpr (STAG) {
            valu(I, I0{}, I0{}, I16{}, std::integral_constant<int, L1>{}, std::integral_constant<int, L1>{});
            valu(I, I1{}, I0{}, I8{}, std::integral_constant<int, ACC0>{}, std::integral_constant<int, 2 * DKB>{});
            valu(I, I1{}, I8{}, I8{}, std::integral_constant<int, ACC1>{}, std::integral_constant<int, DKB>{});
          }
          __builtin_amdgcn_sched_barrier(0);
        });
      };
      if (!skip) {
        if (need_mask) body(std::true_type{});
        else body(std::false_type{});
      }
      if (NW == 4 || skip) {
        if (it + 1 < nact) store_tile(buf ^ 1, buf ^ 1, it);
      } else if (SEG && tid < BN) {
        ((int*)(smem + SEG_AT + (buf ^ 1) * BN * 4))[tid] = sreg;
      }
      __syncthreads();
      cur = nxt;
      nxt = __builtin_amdgcn_readfirstlane(after);
    }
  
  }

  // (pinned accumulators come out of asm MFMAs: the compiler inserts no wait states before reading them)
  if constexpr (ACC_PINNED) asm volatile("s_nop 15\n\ts_nop 3" ::: "memory");
  if (qrow < Sq) {
    T* dqp = (T*)a.dq + b * a.dqs[0] + h * a.dqs[1] + qrow * a.dqs[2];
    const float sc = a.sm_scale;
#pragma unroll
    for (int d = 0; d < DKB; d++)
#pragma unroll
      for (int vq = 0; vq < 4; vq++) {
        const f32x16& o = dqacc[d];
        *(u32x2*)(dqp + d * 32 + 8 * vq + 4 * g) =
            pack4<T>(o[4 * vq] * sc, o[4 * vq + 1] * sc, o[4 * vq + 2] * sc, o[4 * vq + 3] * sc);
      }
  }
}

// ------------------------------------------------------------------------------------------------
// dQ, the plain kernels (no segment ids, no mask extensions; equal head dims up to 128)
// ------------------------------------------------------------------------------------------------
// Shaped like the forward: workgroup = 4 waves = 128 query rows of one (batch, head), two workgroups per CU (so two
// waves per SIMD whose barriers are independent of each other); Q and dO fragments, LSE and delta stay in registers;
// K and V tiles of 64 rows travel into LDS by loads that write LDS themselves (two buffers, one barrier per tile, no
// staging registers, no second copy of K: the K^T operand of dQ^T += K^T dS^T comes out of transposing reads).
// S^T = K Q^T and dP^T = V dO^T are computed transposed, so LSE and delta are per-lane scalars and dS^T, converted to
// 16 bit, is the B operand of the accumulating product as it stands.  -delta joins dP through the matrix unit (one
// more k-step per block: a column of ones on the V side, the lane's -delta split into two 16-bit values on the dO
// side) instead of 32 additions per lane and tile: the kernels are bound by the instructions a SIMD can issue.
// Per tile and 32-row half h of it:  S_h (KS MFMAs) | dP_h (KS + 1) | ... | dQ += K_h^T dS_h (2 DB), with P_h computed
// under dP_h and dS_h under what follows.
// With segment ids (SEG) the kernel visits the kv tiles whose id range meets the workgroup's, a list built once per
// workgroup; a wave skips the tiles that miss its own 32 rows, and masked tiles take the rows of the lane's id from
// a ballot over the tile's id vector, which wave 0 fetches with the tile (one more LDS-writing load).
// Unequal head dims (192, 128): the same kernel with one workgroup per CU (its fragments and accumulators need more
// than half a SIMD's registers) and the dQ accumulators pinned to the accumulation registers.
template <typename T, int DQK, int DV, bool CAUSAL, bool SEG>
__global__ __launch_bounds__(256, DQK == DV ? 2 : 1) void attn_bwd_dq_plain_kernel(const BwdArgs a) {
  typedef typename MT<T>::v8 v8;
  constexpr bool WIDE = DQK != DV;
  constexpr int BN = 64, BM = 128, KS = DQK / 16, KSV = DV / 16, DB = DQK / 32;
  typedef DmaTile<DQK, true> KT;
  typedef DmaTile<DV, true> VT;
  constexpr int K_BYTES = KT::BYTES, V_BYTES = VT::BYTES, K_AT = 0, V_AT = 2 * K_BYTES;
  constexpr int SEG_AT = 2 * (K_BYTES + V_BYTES), CTL_AT = SEG_AT + 2 * BN * 4;  // two id vectors; 16 bytes per visited tile
  constexpr int NLOAD_K = KT::PER_WAVE, NLOAD_V = VT::PER_WAVE, NLOAD2 = NLOAD_K + NLOAD_V;  // loads per wave and tile

  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, ln = lane & 31;
  const int n_qt = (a.Sq + BM - 1) / BM;
  int tile, inner, group;
  if (!xcd_map(n_qt, a.n_rep, a.B * a.Hkv, tile, inner, group)) return;
  const int qt = n_qt - 1 - tile;  // the longest rows first
  const int b = group / a.Hkv, hk = group - b * a.Hkv, h = hk * a.n_rep + inner;
  const int q0 = qt * BM, wq0 = q0 + wave * 32;
  const int Sq = a.Sq, Skv = a.Skv;
  const int band_lo = CAUSAL ? a.band_lo : BAND_INF, band_hi = CAUSAL ? a.band_hi : BAND_INF;
  const int kv_end = CAUSAL ? max(min(Skv, q0 + BM + band_hi), 0) : Skv;
  const int ntiles = (kv_end + BN - 1) / BN;
  const int t_first = CAUSAL ? min(max(q0 - band_lo, 0) / BN, ntiles) : 0;  // (tiles before it lie left of every row's band)

  // ---- Q, dO fragments (B operands: lane = query column), per-lane LSE / -delta
  const int qrow = wq0 + ln, qrow_c = min(qrow, Sq - 1);
  const int wq0_s = __builtin_amdgcn_readfirstlane(wq0);  // (for the masked tiles, which form the row again)
  v8 qf[KS], dof[KSV];
  {
    const T* qp = (const T*)a.q + b * a.qs[0] + h * a.qs[1] + qrow_c * a.qs[2] + 8 * g;
    const T* dp = (const T*)a.dout + b * a.dos[0] + h * a.dos[1] + qrow_c * a.dos[2] + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *(const v8*)(qp + 16 * ks);
#pragma unroll
    for (int ks = 0; ks < KSV; ks++) dof[ks] = *(const v8*)(dp + 16 * ks);
  }
  const int64_t ro = ((int64_t)b * a.Hq + h) * Sq + qrow_c;
  const float lraw = a.lse[ro];
  const float nlse = (lraw == -INFINITY) ? -INFINITY : -lraw * LOG2E;  // (a row without keys: P = exp2(-inf) = 0)
  // -delta = -rowsum(dO o O) of this lane's row, computed here from the dO fragments and the matching pieces of O
  // (the two lanes that share a row hold the two halves of the head dim), and left in the workspace together with
  // -LSE in log2 units for the dK/dV kernel, which runs after this one: no separate pass over dO and O
  float ndelta;
  {
    const T* op = (const T*)a.out + b * a.os[0] + h * a.os[1] + qrow_c * a.os[2] + 8 * g;
    float acc = 0.f;
#pragma unroll
    for (int ks = 0; ks < KSV; ks++) {
      const v8 of = *(const v8*)(op + 16 * ks);
#pragma unroll
      for (int e = 0; e < 8; e++) acc = __builtin_fmaf((float)of[e], (float)dof[ks][e], acc);
    }
    acc += __shfl_xor(acc, 32, 64);
    ndelta = -acc;
    if (g == 0 && qrow < Sq) {
      a.delta[ro] = ndelta;
      a.delta[(int64_t)a.B * a.Hq * Sq + ro] = nlse;
    }
  }
  v8 ones_a, ndelta_b;
  {
    const float hi = (float)(T)ndelta, lo = ndelta - hi;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      ones_a[e] = (T)((g == 0 && e < 2) ? 1.0f : 0.0f);
      ndelta_b[e] = (T)0.0f;
    }
    if (g == 0) { ndelta_b[0] = (T)hi; ndelta_b[1] = (T)lo; }
    asm volatile("" : "+v"(ones_a), "+v"(ndelta_b));
  }

  // ---- segment ids: the list of kv tiles to visit (tile, min id, max id), this wave's own id range
  const int32_t* segb = SEG ? a.seg + (int64_t)b * Skv : nullptr;
  const int segq = SEG ? segb[qrow_c] : 0;
  const int* ctl = (const int*)(smem + CTL_AT);
  int nact = ntiles - t_first, wqmin = 0, wqmax = 0;
  if (SEG) {
    wqmin = segq; wqmax = segq;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) {
      wqmin = min(wqmin, __shfl_xor(wqmin, o, 64));
      wqmax = max(wqmax, __shfl_xor(wqmax, o, 64));
    }
    wqmin = __builtin_amdgcn_readfirstlane(wqmin);
    wqmax = __builtin_amdgcn_readfirstlane(wqmax);
    // the tiles' id ranges are only needed until the list is built: they borrow the tile buffers
    int* kvmin = (int*)smem;
    int* kvmax = kvmin + ntiles;
    int* bq = kvmax + ntiles;
    if (lane == 0) { bq[2 * wave] = wqmin; bq[2 * wave + 1] = wqmax; }
    seg_tile_ranges(segb, Skv, 0, ntiles, kvmin, kvmax, tid, 256);
    __syncthreads();
    const int bmin = min(min(bq[0], bq[2]), min(bq[4], bq[6])), bmax = max(max(bq[1], bq[3]), max(bq[5], bq[7]));
    int cnt = 0;
    for (int base = 0; base < ntiles; base += 64) {
      const int t = base + lane;
      const int lo = t < ntiles ? kvmin[t] : 0, hi = t < ntiles ? kvmax[t] : 0;
      const bool act = t >= t_first && t < ntiles && !(hi < bmin || lo > bmax);
      const unsigned long long m = __ballot(act);
      if (act && wave == 0) *(i32x4*)(smem + CTL_AT + 16 * (cnt + __popcll(m & ((1ull << lane) - 1ull)))) = i32x4{t, lo, hi, 0};
      cnt += __popcll(m);
    }
    nact = cnt;
    __syncthreads();  // the list is complete and the ranges are no longer read: the first tile may land on them
  }
  auto entry = [&](int it) -> i32x4 {
    if (SEG) return *(const i32x4*)(ctl + 4 * max(min(it, nact - 1), 0));
    return i32x4{min(t_first + it, ntiles - 1), 0, 0, 0};
  };

  // ---- loads
  const unsigned k_tile_bytes = (unsigned)(BN * a.ks[2] * 2), v_tile_bytes = (unsigned)(BN * a.vs[2] * 2);
  KT kdma;
  VT vdma;
  kdma.init(a.ks[2], wave, lane);
  vdma.init(a.vs[2], wave, lane);
  const u32x4 srw = make_rsrc_words(SEG ? (const void*)segb : (const void*)a.k, SEG ? (unsigned)Skv * 4u : 0u);
  const u32x4 krw = make_rsrc_words((const T*)a.k + b * a.ks[0] + hk * a.ks[1], span_bytes(Skv, a.ks[2], DQK));
  const u32x4 vrw = make_rsrc_words((const T*)a.v + b * a.vs[0] + hk * a.vs[1], span_bytes(Skv, a.vs[2], DV));
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const unsigned lds_base = __builtin_amdgcn_readfirstlane((unsigned)(size_t)smem);
  const unsigned kdst0 = lds_base + (unsigned)K_AT + (unsigned)(wave_s * NLOAD_K * 1024);
  const unsigned vdst0 = lds_base + (unsigned)V_AT + (unsigned)(wave_s * NLOAD_V * 1024);
  auto load_piece = [&](auto Pc, int t, int buf) {
    constexpr int p = decltype(Pc)::value;
    if constexpr (p < NLOAD_K)
      kdma.template issue_one_at<p>(krw, __builtin_amdgcn_readfirstlane((unsigned)t * k_tile_bytes), kdst0 + (unsigned)(buf * K_BYTES));
    else
      vdma.template issue_one_at<p - NLOAD_K>(vrw, __builtin_amdgcn_readfirstlane((unsigned)t * v_tile_bytes), vdst0 + (unsigned)(buf * V_BYTES));
    // the tile's id vector rides with the first piece (rows past the end arrive as zeros and are masked by position)
    if constexpr (SEG && p == 0) {
      if (wave == 0) dma_dword_at(srw, __builtin_amdgcn_readfirstlane((unsigned)(t * BN) * 4u), lds_base + (unsigned)(SEG_AT + buf * BN * 4), lane);
    }
  };

  // ---- per-lane LDS addresses in buffer 0 (opaque registers; reads add immediates)
  const unsigned lds0 = (unsigned)(size_t)smem;
  constexpr bool SWZ3 = KT::CPR % 16 != 0, VSWZ3 = VT::CPR % 16 != 0;
  constexpr int NFO = SWZ3 ? (KS < 4 ? KS : 4) : KS, NVO = WIDE ? (VSWZ3 ? (KSV < 4 ? KSV : 4) : KSV) : 1;
  unsigned kfo[NFO], vfo[NVO], ktr[DB][2];
#pragma unroll
  for (int j = 0; j < NFO; j++) {
    kfo[j] = lds0 + (unsigned)(ln * KT::ROWB + (((2 * j + g) ^ KT::swz(ln)) << 4));  // K (equal head dims: V lies V_AT further on)
    asm volatile("" : "+v"(kfo[j]));
  }
#pragma unroll
  for (int j = 0; j < NVO; j++) {
    vfo[j] = lds0 + (unsigned)V_AT + (unsigned)(ln * VT::ROWB + (((2 * j + g) ^ VT::swz(ln)) << 4));
    asm volatile("" : "+v"(vfo[j]));
  }
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++) {
      ktr[d][h2] = lds0 + (unsigned)KT::tr_off(8 * h2 + 4 * g, 2 * d + ((lane >> 4) & 1), lane & 15);
      asm volatile("" : "+v"(ktr[d][h2]));
    }
  auto ld16 = [](unsigned addr) { return *(const __attribute__((address_space(3))) v8*)addr; };
  auto ldtr = [](unsigned a0, unsigned a1) { return tr_read8<v8>((const lds_byte*)a0, (const lds_byte*)a1); };

  f32x16 dqacc[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int v = 0; v < 16; v++) dqacc[d][v] = 0.f;
  const float c = a.scale_log2;
  const int wq_last = wq0 + 31;

  // slots of a tile: S0 | dP0 | S1 | dP1 | dQ0 | dQ1
  constexpr int KSD = KSV + 1, A2 = 2 * DB;
  constexpr int P_S0 = 0, P_D0 = KS, P_S1 = P_D0 + KSD, P_D1 = P_S1 + KS, P_Q0 = P_D1 + KSD, P_Q1 = P_Q0 + A2, NS = P_Q1 + A2;
  constexpr int AHEAD = 4, NF = AHEAD + 1;

  auto tile_body = [&](auto masked_c, auto BUFc, int t, int t_next) {
    constexpr bool MASKED = decltype(masked_c)::value;
    constexpr int buf = decltype(BUFc)::value;
    constexpr unsigned kl = K_AT + buf * K_BYTES, vl = V_AT + buf * V_BYTES, vlw = buf * V_BYTES;  // (vlw: on top of vfo[])
    const int kv0 = t * BN;
    // masked tiles: which of the tile's 64 kv rows this lane's query row may see, as bits (value v of a half: bit
    // 8 (v / 4) + v % 4 after the shift by 4 g)
    unsigned kbits[2] = {0u, 0u};
    if (MASKED) {
      // (what only a masked tile needs is formed here from an opaque copy of lane * 4, which the loads of the
      // segment ids keep in a register anyway: the query row, the band offsets added to it and the address of the
      // lane's segment id, held across the loop as registers of their own, were spilled in the variant with
      // segment ids, and a reload waits behind the tile loads in flight)
      unsigned l4 = (unsigned)lane * 4u;
      asm volatile("" : "+v"(l4));
      const int qrow_m = wq0_s + (int)((l4 >> 2) & 31u);
      int hi = min(Skv - kv0, BN), lo = 0;
      if (CAUSAL) {
        int bh = band_hi - kv0 + 1, bl = band_lo + kv0;
        asm volatile("" : "+s"(bh), "+s"(bl));
        hi = min(hi, qrow_m + bh);
        lo = max(qrow_m - bl, 0);
      }
      if (qrow_m >= Sq) hi = 0;
      unsigned long long m = hi > lo ? ((~0ull << lo) & (~0ull >> (64 - hi))) : 0ull;
      if (SEG) {
        const int rowseg = *(const int*)(smem + SEG_AT + buf * BN * 4 + l4);  // lane l: id of the tile's kv row l
        unsigned long long ms = 0ull, todo = ~0ull;
        while (todo) {
          const int x = __builtin_amdgcn_readlane(segq, (int)__builtin_ctzll(todo));
          const unsigned long long rows = __ballot(rowseg == x);
          const bool mine = segq == x;
          ms = mine ? rows : ms;
          todo &= ~__ballot(mine);
        }
        m &= ms;
      }
      kbits[0] = (unsigned)m >> (4 * g);
      kbits[1] = (unsigned)(m >> 32) >> (4 * g);
    }
    v8 fr[NF];
    f32x16 s[2], dp[2];
    v8 df[2][2];
    auto has_frag = [](int i) constexpr { return i != P_D0 && i != P_D1; };
    auto frag = [&](auto I) -> v8 {
      constexpr int i = decltype(I)::value;
      auto rowfrag = [&](unsigned base, int hf, int ks) {
        return ld16(kfo[SWZ3 ? (ks & 3) : ks] + (base + (unsigned)(hf * 32 * KT::ROWB + (SWZ3 ? 128 * (ks >> 2) : 0))));
      };
      auto vfrag = [&](int hf, int ks) {
        if constexpr (WIDE) return ld16(vfo[VSWZ3 ? (ks & 3) : ks] + (vlw + (unsigned)(hf * 32 * VT::ROWB + (VSWZ3 ? 128 * (ks >> 2) : 0))));
        else return rowfrag(vl, hf, ks);
      };
      if constexpr (i < P_D0) return rowfrag(kl, 0, i - P_S0);
      else if constexpr (i < P_S1) return vfrag(0, i - P_D0 - 1);
      else if constexpr (i < P_D1) return rowfrag(kl, 1, i - P_S1);
      else if constexpr (i < P_Q0) return vfrag(1, i - P_D1 - 1);
      else {
        // K^T block d, contraction over kv rows 32 hf + 16 kk + {4g..4g+3, 8+4g..8+4g+3}: the order in which dS holds them
        constexpr int hf = i >= P_Q1 ? 1 : 0, j = i - (hf ? P_Q1 : P_Q0), kk = j / DB, d = j % DB;
        constexpr unsigned rows = (unsigned)((32 * hf + 16 * kk) * KT::ROWB);
        return ldtr(ktr[d][0] + (kl + rows), ktr[d][1] + (kl + rows));
      }
    };
    auto mma = [&](auto I, const v8& f) {
      constexpr int i = decltype(I)::value;
      const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if constexpr (i < P_D0) s[0] = MT<T>::mfma32(f, qf[i], i == 0 ? zero : s[0]);
      else if constexpr (i == P_D0) dp[0] = MT<T>::mfma32(ones_a, ndelta_b, zero);
      else if constexpr (i < P_S1) dp[0] = MT<T>::mfma32(f, dof[i - P_D0 - 1], dp[0]);
      else if constexpr (i < P_D1) s[1] = MT<T>::mfma32(f, qf[i - P_S1], i == P_S1 ? zero : s[1]);
      else if constexpr (i == P_D1) dp[1] = MT<T>::mfma32(ones_a, ndelta_b, zero);
      else if constexpr (i < P_Q0) dp[1] = MT<T>::mfma32(f, dof[i - P_D1 - 1], dp[1]);
      else {
        constexpr int hf = i >= P_Q1 ? 1 : 0, j = i - (hf ? P_Q1 : P_Q0), kk = j / DB, d = j % DB;
        if constexpr (WIDE) MT<T>::mfma32_acc(dqacc[d], f, df[hf][kk]);
        else dqacc[d] = MT<T>::mfma32(f, df[hf][kk], dqacc[d]);
      }
    };
    // elements [k 16 / LEN, (k + 1) 16 / LEN) of half HF in slot START + k: P = exp2(s c - lse) (masked) ...
    auto p_piece = [&](auto I, auto HFc, auto STARTc, auto LENc) {
      constexpr int i = decltype(I)::value, hf = decltype(HFc)::value, st = decltype(STARTc)::value, len = decltype(LENc)::value;
      if constexpr (i >= st && i < st + len) {
        constexpr int k = i - st, lo = (k * 16 + len - 1) / len, hi = ((k + 1) * 16 + len - 1) / len;
#pragma unroll
        for (int v = lo; v < hi; v++) {
          float pv = fast_exp2(__builtin_fmaf(s[hf][v], c, nlse));
          if (MASKED) pv = __builtin_bit_cast(float, __builtin_bit_cast(int, pv) & __builtin_amdgcn_sbfe((int)kbits[hf], 8 * (v / 4) + (v % 4), 1));
          asm volatile("" : "+v"(pv));  // keeps the computation in this slot
          s[hf][v] = pv;
        }
      }
    };
    // ... and dS = P o (dP - delta), packed as soon as the eight values of an operand are there
    auto ds_piece = [&](auto I, auto HFc, auto STARTc, auto LENc) {
      constexpr int i = decltype(I)::value, hf = decltype(HFc)::value, st = decltype(STARTc)::value, len = decltype(LENc)::value;
      if constexpr (i >= st && i < st + len) {
        constexpr int k = i - st, lo = (k * 16 + len - 1) / len, hi = ((k + 1) * 16 + len - 1) / len;
#pragma unroll
        for (int v = lo; v < hi; v++) {
          float dsv = s[hf][v] * dp[hf][v];
          asm volatile("" : "+v"(dsv));
          dp[hf][v] = dsv;
        }
        static_for<0, 2>([&](auto H) {
          constexpr int hh = decltype(H)::value;
          if constexpr (8 * hh + 8 > lo && 8 * hh + 8 <= hi) {
            const f32x16& x = dp[hf];
            df[hf][hh] = pack8<T>(x[8 * hh + 0], x[8 * hh + 1], x[8 * hh + 2], x[8 * hh + 3], x[8 * hh + 4], x[8 * hh + 5],
                                  x[8 * hh + 6], x[8 * hh + 7]);
          }
        });
      }
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;
    static_for<0, AHEAD>([&](auto I) { fr[decltype(I)::value % NF] = frag(I); });
    static_for<0, NS>([&](auto I) {
      constexpr int i = decltype(I)::value;
      if constexpr (i + AHEAD < NS && has_frag(i + AHEAD)) fr[(i + AHEAD) % NF] = frag(std::integral_constant<int, i + AHEAD>{});
      mma(I, fr[i % NF]);
      // the next tile's loads, one per slot (past the last tile they re-read the last one: no branch here)
      if constexpr (i < NLOAD2) load_piece(I, t_next, buf ^ 1);
      // P0 under dP0 (its S is complete from slot P_D0 on), dS0 under S1 (dP0 is complete from P_S1 on),
      // P1 under dP1, dS1 under dQ0; each group ends before the MFMAs that need its operand
      p_piece(I, I0{}, std::integral_constant<int, P_D0 + 1>{}, std::integral_constant<int, KSD - 1>{});
      ds_piece(I, I0{}, std::integral_constant<int, P_S1 + 1>{}, std::integral_constant<int, (KS - 1 < 16 ? KS - 1 : 16)>{});
      p_piece(I, I1{}, std::integral_constant<int, P_D1 + 1>{}, std::integral_constant<int, KSD - 1>{});
      ds_piece(I, I1{}, std::integral_constant<int, P_Q0 + 1>{}, std::integral_constant<int, (A2 - 1 < 16 ? A2 - 1 : 16)>{});
      __builtin_amdgcn_sched_barrier(0);
    });
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's share of the next tile has landed
  };

  // the list entries of the tile being computed and of the next one, as scalars, read a tile ahead of their use
  i32x4 cur = entry(0), nxt = entry(1);
#pragma unroll
  for (int j = 0; j < 3; j++) {
    cur[j] = __builtin_amdgcn_readfirstlane(cur[j]);
    nxt[j] = __builtin_amdgcn_readfirstlane(nxt[j]);
  }
  if (nact > 0) {
    static_for<0, NLOAD2>([&](auto P) { load_piece(P, cur[0], 0); });
  }
  __builtin_amdgcn_s_waitcnt(0);  // the fragments above and the first tile have landed (see the forward kernel)
  __syncthreads();
  auto iteration = [&](auto BUFc, int it) {
    const int t = cur[0], t_next = nxt[0];
    const i32x4 after = entry(it + 2);
    const int kv0 = t * BN;
    bool skip = CAUSAL && (kv0 > wq_last + band_hi || kv0 + BN - 1 < wq0 - band_lo);
    bool need_mask = (kv0 + BN > Skv) || (wq0 + 32 > Sq) ||
                     (CAUSAL && (kv0 + BN - 1 > wq0 + band_hi || kv0 < wq_last - band_lo));
    if (SEG) {
      skip = skip || cur[2] < wqmin || cur[1] > wqmax;
      need_mask = need_mask || !(cur[1] == cur[2] && wqmin == wqmax && cur[1] == wqmin);
    }
    if (skip) {
      constexpr int buf = decltype(BUFc)::value;
      if (it + 1 < nact) {
        static_for<0, NLOAD2>([&](auto P) { load_piece(P, t_next, buf ^ 1); });
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
    } else if (need_mask) {
      tile_body(std::true_type{}, BUFc, t, t_next);
    } else {
      tile_body(std::false_type{}, BUFc, t, t_next);
    }
    __syncthreads();
    cur = nxt;
#pragma unroll
    for (int j = 0; j < 3; j++) nxt[j] = __builtin_amdgcn_readfirstlane(after[j]);
  };
  for (int it = 0; it < nact; it += 2) {
    iteration(std::integral_constant<int, 0>{}, it);
    if (it + 1 < nact) iteration(std::integral_constant<int, 1>{}, it + 1);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no LDS-writing load outlives the workgroup
  if constexpr (WIDE) {
    // the pinned accumulators are read by ordinary instructions from here on: past the last MFMA's latency
#pragma unroll
    for (int d = 0; d < DB; d++) asm volatile("s_nop 15\n\ts_nop 3" : "+a"(dqacc[d]) :: "memory");
  }

  if (qrow < Sq) {
    T* dqp = (T*)a.dq + b * a.dqs[0] + h * a.dqs[1] + qrow * a.dqs[2];
    const float sc = a.sm_scale;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int vq = 0; vq < 4; vq++) {
        const f32x16& o = dqacc[d];
        *(u32x2*)(dqp + d * 32 + 8 * vq + 4 * g) =
            pack4<T>(o[4 * vq] * sc, o[4 * vq + 1] * sc, o[4 * vq + 2] * sc, o[4 * vq + 3] * sc);
      }
  }
}

// ------------------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------------------
template <typename K>
static int set_max_lds(K kern, const char* what) {
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  TP_REQUIRE(e == hipSuccess, TP_ERR_LAUNCH, "%s: hipFuncSetAttribute failed: %s", what, hipGetErrorString(e));
  return TP_OK;
}

static inline void mark(void* const* events, int i, hipStream_t st) {
  if (events && events[i]) (void)hipEventRecord((hipEvent_t)events[i], st);
}

// The lean dQ kernel (attn_bwd_dq_plain_kernel) serves the plain and causal problems and segment ids with causality;
// it computes delta itself and runs first.  Everything else (mask extensions, segment ids without causality, unequal
// head dims without causality, a tile list too long for the LDS) takes the delta kernel and the general dQ kernel.
template <int DQK, int DV, bool CAUSAL, bool SEG>
struct LeanDq {
  // (unequal head dims without causality stay with the general kernel: the compiler copies the pinned accumulators
  // between the branches of that variant's loop, right behind the MFMAs that write them)
  static constexpr bool BUILT = (!SEG || CAUSAL) && (DQK == DV || CAUSAL);
  static size_t lds_bytes(int Skv) {
    constexpr int BN = 64;
    return 2 * (size_t)(DmaTile<DQK, true>::BYTES + DmaTile<DV, true>::BYTES) + (SEG ? 2 * BN * 4 + 16 * (size_t)((Skv + BN - 1) / BN) : 0);
  }
  static bool taken(int Skv) { return BUILT && lds_bytes(Skv) <= 160 * 1024; }
};

template <typename T, int DQK, int DV, bool CAUSAL, bool SEG>
static int launch_bwd(const BwdArgs& a, hipStream_t st, void* const* ev) {
  typedef LeanDq<DQK, DV, CAUSAL, SEG> Lean;
  const bool lean = Lean::taken(a.Skv);
  // dK/dV: three row-major buffers of Q and dO tiles, the row vectors, the tile list (checked before anything is launched)
  constexpr int DKDV_NBUF = 3, DKDV_BMQ = 64, DKDV_BNK = 128;
  constexpr int DKDV_BUF = DmaTile<DQK>::BYTES + DmaTile<DV>::BYTES;
  static_assert(DKDV_NBUF * DKDV_BUF <= 144 * 1024, "the three buffers must leave room for the row vectors and the tile list");
  const int nqt = (a.Sq + DKDV_BMQ - 1) / DKDV_BMQ;
  const size_t dkdv_smem = (size_t)DKDV_NBUF * DKDV_BUF + 3 * DKDV_BMQ * 16 + (SEG ? (size_t)(6 * nqt + 8 + 4) * 4 : 0);
  TP_REQUIRE(dkdv_smem <= 160 * 1024 && (size_t)3 * nqt * 4 <= (size_t)DKDV_NBUF * DKDV_BUF, TP_ERR_UNSUPPORTED,
             "tp_attn_bwd: Sq=%d needs %zu bytes of LDS (max 163840)", a.Sq, dkdv_smem);
  mark(ev, 0, st);
  if (!lean) {
    // delta
    const int64_t threads = (int64_t)a.B * a.Hq * a.Sq * (DV / 8);
    attn_delta_kernel<T, DV><<<dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st>>>(a);
    int rc = check_launch("tp_attn_bwd(delta)");
    if (rc) return rc;
  }
  mark(ev, 1, st);
  if constexpr (Lean::BUILT) {
    if (lean) {
      // dQ first: it leaves -delta and -LSE (log2 units) of every query row in the workspace for the dK/dV kernel
      constexpr int BM = 128;
      auto kern = attn_bwd_dq_plain_kernel<T, DQK, DV, CAUSAL, SEG>;
      static bool attr_set = false;
      if (!attr_set) {
        int rc = set_max_lds(kern, "tp_attn_bwd(dq)");
        if (rc) return rc;
        attr_set = true;
      }
      kern<<<dim3(xcd_grid((a.Sq + BM - 1) / BM, a.n_rep, a.B * a.Hkv)), dim3(256), Lean::lds_bytes(a.Skv), st>>>(a);
      int rc = check_launch("tp_attn_bwd(dq)");
      if (rc) return rc;
      mark(ev, 3, st);
    }
  }
  // dK, dV
  {
    auto kern = attn_bwd_dkdv_kernel<T, DQK, DV, DKDV_NBUF, CAUSAL, SEG>;
    static bool attr_set = false;
    if (!attr_set) {
      int rc = set_max_lds(kern, "tp_attn_bwd(dkdv)");
      if (rc) return rc;
      attr_set = true;
    }
    kern<<<dim3(xcd_grid((a.Skv + DKDV_BNK - 1) / DKDV_BNK, 1, a.B * a.Hkv)), dim3(256), dkdv_smem, st>>>(a);
    int rc = check_launch("tp_attn_bwd(dkdv)");
    if (rc) return rc;
  }
  mark(ev, 2, st);
  // dQ, the general kernel
  if constexpr (!Lean::BUILT || SEG) {
    if (!lean) {
    // eight waves (two per SIMD) where a wave's registers fit in half a SIMD's file
    // (the non-causal 128-wide variant does not fit 256 registers without spilling: it keeps four waves)
    constexpr int NW = (DQK == DV && (DQK <= 64 || (DQK <= 128 && CAUSAL))) ? 8 : 4;
    constexpr int BN = 64, BM = 32 * NW;
    constexpr int BUF = BN * RowTile<DQK>::STRIDE + BN * RowTile<DV>::STRIDE + DQK * TrTile64::ROW_BYTES + BN * 4;
    const int nt = (a.Skv + BN - 1) / BN;
    // (8 waves: a third transposed K tile)
    const size_t smem = 2 * (size_t)BUF + (NW == 8 ? (size_t)DQK * TrTile64::ROW_BYTES : 0) + (SEG ? (size_t)(3 * nt + 4 * NW) * 4 : 0);
    TP_REQUIRE(smem <= 160 * 1024, TP_ERR_UNSUPPORTED, "tp_attn_bwd: Skv=%d needs %zu bytes of LDS (max 163840)", a.Skv, smem);
    auto kern = attn_bwd_dq_kernel<T, DQK, DV, NW, CAUSAL, SEG>;
    static bool attr_set = false;
    if (!attr_set) {
      int rc = set_max_lds(kern, "tp_attn_bwd(dq)");
      if (rc) return rc;
      attr_set = true;
    }
    kern<<<dim3(xcd_grid((a.Sq + BM - 1) / BM, a.n_rep, a.B * a.Hkv)), dim3(64 * NW), smem, st>>>(a);
    int rc = check_launch("tp_attn_bwd(dq)");
    if (rc) return rc;
    }
  }
  if (!lean) mark(ev, 3, st);
  return TP_OK;
}

template <typename T, int DQK, int DV>
static int dispatch_bwd(const BwdArgs& a, int causal, hipStream_t st, void* const* ev) {
  if (a.mx.on) {
    // a window and / or a causal offset and nothing else: the causal kernels, with that band instead of (-inf, 0]
    // (where the lean dQ kernel serves the problem; the general dQ kernel knows plain causality only)
    const bool lean = a.seg ? LeanDq<DQK, DV, true, true>::taken(a.Skv) : LeanDq<DQK, DV, true, false>::taken(a.Skv);
    if (band_only(a.mx) && lean) {
      BwdArgs b = a;
      b.band_lo = a.mx.lo_off;
      b.band_hi = a.mx.hi_off;
      b.mx = no_mask_ext();
      if (a.seg) return launch_bwd<T, DQK, DV, true, true>(b, st, ev);
      return launch_bwd<T, DQK, DV, true, false>(b, st, ev);
    }
    // the other mask extensions: the general instantiation (causality is part of the band then)
    return launch_bwd<T, DQK, DV, false, true>(a, st, ev);
  }
  if (causal) {
    if (a.seg) return launch_bwd<T, DQK, DV, true, true>(a, st, ev);
    return launch_bwd<T, DQK, DV, true, false>(a, st, ev);
  }
  if (a.seg) {
    // segment ids without causality: the causal kernels with a band that covers every key, where the lean dQ kernel
    // serves the problem (else the general instantiation)
    if (LeanDq<DQK, DV, true, true>::taken(a.Skv)) {
      BwdArgs b = a;
      b.band_lo = BAND_INF;
      b.band_hi = BAND_INF;
      return launch_bwd<T, DQK, DV, true, true>(b, st, ev);
    }
    return launch_bwd<T, DQK, DV, false, true>(a, st, ev);
  }
  if constexpr (!LeanDq<DQK, DV, false, false>::BUILT) {
    // (head dims for which the lean dQ kernel exists with causality only: the same band)
    if (LeanDq<DQK, DV, true, false>::taken(a.Skv)) {
      BwdArgs b = a;
      b.band_lo = BAND_INF;
      b.band_hi = BAND_INF;
      return launch_bwd<T, DQK, DV, true, false>(b, st, ev);
    }
  }
  return launch_bwd<T, DQK, DV, false, false>(a, st, ev);
}

// One element type per translation unit: this file is compiled twice (TP_BWD_F16 = 0 and 1, side by side, which
// halves the build time).  Either unit defines its own dispatcher over the head dims; the bf16 unit also holds
// the C entry points.  A dispatcher returns TP_DIMS_NOT_BUILT for head dims it has no kernels for.
#ifndef TP_BWD_F16
#define TP_BWD_F16 0
#endif
constexpr int TP_DIMS_NOT_BUILT = -1000;
int bwd_by_dims_bf16(const BwdArgs& a, int Dqk, int Dv, int causal, hipStream_t st, void* const* ev);
int bwd_by_dims_f16(const BwdArgs& a, int Dqk, int Dv, int causal, hipStream_t st, void* const* ev);
template <typename T>
static int bwd_by_dims(const BwdArgs& a, int Dqk, int Dv, int causal, hipStream_t st, void* const* ev) {
  // (TP_ONLY_HEAD_DIM_128 / TP_ONLY_HEAD_DIM_WIDE: build options for quick timing builds of one head-dim pair)
#ifndef TP_ONLY_HEAD_DIM_WIDE
  if (Dqk == 128 && Dv == 128) return dispatch_bwd<T, 128, 128>(a, causal, st, ev);
#endif
#if !defined(TP_ONLY_HEAD_DIM_128) && !defined(TP_ONLY_HEAD_DIM_WIDE)
  if (Dqk == 64 && Dv == 64) return dispatch_bwd<T, 64, 64>(a, causal, st, ev);
#endif
#ifndef TP_ONLY_HEAD_DIM_128
  if (Dqk == 192 && Dv == 128) return dispatch_bwd<T, 192, 128>(a, causal, st, ev);
#endif
  return TP_DIMS_NOT_BUILT;
}
#if TP_BWD_F16
int bwd_by_dims_f16(const BwdArgs& a, int Dqk, int Dv, int causal, hipStream_t st, void* const* ev) {
  return bwd_by_dims<f16_t>(a, Dqk, Dv, causal, st, ev);
}
#else
int bwd_by_dims_bf16(const BwdArgs& a, int Dqk, int Dv, int causal, hipStream_t st, void* const* ev) {
  return bwd_by_dims<bf16_t>(a, Dqk, Dv, causal, st, ev);
}
#endif

}  // namespace tp

#if !TP_BWD_F16
using namespace tp;

extern "C" int tp_attn_bwd_dq_first(int Skv, int Dqk, int Dv, int causal, int has_seg, int masked, int dtype) {
  if (masked || (dtype != TP_BF16 && dtype != TP_F16)) return 0;
  auto pick = [&](auto dq, auto dv) -> int {
    constexpr int DQ = decltype(dq)::value, DVV = decltype(dv)::value;
    if (causal) return has_seg ? LeanDq<DQ, DVV, true, true>::taken(Skv) : LeanDq<DQ, DVV, true, false>::taken(Skv);
    // (segment ids without causality run the causal kernels with an all-covering band where the lean kernel serves them)
    if (has_seg || !LeanDq<DQ, DVV, false, false>::BUILT) return has_seg ? LeanDq<DQ, DVV, true, true>::taken(Skv) : LeanDq<DQ, DVV, true, false>::taken(Skv);
    return LeanDq<DQ, DVV, false, false>::taken(Skv);
  };
  typedef std::integral_constant<int, 64> I64;
  typedef std::integral_constant<int, 128> I128;
  typedef std::integral_constant<int, 192> I192;
  if (Dqk == 128 && Dv == 128) return pick(I128{}, I128{});
  if (Dqk == 64 && Dv == 64) return pick(I64{}, I64{});
  if (Dqk == 192 && Dv == 128) return pick(I192{}, I128{});
  return 0;
}

extern "C" size_t tp_attn_bwd_workspace_bytes(int B, int Hq, int Sq) {
  if (B <= 0 || Hq <= 0 || Sq <= 0) return 0;
  return 2 * (size_t)B * Hq * Sq * sizeof(float);  // delta and the log2-scaled LSE, one float per query row each
}

namespace tp {
// fp32 operands: attn_bwd_f32.hip
int attn_bwd_f32(const void* dout, const void* q, const void* k, const void* v, const void* out, const float* lse,
                 const int32_t* seg, void* dq, void* dk, void* dv, float* ws, int B, int Hq, int Hkv, int Sq, int Skv, int Dqk,
                 int Dv, const int64_t* dos, const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                 const int64_t* dqs, const int64_t* dks, const int64_t* dvs, float sm_scale, int causal, hipStream_t st,
                 const MaskExt& mx);
}  // namespace tp

static int attn_bwd_impl(const void* dout, const void* q, const void* k, const void* v, const void* out,
                         const float* lse, const int32_t* seg, void* dq, void* dk, void* dv, float* ws, int B, int Hq,
                         int Hkv, int Sq, int Skv, int Dqk, int Dv, const int64_t do_strides[3],
                         const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                         const int64_t o_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                         const int64_t dv_strides[3], float sm_scale, int causal, int dtype, void* stream,
                         void* const* events, const MaskExt& mx) {
  TP_REQUIRE(dout && q && k && v && out && lse && dq && dk && dv && ws, TP_ERR_BAD_ARG, "tp_attn_bwd: null pointer");
  TP_REQUIRE(do_strides && q_strides && k_strides && v_strides && o_strides && dq_strides && dk_strides && dv_strides,
             TP_ERR_BAD_ARG, "tp_attn_bwd: null stride array");
  TP_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Sq > 0 && Skv > 0, TP_ERR_BAD_ARG, "tp_attn_bwd: non-positive size");
  TP_REQUIRE(Hq % Hkv == 0, TP_ERR_BAD_ARG, "tp_attn_bwd: Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  TP_REQUIRE(!seg || Sq == Skv, TP_ERR_BAD_ARG, "tp_attn_bwd: segment ids need Sq == Skv (got %d, %d)", Sq, Skv);
  TP_REQUIRE(sm_scale > 0.f, TP_ERR_BAD_ARG, "tp_attn_bwd: sm_scale must be positive");
  if (dtype == TP_F32) {
    return attn_bwd_f32(dout, q, k, v, out, lse, seg, dq, dk, dv, ws, B, Hq, Hkv, Sq, Skv, Dqk, Dv, do_strides, q_strides, k_strides,
                        v_strides, o_strides, dq_strides, dk_strides, dv_strides, sm_scale, causal, (hipStream_t)stream, mx);
  }
  TP_REQUIRE(dtype == TP_BF16 || dtype == TP_F16, TP_ERR_UNSUPPORTED, "tp_attn_bwd: dtype %d (bf16, fp16 and fp32 only)", dtype);
  TP_REQUIRE((int64_t)(B + 8) * Hq * ((Sq + 127) / 128 + (Skv + 127) / 128) < (1ll << 31), TP_ERR_UNSUPPORTED, "tp_attn_bwd: too many workgroups");
  // the row-sum kernel runs one thread per 16 bytes of dO: its 1-D grid of 256-thread blocks has the same limit
  TP_REQUIRE(Dv > 0 && ((int64_t)B * Hq * Sq * (Dv / 8) + 255) / 256 < (1ll << 31), TP_ERR_UNSUPPORTED,
             "tp_attn_bwd: B*Hq*Sq*Dv = %lld elements of dO exceed the row-sum kernel's grid", (long long)B * Hq * Sq * Dv);
  BwdArgs a;
  a.q = q; a.k = k; a.v = v; a.out = out; a.dout = dout; a.lse = lse; a.seg = seg;
  a.dq = dq; a.dk = dk; a.dv = dv; a.delta = ws;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.Sq = Sq; a.Skv = Skv; a.n_rep = Hq / Hkv;
  bool ok = aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out) && aligned16(dout) && aligned16(dq) &&
            aligned16(dk) && aligned16(dv);
  for (int i = 0; i < 3; i++) {
    a.qs[i] = q_strides[i]; a.ks[i] = k_strides[i]; a.vs[i] = v_strides[i]; a.os[i] = o_strides[i];
    a.dos[i] = do_strides[i]; a.dqs[i] = dq_strides[i]; a.dks[i] = dk_strides[i]; a.dvs[i] = dv_strides[i];
    ok = ok && q_strides[i] % 8 == 0 && k_strides[i] % 8 == 0 && v_strides[i] % 8 == 0 && o_strides[i] % 8 == 0 &&
         do_strides[i] % 8 == 0 && dq_strides[i] % 4 == 0 && dk_strides[i] % 4 == 0 && dv_strides[i] % 4 == 0;
  }
  TP_REQUIRE(ok, TP_ERR_BAD_ARG, "tp_attn_bwd: pointers and strides must keep rows 16-byte aligned");
  {
    // tiles are addressed with 32-bit byte offsets inside one (batch, head) slice
    const int64_t lim = 1ll << 31;
    const bool fits = ((int64_t)Sq * q_strides[2] + Dqk) * 2 < lim && ((int64_t)Sq * do_strides[2] + Dv) * 2 < lim &&
                      ((int64_t)Skv * k_strides[2] + Dqk) * 2 < lim && ((int64_t)Skv * v_strides[2] + Dv) * 2 < lim;
    TP_REQUIRE(q_strides[2] > 0 && do_strides[2] > 0 && k_strides[2] > 0 && v_strides[2] > 0, TP_ERR_BAD_ARG,
               "tp_attn_bwd: sequence strides must be positive");
    TP_REQUIRE(fits, TP_ERR_UNSUPPORTED, "tp_attn_bwd: one (batch, head) slice of q, dO, k or v spans 2 GiB or more");
  }
  a.scale_log2 = sm_scale * LOG2E;
  a.sm_scale = sm_scale;
  a.mx = mx;
  a.band_lo = BAND_INF;  // plain causality (used by the causal kernels only)
  a.band_hi = 0;
  hipStream_t st = (hipStream_t)stream;
  const int rc = dtype == TP_BF16 ? bwd_by_dims_bf16(a, Dqk, Dv, causal, st, events) : bwd_by_dims_f16(a, Dqk, Dv, causal, st, events);
  TP_REQUIRE(rc != TP_DIMS_NOT_BUILT, TP_ERR_UNSUPPORTED, "tp_attn_bwd: head dims (qk=%d, v=%d) not built", Dqk, Dv);
  return rc;
}

extern "C" int tp_attn_bwd_ex(const void* dout, const void* q, const void* k, const void* v, const void* out,
                              const float* lse, const int32_t* seg, void* dq, void* dk, void* dv, float* ws, int B, int Hq,
                              int Hkv, int Sq, int Skv, int Dqk, int Dv, const int64_t do_strides[3],
                              const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                              const int64_t o_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                              const int64_t dv_strides[3], float sm_scale, int causal, int dtype, void* stream,
                              void* const* events) {
  return attn_bwd_impl(dout, q, k, v, out, lse, seg, dq, dk, dv, ws, B, Hq, Hkv, Sq, Skv, Dqk, Dv, do_strides, q_strides,
                       k_strides, v_strides, o_strides, dq_strides, dk_strides, dv_strides, sm_scale, causal, dtype, stream,
                       events, no_mask_ext());
}

extern "C" int tp_attn_bwd_masked(const void* dout, const void* q, const void* k, const void* v, const void* out,
                                  const float* lse, const int32_t* seg, const int32_t* q_positions, void* dq, void* dk,
                                  void* dv, float* ws, int B, int Hq, int Hkv, int Sq, int Skv, int Dqk, int Dv,
                                  const int64_t do_strides[3], const int64_t q_strides[3], const int64_t k_strides[3],
                                  const int64_t v_strides[3], const int64_t o_strides[3], const int64_t dq_strides[3],
                                  const int64_t dk_strides[3], const int64_t dv_strides[3], float sm_scale, int causal,
                                  int causal_offset, int window_left, int window_right, float logits_soft_cap, int dtype,
                                  void* stream) {
  TP_REQUIRE(sm_scale > 0.f, TP_ERR_BAD_ARG, "tp_attn_bwd_masked: sm_scale must be positive");
  TP_REQUIRE(window_left < BAND_INF && window_right < BAND_INF && causal_offset > -BAND_INF && causal_offset < BAND_INF, TP_ERR_BAD_ARG,
             "tp_attn_bwd_masked: window or offset out of range");
  return attn_bwd_impl(dout, q, k, v, out, lse, seg, dq, dk, dv, ws, B, Hq, Hkv, Sq, Skv, Dqk, Dv, do_strides, q_strides,
                       k_strides, v_strides, o_strides, dq_strides, dk_strides, dv_strides, sm_scale, causal, dtype, stream,
                       nullptr, make_mask_ext(q_positions, causal, causal_offset, window_left, window_right, logits_soft_cap, sm_scale));
}

extern "C" int tp_attn_bwd_biased(const void* dout, const void* q, const void* k, const void* v, const void* out,
                                  const float* lse, const int32_t* seg, const int32_t* q_positions, const float* bias,
                                  const int64_t bias_strides[3], void* dq, void* dk, void* dv, float* ws, int B, int Hq,
                                  int Hkv, int Sq, int Skv, int Dqk, int Dv, const int64_t do_strides[3],
                                  const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                                  const int64_t o_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                                  const int64_t dv_strides[3], float sm_scale, int causal, int causal_offset, int window_left,
                                  int window_right, float logits_soft_cap, int dtype, void* stream) {
  TP_REQUIRE(sm_scale > 0.f, TP_ERR_BAD_ARG, "tp_attn_bwd_biased: sm_scale must be positive");
  TP_REQUIRE(window_left < BAND_INF && window_right < BAND_INF && causal_offset > -BAND_INF && causal_offset < BAND_INF, TP_ERR_BAD_ARG,
             "tp_attn_bwd_biased: window or offset out of range");
  TP_REQUIRE(bias && bias_strides, TP_ERR_BAD_ARG, "tp_attn_bwd_biased: null bias");
  TP_REQUIRE(bias_strides[0] >= 0 && bias_strides[1] >= 0 && bias_strides[2] >= 0, TP_ERR_BAD_ARG,
             "tp_attn_bwd_biased: negative bias stride");
  return attn_bwd_impl(dout, q, k, v, out, lse, seg, dq, dk, dv, ws, B, Hq, Hkv, Sq, Skv, Dqk, Dv, do_strides, q_strides,
                       k_strides, v_strides, o_strides, dq_strides, dk_strides, dv_strides, sm_scale, causal, dtype, stream,
                       nullptr,
                       make_mask_ext(q_positions, causal, causal_offset, window_left, window_right, logits_soft_cap, sm_scale, bias,
                                     bias_strides));
}

extern "C" int tp_attn_bwd(const void* dout, const void* q, const void* k, const void* v, const void* out,
                           const float* lse, const int32_t* seg, void* dq, void* dk, void* dv, float* ws, int B, int Hq,
                           int Hkv, int Sq, int Skv, int Dqk, int Dv, const int64_t do_strides[3],
                           const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                           const int64_t o_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                           const int64_t dv_strides[3], float sm_scale, int causal, int dtype, void* stream) {
  return tp_attn_bwd_ex(dout, q, k, v, out, lse, seg, dq, dk, dv, ws, B, Hq, Hkv, Sq, Skv, Dqk, Dv, do_strides, q_strides,
                        k_strides, v_strides, o_strides, dq_strides, dk_strides, dv_strides, sm_scale, causal, dtype, stream,
                        nullptr);
}
#endif  // !TP_BWD_F16
