// Attention forward for gfx950: causal / segment-masked GQA, bf16 or fp16 in, fp32 accumulate.
//
// Replaces AttentionModule.forward's three branches (torchprime/torch_xla_models/attention.py:70-170)
// and the segment-id path of torchprime/utils/kernel_utils.py:215-220, 259-263.
//
// Structure (one workgroup = 4 waves = 128 query rows of one (batch, head); KV tiles of 64):
//   * the scores are computed TRANSPOSED, S^T = K Q^T, so that in the MFMA result layout a lane owns
//     one query column and 16 key rows per 32x32 block: row max / sum / rescale are per-lane scalars
//     (one half-wave exchange per tile), and exp(S^T) converted to 16 bit is already the B operand of
//     O^T += V^T P^T - P never goes through LDS;
//   * Q fragments stay in registers for the whole KV loop; K and V tiles are row-major in LDS (dense rows, 16-byte
//     chunks XOR-swizzled by the row): K fragments are conflict-free 16-byte reads, the V^T operand comes out of
//     transposing 8-byte reads of the same kind of tile;
//   * the next tile is fetched while the current one is being multiplied, K and V by buffer loads that write LDS
//     directly (no staging registers, no LDS stores); LDS double buffer, one barrier per tile;
//   * causal: the KV loop ends at the diagonal, element masks only on tiles that straddle it;
//     segments: per-tile [min,max] of the ids is computed once per workgroup, tiles whose id range
//     misses the query rows' range are skipped, element compares only where ranges are not one id.
#include <type_traits>

#include "attn_common.hpp"

namespace tp {

struct FwdArgs {
  const void* q;
  const void* k;
  const void* v;
  const int32_t* seg;
  void* out;
  float* lse;
  int B, Hq, Hkv, Sq, Skv, n_rep;
  int64_t qs[3], ks[3], vs[3], os[3];
  float scale_log2;  // sm_scale * log2(e)
  // the causal kernels' band: query row i sees keys i - band_lo .. i + band_hi (plain causality: no lower bound, 0).
  // Sliding windows and causal offsets without the other mask extensions run through these kernels.
  int band_lo, band_hi;
  MaskExt mx;
};

// Two workgroups per CU (256 registers per lane) where the kernel fits them; the non-causal variants at head dims of
// 128 and more (run-time buffer index, mask extensions) and the 192-wide heads with segment ids need more registers
// or LDS and take one workgroup per CU instead of spilling a hundred registers.
template <int DQK, bool CAUSAL, bool SEG>
constexpr int fwd_blocks_per_cu() { return (DQK >= 128 && !CAUSAL) || (DQK > 128 && SEG) ? 1 : 2; }
// The tiles are filled by buffer loads that write LDS directly (DmaTile): no staging registers, no LDS stores, and
// dense swizzled rows instead of padded ones.  For the causal 192-wide heads that is what lets two workgroups share a
// CU: two double-buffered tile sets of 81920 bytes fill the CU's 160 KB exactly (forward at 128 heads x 4096 rows:
// 1.16 -> 0.89 ms with K loaded that way, 0.72 ms with V as well).

template <typename T, int DQK, int DV, bool CAUSAL, bool SEG>
__global__ __launch_bounds__(256, (fwd_blocks_per_cu<DQK, CAUSAL, SEG>())) void attn_fwd_kernel(const FwdArgs a) {
  typedef typename MT<T>::v8 v8;
  constexpr int BN = 64;              // kv rows per LDS tile, processed as two halves of 32
  constexpr int BM = 128;             // q rows per workgroup, 32 per wave
  constexpr int KSTEPS = DQK / 16;    // MFMA k-steps over the qk head dim
  constexpr int DVB = DV / 32;        // 32-column blocks of the v head dim
  typedef DmaTile<DQK, true> KD;
  typedef DmaTile<DV, true> VD;  // row-major like K; its transposed operand comes out of transposing LDS reads
  constexpr int K_BYTES = KD::BYTES;
  constexpr int V_BYTES = VD::BYTES;
  constexpr int SEG_BYTES = SEG ? BN * 4 : 0;
  constexpr int BUF_BYTES = K_BYTES + V_BYTES + SEG_BYTES;
  // LDS layout: the two K tiles, then the two V^T tiles, then the two segment-id rows: with the buffer index a
  // constant, every address is a loop-invariant per-lane offset plus an immediate
  // (the plain causal kernel only: the other variants keep a buffer's K, V^T and ids together, one base
  // register for all three, which is what their register budget allows)
  constexpr bool STATIC_BUF = CAUSAL && !SEG;
  constexpr int K_AT = 0, K_STEP = STATIC_BUF ? K_BYTES : BUF_BYTES;
  constexpr int V_AT = STATIC_BUF ? 2 * K_BYTES : K_BYTES, V_STEP = STATIC_BUF ? V_BYTES : BUF_BYTES;
  constexpr int SEG_AT = STATIC_BUF ? 2 * (K_BYTES + V_BYTES) : K_BYTES + V_BYTES, SEG_STEP = STATIC_BUF ? SEG_BYTES : BUF_BYTES;
  constexpr int K_ITEMS = KD::PER_WAVE, V_ITEMS = VD::PER_WAVE;  // LDS-writing loads per wave and tile

  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, ln = lane & 31;
  const int n_qt = (a.Sq + BM - 1) / BM;
  int tile, inner, group;
  if (!xcd_map(n_qt, a.n_rep, a.B * a.Hkv, tile, inner, group)) return;
  const int qt = n_qt - 1 - tile;  // longest (latest) query tiles are scheduled first
  const int b = group / a.Hkv, hk = group - b * a.Hkv, h = hk * a.n_rep + inner;
  const int q0 = qt * BM;
  const int wq0 = q0 + wave * 32;
  const int Sq = a.Sq, Skv = a.Skv;

  const T* qb = (const T*)a.q + b * a.qs[0] + h * a.qs[1];
  const T* kb = (const T*)a.k + b * a.ks[0] + hk * a.ks[1];
  const T* vb = (const T*)a.v + b * a.vs[0] + hk * a.vs[1];
  // GEN: the instantiation that also evaluates the mask extensions (and then may run without segment ids)
  constexpr bool GEN = !CAUSAL && SEG;
  const bool has_seg = SEG && (!GEN || a.seg != nullptr);
  const bool ext = GEN && a.mx.on;
  const bool capped = GEN && a.mx.cap_in != 0.f;
  const bool biased = GEN && a.mx.bias != nullptr;
  const int32_t* segb = has_seg ? a.seg + (int64_t)b * Skv : nullptr;

  const int band_lo = CAUSAL ? a.band_lo : BAND_INF, band_hi = CAUSAL ? a.band_hi : BAND_INF;
  const int kv_end = CAUSAL ? max(min(Skv, q0 + BM + band_hi), 0) : Skv;
  const int ntiles = (kv_end + BN - 1) / BN;
  const int t_first = CAUSAL ? min(max(q0 - band_lo, 0) / BN, ntiles) : 0;  // (tiles before it lie left of every row's band)

  // ---- Q fragments (B operand of S^T = K Q^T): lane = query column, 8 head-dim values per k-step
  v8 qf[KSTEPS];
  const int qrow = wq0 + ln;
  {
    const T* qp = qb + min(qrow, Sq - 1) * a.qs[2] + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) qf[ks] = *(const v8*)(qp + 16 * ks);
  }
  const int segq = has_seg ? segb[min(qrow, Sq - 1)] : 0;
  // additive mask: this lane's query row of it
  const float* bias_row = biased ? a.mx.bias + b * a.mx.bias_s[0] + h * a.mx.bias_s[1] + (int64_t)min(qrow, Sq - 1) * a.mx.bias_s[2] : nullptr;
  // band of allowed keys of this lane's query row, and its extent over the wave
  int lo_q = -BAND_INF, hi_q = BAND_INF, wpmin = 0, wpmax = 0;
  if (ext) {
    const int qc = min(qrow, Sq - 1);
    const int qp = a.mx.qpos ? a.mx.qpos[qc] : qc;
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

  // ---- segment bookkeeping: per-tile id ranges, list of tiles that can contain an allowed pair
  // (the tiles' id ranges are only needed until the list is built: they borrow the tile buffers, which nothing has
  // been loaded into yet; the list holds (tile, min id, max id) in 16 bytes per visited tile, which one LDS read
  // fetches a tile ahead of its use)
  int* kvmin = (int*)smem;
  int* kvmax = kvmin + ntiles;
  int* bq = kvmax + ntiles;  // 16 ints: per-wave (min,max) of the query rows' ids, then of their positions
  const int* ctl = (const int*)(smem + 2 * BUF_BYTES);
  int nact = ntiles - t_first;
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
    if (lane == 0) { bq[2 * wave] = wqmin; bq[2 * wave + 1] = wqmax; bq[8 + 2 * wave] = wpmin; bq[9 + 2 * wave] = wpmax; }
    static_assert(BN == 64, "seg_tile_ranges works on 64-row tiles");
    if (has_seg) {
      seg_tile_ranges(segb, Skv, 0, ntiles, kvmin, kvmax, tid, 256);
    } else {
      for (int t = tid; t < ntiles; t += 256) { kvmin[t] = 0; kvmax[t] = 0; }
    }
    __syncthreads();
    const int bqmin = min(min(bq[0], bq[2]), min(bq[4], bq[6]));
    const int bqmax = max(max(bq[1], bq[3]), max(bq[5], bq[7]));
    // keys any row of the workgroup may see
    const int b_lo = ext ? min(min(bq[8], bq[10]), min(bq[12], bq[14])) - a.mx.lo_off : t_first * BN;
    const int b_hi = ext ? max(max(bq[9], bq[11]), max(bq[13], bq[15])) + a.mx.hi_off : BAND_INF;
    // every wave builds the same list redundantly (no second barrier needed for the count)
    int cnt = 0;
    for (int base = 0; base < ntiles; base += 64) {
      const int t = base + lane;
      const int lo = t < ntiles ? kvmin[t] : 0, hi = t < ntiles ? kvmax[t] : 0;
      const bool act = t < ntiles && !(hi < bqmin || lo > bqmax) && t * BN <= b_hi && t * BN + BN - 1 >= b_lo;
      const unsigned long long m = __ballot(act);
      if (act && wave == 0)
        *(i32x4*)(smem + 2 * BUF_BYTES + 16 * (cnt + __popcll(m & ((1ull << lane) - 1ull)))) = i32x4{t, lo, hi, 0};
      cnt += __popcll(m);
    }
    nact = cnt;
    __syncthreads();  // the list is complete and the ranges are no longer read: the first tile may land on them
  }
  // list entry i as scalars (a tile offset in vector registers would put every load into a loop over its values)
  auto entry = [&](int i) -> i32x4 {
    i32x4 e = i32x4{min(t_first + i, ntiles - 1), 0, 0, 0};
    if (SEG) e = *(const i32x4*)(ctl + 4 * max(min(i, nact - 1), 0));
    return e;
  };
  auto scalars = [](i32x4 e) {
    return i32x4{__builtin_amdgcn_readfirstlane(e[0]), __builtin_amdgcn_readfirstlane(e[1]), __builtin_amdgcn_readfirstlane(e[2]), 0};
  };

  // ---- K and V tiles travel from memory into LDS by loads that write LDS themselves (rows past Skv arrive as zeros)
  const unsigned k_tile_bytes = (unsigned)(BN * a.ks[2] * 2), v_tile_bytes = (unsigned)(BN * a.vs[2] * 2);
  KD kdma;
  VD vdma;
  kdma.init(a.ks[2], wave, lane);
  vdma.init(a.vs[2], wave, lane);
  const u32x4 krw = make_rsrc_words(kb, span_bytes(Skv, a.ks[2], DQK));
  const u32x4 vrw = make_rsrc_words(vb, span_bytes(Skv, a.vs[2], DV));
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const unsigned lds_base = __builtin_amdgcn_readfirstlane((unsigned)(size_t)smem);
  // this wave's first LDS destinations in buffer 0 (scalar byte addresses)
  const unsigned kdst0 = lds_base + (unsigned)K_AT + (unsigned)(wave_s * K_ITEMS * 1024);
  const unsigned vdst0 = lds_base + (unsigned)V_AT + (unsigned)(wave_s * V_ITEMS * 1024);
  int sreg = 0;
  // piece P of the K_ITEMS + V_ITEMS loads of tile t into buffer kbuf, for issuing between MFMAs
  auto load_piece = [&](auto Pc, int t, int kbuf) {
    constexpr int p = decltype(Pc)::value;
    if constexpr (p < K_ITEMS)
      kdma.template issue_one_at<p>(krw, __builtin_amdgcn_readfirstlane((unsigned)t * k_tile_bytes), kdst0 + (unsigned)(kbuf * K_STEP));
    else
      vdma.template issue_one_at<p - K_ITEMS>(vrw, __builtin_amdgcn_readfirstlane((unsigned)t * v_tile_bytes), vdst0 + (unsigned)(kbuf * V_STEP));
  };
  // the whole tile at once (nobody reads buffer kbuf before the next barrier)
  auto load_tile = [&](int t, int kbuf) {
    static_for<0, K_ITEMS + V_ITEMS>([&](auto P) { load_piece(P, t, kbuf); });
    if (has_seg && tid < BN) sreg = segb[min(t * BN + tid, Skv - 1)];
  };
  // what is left to do before the barrier that hands buffer `buf` over: the id row, and the wait for this wave's
  // loads (they are outside the compiler's bookkeeping)
  auto store_tile = [&](int buf) {
    if (SEG && tid < BN) ((int*)(smem + SEG_AT + buf * SEG_STEP))[tid] = sreg;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };

  // ---- accumulators: O^T blocks, running max (log2 units), per-lane partial row sum
  f32x16 oacc[DVB];
#pragma unroll
  for (int d = 0; d < DVB; d++)
#pragma unroll
    for (int v = 0; v < 16; v++) oacc[d][v] = 0.f;
  float m_run = -INFINITY;  // reference max of the row (stale by at most 8: lazy rescale)
  float m_use = 0.f;        // m_run, or 0 while the row has seen no allowed key
  // (Row sums by the matrix unit - a block of ones beside V^T, two more MFMAs per 32 key rows instead of 32 additions
  // per lane - were measured and dropped: they sum the 16-bit P, the LSE then carries P's rounding (up to 2^-9
  // relative when one key dominates a row), and the backward, which rebuilds P from the LSE, inherits it.)
  float l_run = 0.f;
  const float c = a.scale_log2;

  // Online softmax of one 32-row half of S^T held in `s` (lane = query column, 16 key rows):
  // updates the row state and returns exp2(s*c - m) in place.  The running max only moves when the
  // half's max exceeds it by more than 2^8, so p stays <= 256 (harmless in fp32 sums and in the 16-bit
  // P operand) and the rescale of O, a wave-uniform branch, is off the common path.
  // Returns true (wave-uniform) when some lane moved its reference max; `alpha` is then the factor its
  // O accumulators must be multiplied by (1 for lanes that kept theirs).  m_run, m_use and l_run are
  // updated here; rescaling O is left to the caller, who knows which P V products are already in O.
  auto row_max_update = [&](const f32x16& s, float& alpha) -> bool {
    float mx = fmaxf(fmaxf(s[0], s[1]), s[2]);
#pragma unroll
    for (int v = 3; v < 15; v += 2) mx = fmaxf(fmaxf(mx, s[v]), s[v + 1]);
    mx = fmaxf(mx, s[15]);
    mx = half_max(mx);
    const float mxs = mx * c;
    const bool grow = mxs > m_run + 8.0f;
    alpha = 1.0f;
    const bool any = __builtin_amdgcn_ballot_w64(grow) != 0;
    if (any) {
      const float m_new = grow ? mxs : m_run;
      const float m_new_use = (m_new == -INFINITY) ? 0.f : m_new;
      alpha = grow ? fast_exp2(m_run - m_new_use) : 1.0f;
      m_run = m_new;
      m_use = m_new_use;
      l_run *= alpha;
    }
    return any;
  };
  auto rescale_o = [&](float alpha) {
#pragma unroll
    for (int d = 0; d < DVB; d++)
#pragma unroll
      for (int v = 0; v < 16; v++) oacc[d][v] *= alpha;
  };
  // One LDS tile, laid out slot by slot (one MFMA per slot, a scheduling barrier after each): the LDS
  // fragment of a slot is requested AHEAD slots earlier, so no phase starts by waiting out an LDS round trip,
  // and the softmax arithmetic of one 32-row half is spread under the MFMAs that follow it:
  //   slots   S0 = K[0:32] Q^T | S1 = K[32:64] Q^T | O += V[0:32]^T P0 | O += V[32:64]^T P1
  //   VALU                     | max0, exp(S0)     | max1, exp(S1)     | (LDS store of the next tile after)
  // Per-lane LDS byte addresses of the operands in buffer 0 (the workgroup's LDS base included), each an opaque
  // register: every fragment read is such a register plus an immediate (plus, where the buffer index is a run-time
  // value, one add per tile).
  //   kfo   K fragments: row ln (+32 for the second half), chunk 2 ks + g.  With 24 chunks per row the swizzle has
  //         three bits, so only the low three bits of the chunk depend on the lane: four offsets (ks & 3), the rest
  //         is an immediate; with 16 chunks per row it has four bits: one offset per k-step
  //   vfo   transposing reads of V: v-dim block d (32 columns), rows 8 h2 + 4 g ..+3 of a group of 16 key rows
  //         (the half of the tile and the k-step are immediates: multiples of 16 rows leave the swizzle alone);
  //         they carry V_AT, which would not fit an instruction offset for the wide heads
  const unsigned lds0 = (unsigned)(size_t)smem;
  constexpr bool KSWZ3 = KD::CPR % 16 != 0;
  constexpr int NKFO = KSWZ3 ? (KSTEPS < 4 ? KSTEPS : 4) : KSTEPS;
  unsigned kfo[NKFO], vfo[DVB][2];
#pragma unroll
  for (int j = 0; j < NKFO; j++) {
    kfo[j] = lds0 + (unsigned)K_AT + (unsigned)(ln * KD::ROWB + (((2 * j + g) ^ KD::swz(ln)) << 4));
    asm volatile("" : "+v"(kfo[j]));
  }
#pragma unroll
  for (int d = 0; d < DVB; d++)
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++) {
      vfo[d][h2] = lds0 + (unsigned)V_AT + (unsigned)VD::tr_off(8 * h2 + 4 * g, 2 * d + ((lane >> 4) & 1), lane & 15);
      asm volatile("" : "+v"(vfo[d][h2]));
    }
  auto ld16 = [](unsigned addr) { return *(const __attribute__((address_space(3))) v8*)addr; };
  auto ldtr = [](unsigned a0, unsigned a1) { return tr_read8<v8>((const lds_byte*)a0, (const lds_byte*)a1); };
  auto tile_body = [&](auto masked_c, auto BUFc, int buf_rt, int t, bool has_next, int t_next) {
    constexpr bool MASKED = decltype(masked_c)::value;
    // the buffer index: a constant, or (-1) the run-time one
    const int buf = decltype(BUFc)::value >= 0 ? decltype(BUFc)::value : buf_rt;
    const int kv0 = t * BN;
    const unsigned kl = (unsigned)(buf * K_STEP), vl = (unsigned)(buf * V_STEP);  // + kfo[] / vfo[]
    const int* sl = (const int*)(smem + SEG_AT + buf * SEG_STEP);
    // Masked tiles: which of the tile's 64 kv rows this lane's query row may see, one bit per row, built once per
    // tile (bounds, causality and the band of the mask extensions are a bit range; the rows of each id present among
    // the wave's query rows come from a ballot over the tile's id vector).  An element then costs a bit-field
    // extract and a bit-field insert of -inf instead of its compares.  kbits[hf] is shifted so that value v of the
    // lane's 16 is bit 8 (v / 4) + v % 4.
    unsigned kbits[2] = {0u, 0u};
    if (MASKED) {
      int lo = 0, hi = min(Skv - kv0, BN);
      if (CAUSAL) {
        hi = min(hi, qrow + band_hi - kv0 + 1);
        lo = max(qrow - band_lo - kv0, 0);
      }
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
    }
    auto mask_half = [&](f32x16& s, int hf) {
#pragma unroll
      for (int v = 0; v < 16; v++) {
        // soft cap on the raw score, rescaled so that the common scale c still applies afterwards
        if (GEN) {
          if (capped) s[v] = a.mx.cap_out * fast_tanh(s[v] * a.mx.cap_in);
          // additive mask, in units of the raw score (-inf stays -inf)
          if (biased) s[v] += a.mx.bias_mul * bias_row[min(kv0 + 32 * hf + 8 * (v / 4) + 4 * g + (v % 4), Skv - 1)];
        }
        const unsigned keep = (unsigned)__builtin_amdgcn_sbfe((int)kbits[hf], 8 * (v / 4) + (v % 4), 1);  // all ones or zero
        const float x = s[v];
        s[v] = __uint_as_float((__float_as_uint(x) & keep) | (0xff800000u & ~keep));
      }
    };
    constexpr int PVB = DVB, S1 = KSTEPS, PV0 = 2 * KSTEPS, PV1 = PV0 + 2 * PVB, NS = PV1 + 2 * PVB;
    constexpr int AHEAD = (CAUSAL && DQK <= 128) ? 5 : 3, NF = AHEAD + 1;  // (the plain causal kernel up to head dim 128 has registers left for a deeper ring; seven slots gain nothing)
    v8 fr[NF];
    f32x16 s[2];
    v8 pf[2][2];
    float alpha0 = 1.f, alpha1 = 1.f, rs0 = 0.f, rs1 = 0.f;
    bool moved1 = false;
    auto frag = [&](auto I) -> v8 {
      constexpr int i = decltype(I)::value;
      if constexpr (i < PV0) {
        constexpr int hf = i / KSTEPS, ks = i % KSTEPS;
        return ld16(kfo[KSWZ3 ? (ks & 3) : ks] + (kl + (unsigned)(hf * 32 * KD::ROWB + (KSWZ3 ? 128 * (ks >> 2) : 0))));
      } else {
        // V^T block d, contraction over key rows 32 hf + 16 kk + {4g..4g+3, 8+4g..8+4g+3}: the order in which P holds them
        constexpr int hf = (i - PV0) / (2 * PVB), j = (i - PV0) % (2 * PVB), kk = j / PVB, d = j % PVB;
        constexpr unsigned rows = (unsigned)((32 * hf + 16 * kk) * VD::ROWB);
        return ldtr(vfo[d][0] + (vl + rows), vfo[d][1] + (vl + rows));
      }
    };

    auto mma = [&](auto I, const v8& f) {
      constexpr int i = decltype(I)::value;
      const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if constexpr (i < PV0) {
        constexpr int hf = i / KSTEPS, ks = i % KSTEPS;
        s[hf] = MT<T>::mfma32(f, qf[ks], ks == 0 ? zero : s[hf]);
      } else {
        constexpr int hf = (i - PV0) / (2 * PVB), j = (i - PV0) % (2 * PVB), kk = j / PVB, d = j % PVB;
        oacc[d] = MT<T>::mfma32(f, pf[hf][kk], oacc[d]);
      }
    };
    // exponentials of half HF: its 16 values spread over the LEN slots from START on (plain adds for the row
    // sum: v_dot2 shares the matrix pipe and would serialise with the MFMAs).  A slot's values join the row sum and
    // the 16-bit operand one slot later (sum_part), so that no instruction waits for an exponential just issued.
    auto exp_part = [&](auto I, auto HFc, auto STARTc, auto LENc) {
      constexpr int i = decltype(I)::value, hf = decltype(HFc)::value, st = decltype(STARTc)::value, len = decltype(LENc)::value;
      if constexpr (i >= st && i < st + len) {
        constexpr int k = i - st, lo = (k * 16 + len - 1) / len, hi = ((k + 1) * 16 + len - 1) / len;
#pragma unroll
        for (int v = lo; v < hi; v++) {
          float pv = fast_exp2(__builtin_fmaf(s[hf][v], c, -m_use));
          asm volatile("" : "+v"(pv));  // keeps the computation in this slot
          s[hf][v] = pv;
        }
      }
    };
    auto sum_part = [&](auto I, auto HFc, auto STARTc, auto LENc) {
      constexpr int i = decltype(I)::value, hf = decltype(HFc)::value, st = decltype(STARTc)::value + 1, len = decltype(LENc)::value;
      if constexpr (i >= st && i < st + len) {
        constexpr int k = i - st, lo = (k * 16 + len - 1) / len, hi = ((k + 1) * 16 + len - 1) / len;
#pragma unroll
        for (int v = lo; v < hi; v++) {
          if (v & 1) rs1 += s[hf][v];
          else rs0 += s[hf][v];
        }
        static_for<0, 2>([&](auto H) {
          constexpr int hh = decltype(H)::value;
          if constexpr (8 * hh + 8 > lo && 8 * hh + 8 <= hi) {
            const f32x16& x = s[hf];
            pf[hf][hh] = pack8<T>(x[8 * hh + 0], x[8 * hh + 1], x[8 * hh + 2], x[8 * hh + 3], x[8 * hh + 4],
                                  x[8 * hh + 5], x[8 * hh + 6], x[8 * hh + 7]);
          }
        });
      }
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;
    static_for<0, AHEAD>([&](auto I) { fr[decltype(I)::value % NF] = frag(I); });
    static_for<0, NS>([&](auto I) {
      constexpr int i = decltype(I)::value;
      if constexpr (i + AHEAD < NS) fr[(i + AHEAD) % NF] = frag(std::integral_constant<int, i + AHEAD>{});
      mma(I, fr[i % NF]);
      // the next tile's loads, one per slot (past the last tile they re-read the last one: no branch here)
      if constexpr (i < K_ITEMS + V_ITEMS) load_piece(I, t_next, buf ^ 1);
      if constexpr (i == 0) {
        if (has_seg && tid < BN) sreg = segb[min(t_next * BN + tid, Skv - 1)];
      }
      // one slot after the last MFMA of a half: mask, running max (the rare rescale of O is a wave-uniform
      // branch), then the exponentials under the following MFMAs
      if constexpr (i == S1) {
        if (MASKED) mask_half(s[0], 0);
        if (row_max_update(s[0], alpha0)) rescale_o(alpha0);
      }
      // (the last values of half 0 join the sums before the sums join l_run below)
      sum_part(I, I0{}, std::integral_constant<int, S1 + 1>{}, std::integral_constant<int, KSTEPS - 1>{});
      if constexpr (i == PV0) {
        if (MASKED) mask_half(s[1], 1);
        // half 0's row sums join l_run before the update can rescale it; P0 itself is relative to the
        // reference max before this update: O is rescaled only after V0^T P0 is in it
        l_run += rs0 + rs1;
        rs0 = 0.f;
        rs1 = 0.f;
        moved1 = row_max_update(s[1], alpha1);
      }
      exp_part(I, I0{}, std::integral_constant<int, S1 + 1>{}, std::integral_constant<int, KSTEPS - 1>{});
      sum_part(I, I1{}, std::integral_constant<int, PV0 + 1>{}, std::integral_constant<int, 2 * PVB - 1>{});
      exp_part(I, I1{}, std::integral_constant<int, PV0 + 1>{}, std::integral_constant<int, 2 * PVB - 1>{});
      if constexpr (i == PV1 - 1) {
        if (moved1) rescale_o(alpha1);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    l_run += rs0 + rs1;
    if (has_next) store_tile(buf ^ 1);
  };

  // the entries of the tile being computed and of the next one; the one after is read at the top of a tile
  i32x4 cur = scalars(entry(0)), nxt = scalars(entry(1));
  if (nact > 0) {
    load_tile(cur[0], 0);
    store_tile(0);
  }
  // Everything loaded so far (the Q fragments above all) has landed before the loop starts.  Without
  // this the compiler must assume those loads may still be in flight at the loop head and, the vector
  // memory counter being in-order, makes the first MFMA of EVERY iteration wait for that iteration's
  // own prefetch loads.
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();

  const int wq_last = wq0 + 31;
  // One kv tile.  BUFc: the buffer index as a constant, or (-1) taken at run time.
  // wave-uniform decisions: nothing to do above the diagonal or outside the rows' segments; element masks
  // only on tiles that straddle the diagonal, the tail, or a segment boundary
  auto iteration = [&](auto BUFc, const int it) {
    const int buf = decltype(BUFc)::value >= 0 ? decltype(BUFc)::value : (it & 1);
    const i32x4 after = entry(it + 2);
    const int t = cur[0];
    const int kv0 = t * BN;
    const bool has_next = it + 1 < nact;
    const int t_next = has_next ? nxt[0] : t;
    bool skip = CAUSAL && (kv0 > wq_last + band_hi || kv0 + BN - 1 < wq0 - band_lo);
    bool need_mask = (kv0 + BN > Skv) || (CAUSAL && (kv0 + BN - 1 > wq0 + band_hi || kv0 < wq_last - band_lo));
    if (SEG) {
      const int lo = cur[1], hi = cur[2];
      skip = skip || hi < wqmin || lo > wqmax;
      need_mask = need_mask || !(lo == hi && wqmin == wqmax && lo == wqmin);
    }
    if (skip) {
      if (has_next) {
        load_tile(t_next, buf ^ 1);
        store_tile(buf ^ 1);
      }
    } else if (need_mask) {
      tile_body(std::true_type{}, BUFc, buf, t, has_next, t_next);
    } else {
      tile_body(std::false_type{}, BUFc, buf, t, has_next, t_next);
    }
    __syncthreads();
    cur = nxt;
    nxt = scalars(after);
  };
  if constexpr (STATIC_BUF) {
    // the plain causal kernel: the loop alternates two copies of the body, one per buffer
    for (int it = 0; it < nact; it += 2) {
      iteration(std::integral_constant<int, 0>{}, it);
      if (it + 1 < nact) iteration(std::integral_constant<int, 1>{}, it + 1);
    }
  } else {
    // The masked variants have no registers to spare for two copies: with segment ids the two-copy loop spills, and a
    // reload from scratch waits, the memory counter being in-order, for the tile loads issued before it.  (Their loop
    // body is written out here:
    // routed through the closure above, the compiler keeps part of the captured state in scratch memory.)
    for (int it = 0; it < nact; it++) {
      const int buf = it & 1;
      const i32x4 after = entry(it + 2);
      const int t = cur[0];
      const int kv0 = t * BN;
      const bool has_next = it + 1 < nact;
      const int t_next = has_next ? nxt[0] : t;
      bool skip = CAUSAL && (kv0 > wq_last + band_hi || kv0 + BN - 1 < wq0 - band_lo);
      bool need_mask = (kv0 + BN > Skv) || (CAUSAL && (kv0 + BN - 1 > wq0 + band_hi || kv0 < wq_last - band_lo));
      if (SEG) {
        const int lo = cur[1], hi = cur[2];
        skip = skip || hi < wqmin || lo > wqmax;
        need_mask = need_mask || !(lo == hi && wqmin == wqmax && lo == wqmin);
      }
      if (ext) {
        // outside every row's band: nothing to do; not inside every row's band (or a soft cap): element-wise path
        skip = skip || kv0 > wpmax + a.mx.hi_off || kv0 + BN - 1 < wpmin - a.mx.lo_off;
        need_mask = need_mask || capped || biased || !(kv0 >= wpmax - a.mx.lo_off && kv0 + BN - 1 <= wpmin + a.mx.hi_off);
      }
      typedef std::integral_constant<int, -1> RT;
      if (skip) {
        if (has_next) {
          load_tile(t_next, buf ^ 1);
          store_tile(buf ^ 1);
        }
      } else if (need_mask) {
        tile_body(std::true_type{}, RT{}, buf, t, has_next, t_next);
      } else {
        tile_body(std::false_type{}, RT{}, buf, t, has_next, t_next);
      }
      __syncthreads();
      cur = nxt;
      nxt = scalars(after);
    }
  }

  // (the last tile's body issues its loads without a successor to wait for them: no LDS-writing load may be in flight
  // when the workgroup's LDS is handed to the next one)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // ---- epilogue: normalise, write O (row = query, 4 consecutive v-dims per store) and LSE
  T* ob = (T*)a.out + b * a.os[0] + h * a.os[1];
  float* lb = a.lse + ((int64_t)b * a.Hq + h) * Sq;
  {
    const float l = half_sum(l_run);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    if (qrow < Sq) {
      if (g == 0) lb[qrow] = l > 0.f ? (m_run + log2f(l)) * LN2 : -INFINITY;
      T* op = ob + qrow * a.os[2];
#pragma unroll
      for (int d = 0; d < DVB; d++)
#pragma unroll
        for (int vq = 0; vq < 4; vq++) {
          const f32x16& o = oacc[d];
          *(u32x2*)(op + d * 32 + 8 * vq + 4 * g) =
              pack4<T>(o[4 * vq] * inv, o[4 * vq + 1] * inv, o[4 * vq + 2] * inv, o[4 * vq + 3] * inv);
        }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------------------
template <typename T, int DQK, int DV, bool CAUSAL, bool SEG>
static int launch_fwd(const FwdArgs& a, int B, hipStream_t st) {
  constexpr int BN = 64, BM = 128;
  constexpr int BUF = DmaTile<DQK>::BYTES + DmaTile<DV>::BYTES + (SEG ? BN * 4 : 0);
  const int ntiles_max = (a.Skv + BN - 1) / BN;
  const size_t smem = 2 * (size_t)BUF + (SEG ? (size_t)16 * ntiles_max : 0);  // (the id ranges borrow the tile buffers)
  TP_REQUIRE(smem <= 160 * 1024 && (!SEG || (size_t)(2 * ntiles_max + 16) * 4 <= 2 * (size_t)BUF), TP_ERR_UNSUPPORTED, "tp_attn_fwd: Skv=%d needs %zu bytes of LDS (max 163840)", a.Skv, smem);
  auto kern = attn_fwd_kernel<T, DQK, DV, CAUSAL, SEG>;
  static bool attr_set = false;  // benign race: every thread sets the same value
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    TP_REQUIRE(e == hipSuccess, TP_ERR_LAUNCH, "tp_attn_fwd: hipFuncSetAttribute failed: %s", hipGetErrorString(e));
    attr_set = true;
  }
  const dim3 grid(xcd_grid((a.Sq + BM - 1) / BM, a.n_rep, B * a.Hkv)), block(256);
  kern<<<grid, block, smem, st>>>(a);
  return check_launch("tp_attn_fwd");
}

template <typename T, int DQK, int DV>
static int dispatch_fwd(const FwdArgs& a, int B, int causal, hipStream_t st) {
  if (a.mx.on) {
    if (band_only(a.mx)) {
      // a window and / or a causal offset and nothing else: the causal kernels, with that band instead of (-inf, 0]
      FwdArgs b = a;
      b.band_lo = a.mx.lo_off;
      b.band_hi = a.mx.hi_off;
      b.mx = no_mask_ext();
      if (a.seg) return launch_fwd<T, DQK, DV, true, true>(b, B, st);
      return launch_fwd<T, DQK, DV, true, false>(b, B, st);
    }
    // the other mask extensions: the general instantiation (causality is part of the band then)
    return launch_fwd<T, DQK, DV, false, true>(a, B, st);
  }
  if (causal) {
    if (a.seg) return launch_fwd<T, DQK, DV, true, true>(a, B, st);
    return launch_fwd<T, DQK, DV, true, false>(a, B, st);
  }
  // no causality and no mask extension: the causal kernels with a band that covers every key.  (The instantiation
  // without causality ran the same tiles 1.8 times slower at the benchmark's shape, 5.03 against 2.76 ms, with bit-identical
  // results; with segment ids it is the general instantiation, which is sized for correctness.)
  FwdArgs b = a;
  b.band_lo = BAND_INF;
  b.band_hi = BAND_INF;
  if (a.seg) return launch_fwd<T, DQK, DV, true, true>(b, B, st);
  return launch_fwd<T, DQK, DV, true, false>(b, B, st);
}

// fp32 operands: attn_fwd_f32.hip
int attn_fwd_f32(const void* q, const void* k, const void* v, const int32_t* seg, void* out, float* lse, int B, int Hq, int Hkv,
                 int Sq, int Skv, int Dqk, int Dv, const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                 float sm_scale, int causal, hipStream_t st, const MaskExt& mx);

}  // namespace tp

using namespace tp;

static int attn_fwd_impl(const void* q, const void* k, const void* v, const int32_t* seg, void* out, float* lse,
                         int B, int Hq, int Hkv, int Sq, int Skv, int Dqk, int Dv, const int64_t q_strides[3],
                         const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3],
                         float sm_scale, int causal, int dtype, void* stream, const MaskExt& mx) {
  TP_REQUIRE(q && k && v && out && lse && q_strides && k_strides && v_strides && o_strides, TP_ERR_BAD_ARG,
             "tp_attn_fwd: null pointer");
  TP_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Sq > 0 && Skv > 0, TP_ERR_BAD_ARG, "tp_attn_fwd: non-positive size");
  TP_REQUIRE(Hq % Hkv == 0, TP_ERR_BAD_ARG, "tp_attn_fwd: Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  TP_REQUIRE(!seg || Sq == Skv, TP_ERR_BAD_ARG, "tp_attn_fwd: segment ids need Sq == Skv (got %d, %d)", Sq, Skv);
  TP_REQUIRE(sm_scale > 0.f, TP_ERR_BAD_ARG, "tp_attn_fwd: sm_scale must be positive");
  if (dtype == TP_F32)
    return attn_fwd_f32(q, k, v, seg, out, lse, B, Hq, Hkv, Sq, Skv, Dqk, Dv, q_strides, k_strides, v_strides, o_strides, sm_scale,
                        causal, (hipStream_t)stream, mx);
  TP_REQUIRE(dtype == TP_BF16 || dtype == TP_F16, TP_ERR_UNSUPPORTED, "tp_attn_fwd: dtype %d (bf16, fp16 and fp32 only)", dtype);
  TP_REQUIRE((int64_t)(B + 8) * Hq * ((Sq + 127) / 128) < (1ll << 31), TP_ERR_UNSUPPORTED, "tp_attn_fwd: too many workgroups");
  FwdArgs a;
  a.q = q; a.k = k; a.v = v; a.seg = seg; a.out = out; a.lse = lse;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.Sq = Sq; a.Skv = Skv; a.n_rep = Hq / Hkv;
  bool ok = aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out);
  for (int i = 0; i < 3; i++) {
    a.qs[i] = q_strides[i]; a.ks[i] = k_strides[i]; a.vs[i] = v_strides[i]; a.os[i] = o_strides[i];
    ok = ok && q_strides[i] % 8 == 0 && k_strides[i] % 8 == 0 && v_strides[i] % 8 == 0 && o_strides[i] % 4 == 0;
  }
  TP_REQUIRE(ok, TP_ERR_BAD_ARG, "tp_attn_fwd: pointers and strides must keep rows 16-byte aligned");
  // tiles are addressed with 32-bit byte offsets inside one (batch, head) slice
  TP_REQUIRE(k_strides[2] > 0 && v_strides[2] > 0, TP_ERR_BAD_ARG, "tp_attn_fwd: k / v sequence strides must be positive");
  TP_REQUIRE(((int64_t)Skv * k_strides[2] + Dqk) * 2 < (1ll << 31) && ((int64_t)Skv * v_strides[2] + Dv) * 2 < (1ll << 31),
             TP_ERR_UNSUPPORTED, "tp_attn_fwd: one (batch, head) slice of k or v spans 2 GiB or more");
  a.scale_log2 = sm_scale * LOG2E;
  a.mx = mx;
  a.band_lo = BAND_INF;  // plain causality (used by the causal kernels only)
  a.band_hi = 0;
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

extern "C" int tp_attn_fwd(const void* q, const void* k, const void* v, const int32_t* seg, void* out, float* lse,
                           int B, int Hq, int Hkv, int Sq, int Skv, int Dqk, int Dv, const int64_t q_strides[3],
                           const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3],
                           float sm_scale, int causal, int dtype, void* stream) {
  return attn_fwd_impl(q, k, v, seg, out, lse, B, Hq, Hkv, Sq, Skv, Dqk, Dv, q_strides, k_strides, v_strides, o_strides, sm_scale,
                       causal, dtype, stream, no_mask_ext());
}

extern "C" int tp_attn_fwd_masked(const void* q, const void* k, const void* v, const int32_t* seg, const int32_t* q_positions,
                                  void* out, float* lse, int B, int Hq, int Hkv, int Sq, int Skv, int Dqk, int Dv,
                                  const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                                  const int64_t o_strides[3], float sm_scale, int causal, int causal_offset, int window_left,
                                  int window_right, float logits_soft_cap, int dtype, void* stream) {
  TP_REQUIRE(sm_scale > 0.f, TP_ERR_BAD_ARG, "tp_attn_fwd_masked: sm_scale must be positive");
  TP_REQUIRE(window_left < BAND_INF && window_right < BAND_INF && causal_offset > -BAND_INF && causal_offset < BAND_INF, TP_ERR_BAD_ARG,
             "tp_attn_fwd_masked: window or offset out of range");
  return attn_fwd_impl(q, k, v, seg, out, lse, B, Hq, Hkv, Sq, Skv, Dqk, Dv, q_strides, k_strides, v_strides, o_strides, sm_scale,
                       causal, dtype, stream,
                       make_mask_ext(q_positions, causal, causal_offset, window_left, window_right, logits_soft_cap, sm_scale));
}

extern "C" int tp_attn_fwd_biased(const void* q, const void* k, const void* v, const int32_t* seg, const int32_t* q_positions,
                                  const float* bias, const int64_t bias_strides[3], void* out, float* lse, int B, int Hq,
                                  int Hkv, int Sq, int Skv, int Dqk, int Dv, const int64_t q_strides[3],
                                  const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3],
                                  float sm_scale, int causal, int causal_offset, int window_left, int window_right,
                                  float logits_soft_cap, int dtype, void* stream) {
  TP_REQUIRE(sm_scale > 0.f, TP_ERR_BAD_ARG, "tp_attn_fwd_biased: sm_scale must be positive");
  TP_REQUIRE(window_left < BAND_INF && window_right < BAND_INF && causal_offset > -BAND_INF && causal_offset < BAND_INF, TP_ERR_BAD_ARG,
             "tp_attn_fwd_biased: window or offset out of range");
  TP_REQUIRE(bias && bias_strides, TP_ERR_BAD_ARG, "tp_attn_fwd_biased: null bias");
  TP_REQUIRE(bias_strides[0] >= 0 && bias_strides[1] >= 0 && bias_strides[2] >= 0, TP_ERR_BAD_ARG,
             "tp_attn_fwd_biased: negative bias stride");
  return attn_fwd_impl(q, k, v, seg, out, lse, B, Hq, Hkv, Sq, Skv, Dqk, Dv, q_strides, k_strides, v_strides, o_strides, sm_scale,
                       causal, dtype, stream,
                       make_mask_ext(q_positions, causal, causal_offset, window_left, window_right, logits_soft_cap, sm_scale, bias,
                                     bias_strides));
}
