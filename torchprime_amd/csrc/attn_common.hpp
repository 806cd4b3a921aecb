// Shared pieces of the attention kernels: MFMA wrappers, fragment packing, LDS tile layouts.
//
// MFMA operand layouts used throughout (v_mfma_f32_32x32x16_{bf16,f16}, wave64; ln = lane % 32,
// g = lane / 32):
//   A (32 x 16): lane holds row ln,    k = 8*g + 0..7
//   B (16 x 32): lane holds column ln, k = 8*g + 0..7
//   C (32 x 32): lane holds column ln, rows 8*(v/4) + 4*g + v%4 for v = 0..15
// The hardware pairs A and B element-for-element inside a lane group g, so any ordering of the 16
// k-values works as long as both operands use the same one.  The kernels exploit that when a C tile
// (lane <-> column) is fed back as a B operand: its values v = 8h..8h+7 cover rows
// 16h + 8a + 4g + e (a = 0..1, e = 0..3), and the other operand is laid out in LDS so that a lane's
// 16 bytes hold exactly those rows ("quad-swapped" order, see vt_offset).
#pragma once
#include <type_traits>

#include "common.hpp"

namespace tp {

// compile-time loop: f(std::integral_constant<int, B>{}), ..., f(std::integral_constant<int, E - 1>{})
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    static_for<B + 1, E>(f);
  }
}


template <typename T> struct MT;
template <> struct MT<bf16_t> {
  typedef bf16x8 v8;
  typedef bf16x2 v2;
  static __device__ __forceinline__ f32x16 mfma32(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // c += a b with the accumulator pinned to the accumulation registers (see mfma32_acc below)
  static __device__ __forceinline__ void mfma32_acc(f32x16& c, v8 a, v8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma32_acc_guarded(f32x16& c, v8 a, v8 b) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
template <> struct MT<f16_t> {
  typedef f16x8 v8;
  typedef f16x2 v2;
  static __device__ __forceinline__ f32x16 mfma32(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ void mfma32_acc(f32x16& c, v8 a, v8 b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma32_acc_guarded(f32x16& c, v8 a, v8 b) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
// mfma32_acc: long-lived accumulators that only MFMAs touch inside a loop (dK, dV) are kept in the
// accumulation half of the register file by writing the instruction out with an "a" constraint.  With the
// compiler's own MFMA form every result sits in the 256 architectural VGPRs, which then cannot also hold
// the K/V fragments, and each fragment is copied out of an AGPR right before the MFMA that needs it.
// What the compiler no longer sees, and the callers guarantee: the same accumulator is reused by a later
// mfma32_acc only (exactly overlapping destination, for which the matrix unit forwards), and it is read
// by ordinary instructions only after the loop and a barrier, hundreds of cycles after the last MFMA.
// One more thing the compiler does for its own MFMAs and not for these: an A/B operand register written by a
// vector-ALU instruction needs two wait states before a matrix instruction reads it (the packed P / dS operands
// are such registers).  mfma32_acc leaves that distance to the caller's hand-placed schedule;
// mfma32_acc_guarded carries the two wait states itself, for code whose order is left to the compiler.

// eight floats -> one 16-byte MFMA operand (round to nearest even)
template <typename T>
__device__ __forceinline__ typename MT<T>::v8 pack8(float a0, float a1, float a2, float a3, float a4, float a5,
                                                    float a6, float a7) {
  typename MT<T>::v8 r;
  r[0] = (T)a0; r[1] = (T)a1; r[2] = (T)a2; r[3] = (T)a3;
  r[4] = (T)a4; r[5] = (T)a5; r[6] = (T)a6; r[7] = (T)a7;
  return r;
}
// four floats -> 8 bytes
template <typename T>
__device__ __forceinline__ u32x2 pack4(float a0, float a1, float a2, float a3) {
  typedef T v4 __attribute__((ext_vector_type(4)));
  v4 r;
  r[0] = (T)a0; r[1] = (T)a1; r[2] = (T)a2; r[3] = (T)a3;
  return __builtin_bit_cast(u32x2, r);
}

// Combine a value with the one held by the partner lane (lane ^ 32): max / sum across the two
// half-waves.  v_permlane32_swap(old, src) returns x = {old.lo, src.lo}, y = {old.hi, src.hi}; with
// old = src = v every lane gets its own half's value in one of x / y and the partner's in the other.
// The elements are copied to scalars before the bit casts: __builtin_bit_cast applied directly to a
// vector element expression (r.y) reads element 0 with this compiler.
__device__ __forceinline__ void half_swap(float v, float& lo, float& hi) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  const u32x2 r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned x = r.x, y = r.y;
  lo = __builtin_bit_cast(float, x);
  hi = __builtin_bit_cast(float, y);
}
__device__ __forceinline__ float half_max(float v) {
  float lo, hi;
  half_swap(v, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float half_sum(float v) {
  float lo, hi;
  half_swap(v, lo, hi);
  return lo + hi;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

// tanh(x) = 1 - 2 / (exp(2x) + 1); saturates cleanly (exp -> inf gives 1, exp -> 0 gives -1)
__device__ __forceinline__ float fast_tanh(float x) {
  const float e = fast_exp2(x * (2.f * LOG2E));
  return 1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f);
}

// ---- mask extensions -------------------------------------------------------------------------------
// Beyond causal / full and segment ids the functional API names three more things
// (torchprime/utils/kernel_utils.py:259-294, torchprime/utils/parallelism_utils.py:87-152): a sliding window
// (LocalMask), a soft cap on the logits, and a causal mask whose query rows are in another order than the keys
// (LoadBalancedCausalMask: row i stands for position q_sequence[i]).  All three are a band per query row,
//     allowed(i, j)  <=>  qp(i) - lo_off <= j <= qp(i) + hi_off,     qp(i) = qpos ? qpos[i] : i,
// (causal: hi_off = offset, no window: the offsets are BAND_INF) plus s <- cap_out * tanh(s * cap_in) on the raw
// scores.  Only the <non-causal, segment ids> instantiation of each kernel evaluates them (the host routes every
// call that uses one there, with or without segment ids), so the other instantiations carry none of this.
constexpr int BAND_INF = 1 << 29;
struct MaskExt {
  const int32_t* qpos;
  int lo_off, hi_off;
  float cap_in, cap_out;  // 0: no soft cap
  // additive mask: bias[b * bias_s[0] + h * bias_s[1] + q * bias_s[2] + kv] is added to the scaled (and capped)
  // logit of (query row q, key kv) of query head h; a broadcast axis has stride 0; -inf forbids the pair
  const float* bias;
  int64_t bias_s[3];
  float bias_mul;  // 1 / softmax scale: the kernels that add the bias before scaling multiply by this
  int on;
};
// window_left / window_right < 0: unbounded on that side; soft_cap <= 0: none
inline MaskExt make_mask_ext(const int32_t* q_positions, int causal, int causal_offset, int window_left, int window_right,
                             float soft_cap, float sm_scale, const float* bias = nullptr, const int64_t* bias_strides = nullptr) {
  MaskExt m;
  m.qpos = q_positions;
  const int hi_c = causal ? causal_offset : BAND_INF, hi_w = window_right >= 0 ? window_right : BAND_INF;
  m.hi_off = hi_c < hi_w ? hi_c : hi_w;
  m.lo_off = window_left >= 0 ? window_left : BAND_INF;
  m.cap_in = soft_cap > 0.f ? sm_scale / soft_cap : 0.f;
  m.cap_out = soft_cap > 0.f ? soft_cap / sm_scale : 0.f;
  m.bias = bias;
  for (int i = 0; i < 3; i++) m.bias_s[i] = bias && bias_strides ? bias_strides[i] : 0;
  m.bias_mul = 1.f / sm_scale;
  m.on = (q_positions != nullptr || window_left >= 0 || window_right >= 0 || soft_cap > 0.f || (causal && causal_offset != 0) ||
          bias != nullptr) ? 1 : 0;
  return m;
}
// a band of key positions around the row's own index and nothing else (no per-row positions, soft cap or additive
// mask): the causal kernels evaluate it themselves
inline bool band_only(const MaskExt& m) { return m.on && !m.qpos && m.cap_in == 0.f && !m.bias; }
inline MaskExt no_mask_ext() {
  MaskExt m;
  m.qpos = nullptr; m.lo_off = BAND_INF; m.hi_off = BAND_INF; m.cap_in = 0.f; m.cap_out = 0.f; m.on = 0;
  m.bias = nullptr; m.bias_s[0] = m.bias_s[1] = m.bias_s[2] = 0; m.bias_mul = 1.f;
  return m;
}

// ---- buffer loads ---------------------------------------------------------------------------------
// K/V/Q/dO tiles are fetched with raw buffer loads: the per-thread byte offset inside a tile is computed
// once, the tile's offset is a scalar, so the per-tile address arithmetic is free, and rows past the end
// of the tensor (offset >= num_records) read as zero instead of needing a clamp per row.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load16(rsrc_t r, unsigned voffset, unsigned soffset) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, (int)voffset, (int)soffset, 0);
}
// bytes spanned by `rows` rows of `row_elems` 16-bit elements at a row stride of `stride` elements
__device__ __forceinline__ unsigned span_bytes(int rows, int64_t stride, int row_elems) {
  return (unsigned)(((int64_t)(rows - 1) * stride + row_elems) * 2);
}

// ---- workgroup -> work mapping ---------------------------------------------------------------------
// The 256 CUs sit in 8 XCDs with one L2 each, and workgroups of a 1-D grid are handed to the XCDs round
// robin by linear id.  Work is therefore numbered so that every workgroup that streams the same K/V (or
// Q/dO) slice - one (batch, kv head) "group" - lands on the same XCD and runs at about the same time:
//     id = (group_local * per_group + r) * 8 + xcd,   group = group_local * 8 + xcd,
//     r  = tile * n_inner + inner   (tiles outer so the heaviest tiles start first).
// Returns false for the padding ids of a group count that is not a multiple of 8.
constexpr int NUM_XCD = 8;
__device__ __forceinline__ bool xcd_map(int n_tiles, int n_inner, int n_groups, int& tile, int& inner, int& group) {
  const int n = blockIdx.x;
  const int xcd = n % NUM_XCD, slot = n / NUM_XCD;
  const int per_group = n_tiles * n_inner;
  const int gl = slot / per_group, r = slot - gl * per_group;
  group = gl * NUM_XCD + xcd;
  tile = r / n_inner;
  inner = r - tile * n_inner;
  return group < n_groups;
}
inline unsigned xcd_grid(int n_tiles, int n_inner, int n_groups) {
  return (unsigned)(NUM_XCD * ((n_groups + NUM_XCD - 1) / NUM_XCD) * n_tiles * n_inner);
}

// Per-tile [min, max] of the segment ids of the 64-row tiles t0..t1-1, into LDS.  One thread per tile: its 64
// ids are independent loads in flight together (a lane-per-row reduction waits out one load and twelve
// shuffles per tile, which for short documents took longer than the tiles' own work).  Rows past S repeat the
// last id.
__device__ __forceinline__ void seg_tile_ranges(const int32_t* segb, int S, int t0, int t1, int* tmin, int* tmax,
                                                int tid, int nthreads) {
  const bool vec = (((size_t)segb) & 15) == 0;
  for (int t = t0 + tid; t < t1; t += nthreads) {
    const int base = t * 64;
    int lo, hi;
    if (vec && base + 64 <= S) {
      const int4* p = (const int4*)(segb + base);
      int4 v = p[0];
      lo = min(min(v.x, v.y), min(v.z, v.w));
      hi = max(max(v.x, v.y), max(v.z, v.w));
#pragma unroll
      for (int i = 1; i < 16; i++) {
        v = p[i];
        lo = min(min(lo, v.x), min(min(v.y, v.z), v.w));
        hi = max(max(hi, v.x), max(max(v.y, v.z), v.w));
      }
    } else {
      lo = hi = segb[min(base, S - 1)];
      for (int i = 1; i < 64; i++) {
        const int v = segb[min(base + i, S - 1)];
        lo = min(lo, v);
        hi = max(hi, v);
      }
    }
    tmin[t - t0] = lo;
    tmax[t - t0] = hi;
  }
}

// ---- LDS layouts ---------------------------------------------------------------------------------
// Row-major tile [rows][D] of 16-bit elements: rows padded by 16 bytes so that 16-byte reads by lanes
// in consecutive rows land in different banks.
template <int D> struct RowTile {
  static constexpr int STRIDE = D * 2 + 16;  // bytes
  static __device__ __forceinline__ int off(int row, int elem) { return row * STRIDE + elem * 2; }
};

// Transposed tile [C columns][R rows-as-contraction-index] of 16-bit elements, R = 64: the element of
// source row r (0..63) and column c lives in LDS row c.  Within each group of 16 source rows the
// quads are stored in the order [0-3, 8-11, 4-7, 12-15] so that 16-byte chunk (2*ks + g) of LDS row c
// holds source rows 16ks + {4g..4g+3, 8+4g..8+4g+3}: exactly what lane group g needs as the k-values
// of an MFMA operand whose partner is a C tile converted in registers.  Chunks are XOR-swizzled by the
// column so reads (lanes = consecutive columns) are bank-conflict free.
struct TrTile64 {
  static constexpr int ROW_BYTES = 128;
  static __device__ __forceinline__ int swz(int c) { return ((c >> 1) ^ (c >> 4)) & 7; }
  // byte offset of the 16-byte chunk for k-step ks (16 source rows) and lane group g, column c
  static __device__ __forceinline__ int chunk_off(int c, int ks, int g) {
    return c * ROW_BYTES + (((2 * ks + g) ^ swz(c)) << 4);
  }
  // byte offset at which the four values of source rows 4*rq..4*rq+3 (rq = 0..15), column c, are
  // written as one 8-byte store
  static __device__ __forceinline__ int quad_off(int c, int rq) {
    return c * ROW_BYTES + (((2 * (rq >> 2) + (rq & 1)) ^ swz(c)) << 4) + (((rq >> 1) & 1) << 3);
  }
};

// 4 x 8 block of 16-bit values held as four u32x4 rows -> column j (0..7) as 4 consecutive 16-bit
// values (rows 0..3) packed into 8 bytes
__device__ __forceinline__ u32x2 transpose_col(const u32x4 (&r)[4], int j) {
  const unsigned sel = (j & 1) ? 0x07060302u : 0x05040100u;
  const int w = j >> 1;
  u32x2 o;
  o.x = __builtin_amdgcn_perm(r[1][w], r[0][w], sel);
  o.y = __builtin_amdgcn_perm(r[3][w], r[2][w], sel);
  return o;
}

// ------------------------------------------------------------------------------------------------
// row-major tiles filled by buffer loads that write LDS directly (no staging registers)
// ------------------------------------------------------------------------------------------------
// One such load moves 16 bytes per lane to LDS address  base + 16 * lane: where a chunk lands is fixed by
// the lane, which global chunk it carries is free.  A tile of 64 rows x D 16-bit elements is stored
// densely (row r at r * D*2) with the 16-byte chunks of a row XOR-swizzled by the row, so that the MFMA
// fragment reads (lanes = consecutive rows, same logical chunk) fall into different banks.
// ROT picks the swizzle that also serves transposing reads (ds_read_b64_tr_b16) of the same tile: such a read
// takes, per 32 lanes, a patch of 4 rows x 64 bytes, so the four rows of a quad must differ in the bits that select
// the 64-byte quarter of the 256-byte bank line; the row's low bits go to the swizzle's high bits for that.  Both
// swizzles are a permutation of the chunk positions over any 16 consecutive rows (fragment reads stay conflict free).
template <int D, bool ROT = false>
struct DmaTile {
  static constexpr int CPR = D / 8;              // 16-byte chunks per row
  static constexpr int ROWB = D * 2;             // bytes per row
  static constexpr int BYTES = 64 * ROWB;
  static constexpr int PER_WAVE = CPR / 4;       // load instructions per wave for one tile (4 waves)
  static_assert(CPR % 8 == 0, "head dim must be a multiple of 64");
  static __device__ __forceinline__ int swz(int row) {
    if constexpr (ROT) return (CPR % 16 == 0) ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
    else return (CPR % 16 == 0) ? (row & 15) : ((row >> 1) & 7);
  }
  // byte offset of logical chunk c of a row
  static __device__ __forceinline__ int off(int row, int c) { return row * ROWB + ((c ^ swz(row)) << 4); }
  // Transposing read of the patch rows r0..r0+3 (r0 a multiple of 4) x columns 16 cb..16 cb + 15 by a group of 16
  // lanes: lane 4 e + m of the group supplies the address of (row r0 + e, columns 16 cb + 4 m ..+3), and receives
  // the four values (rows r0..r0+3) of column 16 cb + its own index in the group.  Byte offset inside the tile:
  static __device__ __forceinline__ int tr_off(int r0, int cb, int lane16) {
    static_assert(ROT || D == 0, "transposing reads need the rotated swizzle");
    const int row = r0 + (lane16 >> 2), col = 16 * cb + 4 * (lane16 & 3);
    return row * ROWB + (((col >> 3) ^ swz(row)) << 4) + (col & 7) * 2;
  }

  unsigned vo[PER_WAVE];  // global byte offset (inside a tile) of the chunk this lane carries, per instruction

  __device__ __forceinline__ void init(int64_t row_stride, int wave, int lane) {
#pragma unroll
    for (int i = 0; i < PER_WAVE; i++) {
      const int slot = (wave * PER_WAVE + i) * 64 + lane;  // 16-byte slot inside the LDS tile
      const int row = slot / CPR, c = (slot % CPR) ^ swz(row);
      vo[i] = (unsigned)((row * row_stride + c * 8) * 2);
    }
  }
  // Issue this wave's share of the tile.  The loads are written as assembly on purpose: the compiler
  // orders every later LDS read behind an LDS-writing load it knows of, which would stall the tile being
  // computed on the one in flight; the caller waits (s_waitcnt 0 + barrier) before the tile is read.
  // Rows past the end of the tensor (offset >= rs.z) arrive as zeros.
  template <int I>
  __device__ __forceinline__ void issue_one(u32x4 rs, unsigned tile_byte_offset, unsigned char* lds_tile, int wave) const {
    const unsigned dst = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lds_tile + (wave * PER_WAVE + I) * 1024));
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(dst), "v"(vo[I]), "s"(rs), "s"(tile_byte_offset) : "memory", "m0");
  }
  // same, with the wave's first LDS destination given as a scalar byte address (keeps the address
  // arithmetic on the scalar unit)
  template <int I>
  __device__ __forceinline__ void issue_one_at(u32x4 rs, unsigned tile_byte_offset, unsigned wave_dst) const {
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(wave_dst + I * 1024), "v"(vo[I]), "s"(rs), "s"(tile_byte_offset) : "memory", "m0");
  }
  __device__ __forceinline__ void issue(u32x4 rs, unsigned tile_byte_offset, unsigned char* lds_tile, int wave) const {
    tile_byte_offset = __builtin_amdgcn_readfirstlane(tile_byte_offset);
    if constexpr (PER_WAVE > 0) issue_one<0>(rs, tile_byte_offset, lds_tile, wave);
    if constexpr (PER_WAVE > 1) issue_one<1>(rs, tile_byte_offset, lds_tile, wave);
    if constexpr (PER_WAVE > 2) issue_one<2>(rs, tile_byte_offset, lds_tile, wave);
    if constexpr (PER_WAVE > 3) issue_one<3>(rs, tile_byte_offset, lds_tile, wave);
    if constexpr (PER_WAVE > 4) issue_one<4>(rs, tile_byte_offset, lds_tile, wave);
    if constexpr (PER_WAVE > 5) issue_one<5>(rs, tile_byte_offset, lds_tile, wave);
    static_assert(PER_WAVE <= 6, "head dim above 192");
  }
};
// two transposing reads -> one 16-byte MFMA operand: values 0..3 from the first address, 4..7 from the second
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) unsigned char lds_byte;
template <typename V8>
__device__ __forceinline__ V8 tr_read8(const lds_byte* p0, const lds_byte* p1) {
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p0);
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p1);
  const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(V8, v);
}
// buffer resource words for the assembly loads: base, stride 0, size in bytes, raw-buffer flags
__device__ __forceinline__ u32x4 make_rsrc_words(const void* base, unsigned bytes) {
  const unsigned long long p = (unsigned long long)base;
  u32x4 r;
  r.x = __builtin_amdgcn_readfirstlane((unsigned)p);
  r.y = __builtin_amdgcn_readfirstlane((unsigned)(p >> 32));
  r.z = __builtin_amdgcn_readfirstlane(bytes);
  r.w = 0x00020000u;
  return r;
}

}  // namespace tp
