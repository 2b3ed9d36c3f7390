// Decode attention over packed KV on the gfx950 matrix cores: the split pass of split-K.
//
// One wavefront (64 lanes) per workgroup walks a range of 128-token tiles of one (batch row,
// kv head) and leaves an un-normalised partial (running max, running sum, output) per query head.
//
// Formulation.  With lane = 16*kg + n, v_mfma_f32_16x16x32_f16 takes A[row n][k 8kg..8kg+7],
// B[k 8kg..8kg+7][col n] and returns C[rows 4kg..4kg+3][col n].  Both products are computed
// transposed so that the accumulator of the first is, lane for lane, the B operand of the second:
//
//   S^T[token][col] = sum_ch  code[token][ch]            * (q[col][ch] * scale_k[ch])     (QK)
//   O^T[ch][col]    = sum_tok code[tok][ch]               * (p[tok][col] * scale_v[tok])   (PV)
//
// The 16 columns hold the G query heads of the kv head, replicated (col n -> head n % G; with at
// most 8 heads col n -> head (n % 8) % G, and columns 8..15 carry the low-order part of the QK
// operand, see qk_packed).  The zero points never touch the codes: sum_ch q*zero_k and
// sum_tok p*zero_v are one more small matrix product each.
// With at most 4 heads per kv head every head sits in at least four columns; each of the four then
// does the softmax and feeds PV for a quarter of a page's tokens only (see combine_quarter).
// In that case the q * scale operands of a page are not computed by every lane for itself but once
// per page into an LDS table, and the high plane's operands are scattered to their slots (see
// qk_packed_tab).
//
// Codes as operands.  A 32-bit word of a packed plane holds 16 two-bit codes of ONE row (K: one
// channel, 16 tokens; V: one token, 16 channels) but an MFMA register must hold two consecutive k
// (K: two channels, V: two tokens) of one row of A: X = [8 codes of row r | 8 codes of row r+1].
// With the tile in LDS one transposing read (ds_read_b64_tr_b16: a 16-lane block reads 4 plane
// rows, lane i receives 16-bit piece i of each) delivers two such registers; with the tile in
// registers lanes n and n^1 each load one word of two neighbouring plane rows, swap them with one
// DPP move and v_perm the matching 16-bit halves together.  `X & (3 << 2u | 3 << 2u+16)` is then
// already a valid operand: fp16 SUBNORMALS code * 4^u * 2^-24 (the matrix cores do not flush
// them), so unpacking costs one v_and_b32 per register and the factor is undone per tile after
// the contraction.  Codes above bit 9 are reached through X >> 10.
//
// Index maps (all bijections chosen so that every load is 64 contiguous bytes per 16 lanes):
//   K: lane n keeps tokens 8n .. 8n+7 of every plane row it touches; MFMA tile u (0..7) = tokens
//     {8n + u}; k-slot (kg, 2pi + h) of the 32-channel chunk kc = channel 32kc + krow(pi, kg) + h
//     with krow = 16 (pi>>1) + 4kg + 2 (pi&1): the four rows of a transposing read are consecutive.
//   C[u][j] of lane (kg, n) = token 32kg + 8j + u, column n.
//   V plane rows are tokens: lane group kg owns rows 32kg .. 32kg+31 (its own tokens), k-chunk j
//   = rows 32kg + 8j .. +7, d-tile u = channels {8n + u}; O^T[u][j] = channel 32kg + 8j + u.
#include <algorithm>
#include <type_traits>

#include <hip/hip_ext.h>

#include "decode_common.h"

// Wave priority while a phase is dominated by matrix instructions / by vector instructions: the
// wave that feeds the matrix pipe wins arbitration, the other one fills the gaps (worth ~2 %; one
// level of difference, not two: at 2 / 0 the kernel is 1-2 % slower, at 3 / 0 4 %, at equal levels 2 %).
#define KITTY_PRIO_MFMA 1
#define KITTY_PRIO_VALU 0

namespace kitty {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.44269504088896340736f;
constexpr int kQPad = 136;   // q_nat row length in halves: 128 channels + a zero entry at 128

// A packed K page-head as it sits in LDS after the global->LDS loads: low plane, high plane, slot
// map (128 bytes, loaded twice), (scale, zero) pairs.  A V page-head: codes and (scale, zero) pairs.
constexpr int kKOffHi = 4096, kKOffIdx = 5120, kKOffMeta = 5376, kKTile = 5888;
constexpr int kVOffMeta = 4096, kVTile = 4608;

struct Tables {
  uint32_t ks_perm[64], kz_perm[64];  // K scale / zero pairs in operand order (see stage_k_meta)
  _Float16 ks4_nat[kQPad];            // 4 * K scale by channel; [128] = 0
  uint32_t vs_nat[64], vz_nat[64];    // V scale / zero pairs by token pair
  uint32_t ones[64];                  // fp16 (1, 1) pairs: the "row of ones" operand
  uint8_t inv[32];                    // high-plane slot -> channel (128 = slot unused)
};
// LDS of one wave.  With tiles streamed through LDS (DMA) the budget is 160 KB / 8 waves per CU,
// which leaves room for the q rows of 8 heads; larger groups use the register-fed variant.
// QUARTER (at most 4 query heads per kv head, see softmax_quarter): four more V scale tables, q rows
// of 4 heads.
template <bool DMA, bool QUARTER>
struct WaveLds;
template <>
struct WaveLds<true, false> : Tables {
  __attribute__((aligned(16))) uint8_t kbuf[2][kKTile];
  __attribute__((aligned(16))) uint8_t vbuf[kVTile];
  __attribute__((aligned(16))) _Float16 q_nat[8][kQPad];   // [head][channel]; [..][128] = 0 ("no channel")
};
// Quarter variant: the B operands of QK (q * scale, both parts, for the four heads) are a table
// built once per page (qs, see qk_packed_tab), so the per-page tables of the generic path are only
// needed by the tail tiles, which run after the body loop: they share the space of the V tile.
constexpr int kQsPitch = 72;   // dwords per row of qs: 64 channel pairs + 8, so that rows fall on different banks
template <>
struct WaveLds<true, true> {
  __attribute__((aligned(16))) uint8_t kbuf[2][kKTile];
  union {
    __attribute__((aligned(16))) uint8_t vbuf[kVTile];
    struct {   // tail tiles only (staged by stage_tail_tables)
      __attribute__((aligned(16))) uint32_t ks_perm[64];
      _Float16 ks4_nat[kQPad];
      uint32_t vs_nat[64], ones[64];
      uint8_t inv[32];
      __attribute__((aligned(16))) _Float16 q_nat[4][kQPad];
    };
  };
  __attribute__((aligned(16))) uint32_t kz_perm[64];
  uint32_t vz_nat[64];
  // vs_q[t][e]: the V scale pair of token pair e if e % 4 == t, else 0 (cleared once per kernel):
  // a column that owns operand register t of every chunk multiplies by table t and so feeds
  // zeros for the tokens of the other columns
  __attribute__((aligned(16))) uint32_t vs_q[4][64];
  __attribute__((aligned(16))) uint32_t ones4[4];      // fp16 (1, 1) pairs
  // qs[r][l]: fp16 pair for channels 2l, 2l+1; rows 0..3 = fp16(q_head * scale) of the four heads,
  // rows 4..7 = the exact remainders
  __attribute__((aligned(16))) uint32_t qs[8][kQsPitch];
};
static_assert(sizeof(WaveLds<true, true>) <= 160 * 1024 / 8, "eight waves per CU");
template <>
struct WaveLds<false, false> : Tables {
  __attribute__((aligned(16))) _Float16 q_nat[16][kQPad];
  __attribute__((aligned(16))) uint8_t kbuf[1][10240];     // staging of fp16 V rows (pv_fp16)
};

__device__ __forceinline__ float4v mfma16(const uint32_t (&a)[4], const uint32_t (&b)[4], float4v c) {
  const uint4v av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, av), __builtin_bit_cast(half8, bv), c, 0,
                                                0, 0);
}
__device__ __forceinline__ half2v as_h2(uint32_t u) { return __builtin_bit_cast(half2v, u); }
__device__ __forceinline__ uint32_t as_u32(half2v h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ uint32_t swap_pair(uint32_t v) {   // value of lane n^1
  return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1 /* quad_perm [1,0,3,2] */, 0xf, 0xf, true);
}
// Maximum over the four lane groups (lanes l, l^16, l^32, l^48) with the row-swap instructions of
// gfx950: two vector instructions per step, where a shuffle would be a round trip through LDS.
// v_permlane16_swap exchanges rows 1 and 3 of its first operand with rows 0 and 2 of its second.
__device__ __forceinline__ float max_over_lane_groups(float v) {
  const unsigned b = __builtin_bit_cast(unsigned, v);
  const auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  const unsigned r0 = r[0], r1 = r[1];   // as scalars first: a bit_cast of r[1] itself reads element 0
  const float m = fmaxf(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
  const unsigned c = __builtin_bit_cast(unsigned, m);
  const auto q = __builtin_amdgcn_permlane32_swap(c, c, false, false);
  const unsigned q0 = q[0], q1 = q[1];
  return fmaxf(__builtin_bit_cast(float, q0), __builtin_bit_cast(float, q1));
}

// The workgroup is one wavefront, and the LDS unit executes a wavefront's instructions in order:
// a write followed by a read needs no hardware wait, only the compiler must keep the order.
__device__ __forceinline__ void wave_lds_fence() { asm volatile("" ::: "memory"); }

// first plane row (of a 32-row chunk) behind operand register pi of lane group kg
__device__ __forceinline__ constexpr int krow(int pi, int kg) { return 16 * (pi >> 1) + 4 * kg + 2 * (pi & 1); }

// Transposing LDS read: the 16 lanes of a block address 4 rows x 16 pieces of 16 bits (lane s:
// row s/4, pieces 4(s%4) ..); lane i receives piece i of the 4 rows = two operand registers.
typedef short short4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void lds_tr2(const uint8_t* p, uint32_t& r0, uint32_t& r1) {
  const short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)p);
  const uint2 u = __builtin_bit_cast(uint2, v);
  r0 = u.x;
  r1 = u.y;
}

// Mask of tile / d-tile u inside X (u < 5) or X >> 10 (u >= 5), and the factor that undoes the
// subnormal encoding code * 4^u' * 2^-24.
__device__ __forceinline__ constexpr uint32_t code_mask(int u) { return 0x00030003u << (2 * (u < 5 ? u : u - 5)); }
__device__ __forceinline__ constexpr float code_unscale(int u) {
  return 16777216.0f / (float)(1 << (2 * (u < 5 ? u : u - 5)));
}

// The eight tiles of one k-chunk against a two-part B operand; the operand registers of the next
// tile are masked out while the MFMAs of the current one run (two register sets, no copies).
__device__ __forceinline__ void unpack_mfma2(const uint32_t (&X)[4], const uint32_t (&Y)[4], const uint32_t (&bh)[4],
                                             const uint32_t (&bl)[4], float4v (&C)[8]) {
  uint32_t a0[4], a1[4];
#pragma unroll
  for (int pi = 0; pi < 4; ++pi) a0[pi] = X[pi] & code_mask(0);
#pragma unroll
  for (int u = 0; u < 8; u += 2) {
    C[u] = mfma16(a0, bh, C[u]);
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) a1[pi] = (u + 1 < 5 ? X[pi] : Y[pi]) & code_mask(u + 1);
    C[u] = mfma16(a0, bl, C[u]);
    C[u + 1] = mfma16(a1, bh, C[u + 1]);
    if (u + 2 < 8) {
#pragma unroll
      for (int pi = 0; pi < 4; ++pi) a0[pi] = (u + 2 < 5 ? X[pi] : Y[pi]) & code_mask(u + 2);
    }
    C[u + 1] = mfma16(a1, bl, C[u + 1]);
  }
}
__device__ __forceinline__ void unpack_mfma1(const uint32_t (&X)[4], const uint32_t (&Y)[4], const uint32_t (&b)[4],
                                             float4v (&C)[8]) {
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    uint32_t a[4];
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) a[pi] = (u < 5 ? X[pi] : Y[pi]) & code_mask(u);
    C[u] = mfma16(a, b, C[u]);
  }
}

struct Acc {
  float4v out[8];     // O^T accumulators, d-tile u: channel 32kg + 8j + u, column n
  float m;            // running max of the column's logits, log2 units
  float4v lz;         // [0] = sum of p, [1] = sum of p * zero_v over all tokens seen (whole column)
  bool first;         // nothing accumulated yet
  bool true_units;    // out[] already multiplied by code_unscale (fp16-V tiles accumulate directly)
};

struct Ctx {
  const kitty_kv_layer* L;
  SeqCounts c;
  int b, h, lane, kg, n;
  uint32_t lane_off;    // register-fed tiles: byte offset of this lane's word relative to plane row krow(pi, 0)
  uint32_t sel;         // v_perm selector merging own / partner halves
  int g;                // query head of this column
  bool lo_part;         // split columns: this column carries the low part of q * scale (see qk_packed)
  int pi_own;           // quarter columns: the operand register (token pairs 2 pi_own + {0,1} of every octet) of this column
  float usc[2];         // quarter columns: code_unscale(2 pi_own + i) * sc2
  uint32_t ktr;         // LDS: this lane's corner of a transposing read of K plane rows 4kg .. 4kg+3
  uint32_t vtr;         // LDS: same for V rows 32kg .. 32kg+3
  float sc2;            // scaling * log2(e)
  uint32_t qpair[16];   // q[col][32kc + 8pi + 2kg + {0,1}] as an fp16 pair, index 4kc + pi
  // quarter columns (qk_packed_tab):
  uint32_t q4[4];       // q[head r][2 lane + {0,1}] of the four heads behind the table rows
  uint32_t qs_rd;       // byte offset of this lane's first read in the q * scale table: row, lane group
  uint32_t qb_rd;       // the same in the table of the high-plane slots
  mutable int bad_page; // a page id outside the cache was met (checked_page); reported when the wave is done
};

// ---------------------------------------------------------------------------------------------
// K side
// ---------------------------------------------------------------------------------------------
// Two ways a packed K page-head reaches the operands.  Both hand out, per 256-byte plane chunk,
// X = [8 codes of plane row 2kg | 8 codes of row 2kg+1] for this lane's token octet.
//
// KRegs: 20 words in registers, loaded straight from HBM; halves swapped between lanes n, n^1.
struct KRegs {
  uint32_t lo[16], hi[4];
  uint2 meta;
  uint32_t idx2;
  __device__ __forceinline__ void x4_lo(const Ctx& x, int kc, uint32_t (&X)[4]) const {
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) X[pi] = __builtin_amdgcn_perm(swap_pair(lo[4 * kc + pi]), lo[4 * kc + pi], x.sel);
  }
  __device__ __forceinline__ void x4_hi(const Ctx& x, uint32_t (&X)[4]) const {
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) X[pi] = __builtin_amdgcn_perm(swap_pair(hi[pi]), hi[pi], x.sel);
  }
  __device__ __forceinline__ uint2 meta2(const Ctx&) const { return meta; }
  __device__ __forceinline__ uint32_t idx(const Ctx&) const { return idx2; }
};
// KLds: the whole page-head in LDS; two transposing reads per 32-row chunk.
struct KLds {
  const uint8_t* base;
  __device__ __forceinline__ void x4_lo(const Ctx& x, int kc, uint32_t (&X)[4]) const {
    lds_tr2(base + kc * 1024 + x.ktr, X[0], X[1]);
    lds_tr2(base + kc * 1024 + 512 + x.ktr, X[2], X[3]);
  }
  __device__ __forceinline__ void x4_hi(const Ctx& x, uint32_t (&X)[4]) const {
    lds_tr2(base + kKOffHi + x.ktr, X[0], X[1]);
    lds_tr2(base + kKOffHi + 512 + x.ktr, X[2], X[3]);
  }
  __device__ __forceinline__ uint2 meta2(const Ctx& x) const { return *(const uint2*)(base + kKOffMeta + x.lane * 8); }
  __device__ __forceinline__ uint32_t idx(const Ctx& x) const { return *(const uint16_t*)(base + kKOffIdx + 2 * x.lane); }
};

template <bool BOOST>
__device__ __forceinline__ void k_load_regs(const Ctx& x, int page_index, KRegs& kb) {
  const kitty_kv_layer& L = *x.L;
  const int64_t pg = checked_page(page_id(L.page_table_k, (int64_t)x.b * L.page_table_k_stride_b + page_index), L.cache_pages_k, x.bad_page);
  const uint8_t* page = L.key_cache + pg * L.key_cache_stride_page + (int64_t)x.h * k_head_bytes(BOOST ? 32 : 0);
  const uint8_t* meta = (const uint8_t*)L.key_meta + pg * L.key_meta_stride_page + (int64_t)x.h * kD * 4;
#pragma unroll
  for (int c = 0; c < 16; ++c)   // register 4kc + pi: plane rows 32kc + krow(pi, kg) + (n&1)
    kb.lo[c] = *(const uint32_t*)(page + ((c >> 2) * 32 + krow(c & 3, 0)) * kRowBytes + x.lane_off);
  if (BOOST) {
#pragma unroll
    for (int c = 0; c < 4; ++c) kb.hi[c] = *(const uint32_t*)(page + kLoBytes + krow(c, 0) * kRowBytes + x.lane_off);
    kb.idx2 = *(const uint16_t*)(page + kRowBytes * (kD + 32) + 2 * x.lane);
  }
  kb.meta = *(const uint2*)(meta + x.lane * 8);                          // [s0|z0], [s1|z1]
}

// Global -> LDS loads (no registers involved): scalar base + per-lane offset; the LDS destination of
// lane l is M0 + instruction offset + l * BYTES, and the instruction offset advances the global
// address as well.  N instructions of BYTES (4 or 16) per lane, 64 * BYTES apart.  M0 reaches the
// instructions as an operand bound to that register (the compiler loads it and knows it is read),
// not through a clobber.  Every tile is read exactly once, so the loads are marked non-temporal.
template <int N, int BYTES>
__device__ __forceinline__ void lds_dma(uint32_t lane_off, const uint8_t* base, uint32_t lds) {
  static_assert((BYTES == 16 && (N == 1 || N == 4)) || (BYTES == 4 && (N == 1 || N == 2)), "forms in use");
  register uint32_t m0_lds asm("m0") = lds;
  if constexpr (BYTES == 16 && N == 4)
    asm volatile(
        "global_load_lds_dwordx4 %0, %1 nt\n\t"
        "global_load_lds_dwordx4 %0, %1 offset:1024 nt\n\t"
        "global_load_lds_dwordx4 %0, %1 offset:2048 nt\n\t"
        "global_load_lds_dwordx4 %0, %1 offset:3072 nt"
        :: "v"(lane_off), "s"(base), "s"(m0_lds) : "memory");
  else if constexpr (BYTES == 16)
    asm volatile("global_load_lds_dwordx4 %0, %1 nt" :: "v"(lane_off), "s"(base), "s"(m0_lds) : "memory");
  else if constexpr (N == 2)
    asm volatile(
        "global_load_lds_dword %0, %1 nt\n\t"
        "global_load_lds_dword %0, %1 offset:256 nt"
        :: "v"(lane_off), "s"(base), "s"(m0_lds) : "memory");
  else
    asm volatile("global_load_lds_dword %0, %1 nt" :: "v"(lane_off), "s"(base), "s"(m0_lds) : "memory");
}

// Global -> LDS loads of one K page-head: 8 instructions with the high plane, 6 without
// (non-temporal: 2 % on the whole launch; a read-only stream runs at 6.5 TB/s with the hint and
// 5.9 TB/s without).
template <bool BOOST>
constexpr int kDmaK = BOOST ? 8 : 6;
constexpr int kDmaV = 6;

template <bool BOOST>
__device__ __forceinline__ void dma_k(const Ctx& x, int page_index, uint32_t lds) {
  const kitty_kv_layer& L = *x.L;
  const int64_t pg = checked_page(page_id(L.page_table_k, (int64_t)x.b * L.page_table_k_stride_b + page_index), L.cache_pages_k, x.bad_page);
  const uint8_t* page = L.key_cache + pg * L.key_cache_stride_page + (int64_t)x.h * k_head_bytes(BOOST ? 32 : 0);
  const uint8_t* meta = (const uint8_t*)L.key_meta + pg * L.key_meta_stride_page + (int64_t)x.h * kD * 4;
  const uint32_t off16 = x.lane * 16, off4 = x.lane * 4, off4dup = (x.lane & 31) * 4;
  lds_dma<4, 16>(off16, page, lds);
  if (BOOST) {
    lds_dma<1, 16>(off16, page + kLoBytes, lds + kKOffHi);
    lds_dma<1, 4>(off4dup, page + kLoBytes + 1024, lds + kKOffIdx);
  }
  lds_dma<2, 4>(off4, meta, lds + kKOffMeta);
}

// Stage the page-head's (scale, zero) pairs and slot map in LDS in the order the operands need:
// channel pair (2l, 2l+1) of lane l belongs to chunk kc = l/16; within the chunk 2(l%16) =
// krow(pi, kg) gives kg = (l/2)%4 and pi = 2((l/8)%2) + l%2.  It is stored at word
// 16kc + 4kg + pi, so that a lane reads the four pairs of a chunk with one 128-bit LDS read.
template <bool BOOST, class LDS, class KSRC>
__device__ __forceinline__ void stage_k_meta(LDS& S, const Ctx& x, const KSRC& kb) {
  const int l = x.lane;
  const uint2 km = kb.meta2(x);
  const uint32_t ib = BOOST ? kb.idx(x) : 0u;   // both reads first: one round trip through LDS, not two
  const uint32_t ss = __builtin_amdgcn_perm(km.y, km.x, 0x05040100u);   // (s0, s1)
  const uint32_t zz = __builtin_amdgcn_perm(km.y, km.x, 0x07060302u);   // (z0, z1)
  const int pos = (l >> 4) * 16 + ((l >> 1) & 3) * 4 + 2 * ((l >> 3) & 1) + (l & 1);
  wave_lds_fence();
  S.ks_perm[pos] = ss;
  S.kz_perm[pos] = zz;
  if (BOOST) {
    const half2v four = {(_Float16)4.0f, (_Float16)4.0f};
    ((uint32_t*)S.ks4_nat)[l] = as_u32(as_h2(ss) * four);
    if (l < 8) ((uint32_t*)S.inv)[l] = 0x80808080u;
    wave_lds_fence();   // LDS executes a wave's instructions in order: the scatter below lands on the cleared bytes
    const uint32_t i0 = ib & 0xffu, i1 = ib >> 8;
    if (i0 < 32) S.inv[i0] = (uint8_t)(2 * l);
    if (i1 < 32) S.inv[i1] = (uint8_t)(2 * l + 1);
  }
  wave_lds_fence();
}

__device__ __forceinline__ float ror8(float v) {   // value of column n ^ 8 (rotation by 8 within the row of 16 lanes)
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128 /* row_ror:8 */,
                                                                0xf, 0xf, false));
}

__device__ __forceinline__ float ror4(float v) {   // value of column n - 4 (mod 16)
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124 /* row_ror:4 */,
                                                                0xf, 0xf, false));
}

// logits of one packed K page: C[u][j] = sum_ch code * q * scale, still in subnormal units
// (multiply by code_unscale(u)); cz = q . zero.
// q * scale does not fit an fp16 operand (the product of two fp16 numbers has 22 significant bits
// and the logits need more than 11), so it enters as a rounded part and its exact remainder.
// SPLIT_COLS (at most 8 query heads per kv head): the two parts sit in different columns of the
// same B operand - column n carries the rounded part of head n % 8, column n + 8 the remainder -
// and the two partial sums are added across the columns afterwards: one matrix instruction per
// tile of codes instead of two, none of them waiting for the one before it.
template <bool BOOST, bool SPLIT_COLS, class LDS, class KSRC>
__device__ __forceinline__ void qk_packed(LDS& S, const Ctx& x, const KSRC& kb, float4v (&C)[8], float& cz) {
  // One chunk of 32 plane rows ahead: the LDS reads of chunk kc + 1 are issued before the vector
  // and matrix work of chunk kc, so that their latency is covered by this wave's own work.
  uint32_t Xn[4];
  kb.x4_lo(x, 0, Xn);                       // does not depend on the tables staged below
  stage_k_meta<BOOST>(S, x, kb);
  uint4v spn = *(const uint4v*)&S.ks_perm[x.kg * 4];
  uint4v zpn = *(const uint4v*)&S.kz_perm[x.kg * 4];
  uint32_t inv2[4];                          // high-plane chunk: channels behind this lane's slots
  half2v qh[4], sh[4];                       // high-plane chunk: gathered q and 4 * scale
  // q . zero_k on the matrix core as well: an A tile whose 16 rows all hold the zero points
  float4v Cz = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int u = 0; u < 8; ++u) C[u] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int kc = 0; kc < 4; ++kc) {
    uint32_t bh[4], bl[4], bq[4], az[4], X[4], Y[4];
    const uint4v sp = spn, zp = zpn;
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) X[pi] = Xn[pi];
    if (kc < 3) {
      kb.x4_lo(x, kc + 1, Xn);
      spn = *(const uint4v*)&S.ks_perm[(kc + 1) * 16 + x.kg * 4];
      zpn = *(const uint4v*)&S.kz_perm[(kc + 1) * 16 + x.kg * 4];
    } else if (BOOST) {
      kb.x4_hi(x, Xn);
    }
    if (BOOST && kc == 2) {
#pragma unroll
      for (int pi = 0; pi < 4; ++pi) inv2[pi] = *(const uint16_t*)&S.inv[krow(pi, x.kg)];
    }
    if (BOOST && kc == 3) {
#pragma unroll
      for (int pi = 0; pi < 4; ++pi) {
        const uint32_t c0 = inv2[pi] & 0xffu, c1 = inv2[pi] >> 8;
        qh[pi] = half2v{S.q_nat[x.g][c0], S.q_nat[x.g][c1]};
        sh[pi] = half2v{S.ks4_nat[c0], S.ks4_nat[c1]};
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) {
      const half2v qq = as_h2(x.qpair[kc * 4 + pi]), s2 = as_h2(sp[pi]);
      const half2v hi = qq * s2;                                   // q*scale rounded to fp16 ...
      const half2v lo = __builtin_elementwise_fma(qq, s2, -hi);    // ... and its exact remainder
      bh[pi] = SPLIT_COLS ? (x.lo_part ? as_u32(lo) : as_u32(hi)) : as_u32(hi);
      bl[pi] = as_u32(lo);
      bq[pi] = x.qpair[kc * 4 + pi];
      az[pi] = zp[pi];
      Y[pi] = X[pi] >> 10;
    }
    Cz = mfma16(az, bq, Cz);
    if (SPLIT_COLS) unpack_mfma1(X, Y, bh, C);
    else unpack_mfma2(X, Y, bh, bl, C);
  }
  if (BOOST) {
    // fifth chunk: the 32 high-plane slots; slot krow(pi, kg) + h carries bits 3:2 of the channel
    // inv[slot], weight 4 * scale
    uint32_t bh[4], bl[4], X[4], Y[4];
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) {
      X[pi] = Xn[pi];
      const half2v hi = qh[pi] * sh[pi];
      const half2v lo = __builtin_elementwise_fma(qh[pi], sh[pi], -hi);
      bh[pi] = SPLIT_COLS ? (x.lo_part ? as_u32(lo) : as_u32(hi)) : as_u32(hi);
      bl[pi] = as_u32(lo);
      Y[pi] = X[pi] >> 10;
    }
    if (SPLIT_COLS) unpack_mfma1(X, Y, bh, C);
    else unpack_mfma2(X, Y, bh, bl, C);
  }
  if (SPLIT_COLS) {
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j) C[u][j] += ror8(C[u][j]);
  }
  cz = Cz[0];
}

// The same for quarter columns (at most four heads), with the B operands from a table.  The generic
// path has every lane multiply q by the scales of its own operand registers: 16 columns = 4 heads x
// 2 parts, each computed twice, plus a gather of q and scale through the slot map for the high
// plane.  Here lane l, which receives the (scale, zero) pairs of channels 2l and 2l + 1, computes
// both parts for the four heads once and stores them in channel order (qs); an operand register
// pair of a 32-channel chunk - channels 32kc + 16 (pi / 2) + 4kg + {0..3} - is then one 64-bit read,
// and the pipeline spends no vector instruction on the B side.  The operands of the high plane are
// scattered instead of gathered: a boosted channel's lane writes 4 * q * scale to its slot of a
// [row][slot] table, which lies in the tile's slot-map and metadata bytes (in registers by then).
template <bool BOOST, class LDS>
__device__ __forceinline__ void qk_packed_tab(LDS& S, const Ctx& x, uint8_t* kt, float4v (&C)[8], float& cz) {
  const KLds kb{kt};
  uint32_t Xn[4];
  kb.x4_lo(x, 0, Xn);
  const int l = x.lane;
  const uint2 km = kb.meta2(x);
  const uint32_t ib = BOOST ? kb.idx(x) : 0u;
  const uint32_t ss = __builtin_amdgcn_perm(km.y, km.x, 0x05040100u);   // (s0, s1)
  const uint32_t zz = __builtin_amdgcn_perm(km.y, km.x, 0x07060302u);   // (z0, z1)
  const int pos = (l >> 4) * 16 + ((l >> 1) & 3) * 4 + 2 * ((l >> 3) & 1) + (l & 1);   // see stage_k_meta
  uint8_t* bt = kt + kKOffIdx;   // high-plane operands: 8 rows x 32 slots, fp16
  wave_lds_fence();              // the reads above come first: LDS executes a wave's instructions in order
  S.kz_perm[pos] = zz;
  uint32_t hi[4], lo[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const half2v h = as_h2(x.q4[r]) * as_h2(ss);                                    // q*scale rounded to fp16 ...
    hi[r] = as_u32(h);
    lo[r] = as_u32(__builtin_elementwise_fma(as_h2(x.q4[r]), as_h2(ss), -h));       // ... and its exact remainder
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    S.qs[r][l] = hi[r];
    S.qs[4 + r][l] = lo[r];
  }
  if (BOOST) {
    *(uint2*)(bt + 8 * l) = uint2{0u, 0u};   // a slot no channel claims contributes nothing
    wave_lds_fence();
    const half2v four = {(_Float16)4.0f, (_Float16)4.0f};
    const uint32_t i0 = ib & 0xffu, i1 = ib >> 8;
    uint32_t w4[8];   // the high plane's weight: 4 * scale
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      w4[r] = as_u32(as_h2(hi[r]) * four);
      w4[4 + r] = as_u32(as_h2(lo[r]) * four);
    }
    if (i0 < 32) {
#pragma unroll
      for (int r = 0; r < 8; ++r) *(uint16_t*)(bt + 64 * r + 2 * i0) = (uint16_t)(w4[r] & 0xffffu);
    }
    if (i1 < 32) {
#pragma unroll
      for (int r = 0; r < 8; ++r) *(uint16_t*)(bt + 64 * r + 2 * i1) = (uint16_t)(w4[r] >> 16);
    }
  }
  wave_lds_fence();
  const uint8_t* rd = (const uint8_t*)&S.qs[0][0] + x.qs_rd;
  uint2 b01n = *(const uint2*)rd, b23n = *(const uint2*)(rd + 32);
  uint4v zpn = *(const uint4v*)&S.kz_perm[x.kg * 4];
  float4v Cz = float4v{0.f, 0.f, 0.f, 0.f};   // q . zero_k: an A tile whose 16 rows all hold the zero points
#pragma unroll
  for (int u = 0; u < 8; ++u) C[u] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int kc = 0; kc < 4; ++kc) {
    uint32_t bq[4], az[4], X[4], Y[4];
    const uint4v zp = zpn;
    const uint32_t b[4] = {b01n.x, b01n.y, b23n.x, b23n.y};
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) X[pi] = Xn[pi];
    if (kc < 3) {   // one chunk ahead, as in qk_packed
      kb.x4_lo(x, kc + 1, Xn);
      b01n = *(const uint2*)(rd + 64 * (kc + 1));
      b23n = *(const uint2*)(rd + 64 * (kc + 1) + 32);
      zpn = *(const uint4v*)&S.kz_perm[(kc + 1) * 16 + x.kg * 4];
    } else if (BOOST) {
      kb.x4_hi(x, Xn);
      b01n = *(const uint2*)(bt + x.qb_rd);
      b23n = *(const uint2*)(bt + x.qb_rd + 32);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) {
      bq[pi] = x.qpair[kc * 4 + pi];
      az[pi] = zp[pi];
      Y[pi] = X[pi] >> 10;
    }
    Cz = mfma16(az, bq, Cz);
    unpack_mfma1(X, Y, b, C);
  }
  if (BOOST) {
    uint32_t X[4], Y[4];
    const uint32_t b[4] = {b01n.x, b01n.y, b23n.x, b23n.y};
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) {
      X[pi] = Xn[pi];
      Y[pi] = X[pi] >> 10;
    }
    unpack_mfma1(X, Y, b, C);
  }
  cz = Cz[0];
}

// Quarter columns.  With at most 4 query heads per kv head the 16 columns of a tile hold every
// head at least four times (columns n, n ^ 4, n ^ 8, n ^ 12; n and n ^ 8 carry the two parts of
// q * scale), and the softmax of a page would be computed four times over.  Instead each of the four
// columns keeps two of the eight 16-token tiles - tiles 2 pi_own + {0, 1}, i.e. operand register
// pi_own of every PV chunk - does the softmax of those 32 tokens only, and feeds zeros for the other
// tokens into PV; its accumulators then hold a partial sum over its tokens, and the four are added
// once, when the split is written.  The running maximum is shared, so the partials are compatible.
//
// own[i][j] = the full logit (both parts) of tile 2 pi_own + i, still in code units.  Two selects
// around the cross-column add: columns n and n ^ 8 must hold the same tiles when they are added.
__device__ __forceinline__ void combine_quarter(const Ctx& x, const float4v (&C)[8], float4v (&own)[2]) {
  const bool upper = x.pi_own & 2, odd = x.pi_own & 1;   // pi_own = 2 * bit 2 of n + bit 3 of n
  float4v T[4];
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float v = upper ? C[4 + k][j] : C[k][j];
      T[k][j] = v + ror8(v);
    }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) own[i][j] = odd ? T[2 + i][j] : T[i][j];
}

// logits of up to 128 fp16 rows (sink or K Q-buffer): A = the rows themselves, B = q.  Here the k-slots
// are in natural order - slot (kg, 2pi + h) = channel 32kc + 8kg + 2pi + h - so that an operand is one
// 16-byte load of the row, and q comes from its natural-order copy in LDS (q_nat).  The loads of
// four tiles (16 per lane) are issued together: the rows come straight from HBM and a wave has
// nothing else to do while it waits, so the depth of the queue is what the phase costs.  Lanes whose
// row lies past the `nrows` valid ones read the last valid row again (their logits are masked later):
// nothing is fetched that does not count.
template <class LDS>
__device__ __forceinline__ void qk_fp16(const LDS& S, const Ctx& x, const uint8_t* rows, int nrows, float4v (&C)[8]) {
  uint4v bq[4];
#pragma unroll
  for (int kc = 0; kc < 4; ++kc) bq[kc] = *(const uint4v*)&S.q_nat[x.g][32 * kc + 8 * x.kg];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    uint4v a[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = min(8 * x.n + 4 * half + i, nrows - 1);   // A row of this lane; clamped rows are masked later
      const uint8_t* rp = rows + (int64_t)row * (kD * 2) + 16 * x.kg;
#pragma unroll
      for (int kc = 0; kc < 4; ++kc) a[i][kc] = *(const uint4v*)(rp + 64 * kc);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float4v acc = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kc = 0; kc < 4; ++kc)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a[i][kc]),
                                                     __builtin_bit_cast(half8, bq[kc]), acc, 0, 0, 0);
      C[4 * half + i] = acc;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// softmax bookkeeping: C holds raw dot products on entry (SUBNORMAL: in code units, to be
// multiplied by code_unscale(u)), probabilities on exit
// ---------------------------------------------------------------------------------------------
template <bool SUBNORMAL>
__device__ __forceinline__ void softmax_tile(const Ctx& x, Acc& A, float4v (&C)[8], float cz, int ntok) {
  const float cst = cz * x.sc2 - A.m;
  float mt = -INFINITY;
#pragma unroll
  for (int u = 0; u < 8; ++u)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v = C[u][j] * (SUBNORMAL ? code_unscale(u) * x.sc2 : x.sc2) + cst;   // log2-logit - running max
      if (ntok < kPage && 32 * x.kg + 8 * j + u >= ntok) v = -INFINITY;
      C[u][j] = v;
    }
#pragma unroll
  for (int u = 0; u < 8; ++u) mt = fmaxf(fmaxf(mt, fmaxf(C[u][0], C[u][1])), fmaxf(C[u][2], C[u][3]));
  mt = max_over_lane_groups(mt);
  if (__any(A.first || mt > 0.f)) {
    // the column's max moves: shift this tile's logits and rescale what is accumulated
    const float dm = A.first ? mt : fmaxf(mt, 0.f);
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j) C[u][j] -= dm;
    if (!A.first) {
      const float alpha = __builtin_amdgcn_exp2f(-dm);
      A.lz *= alpha;
#pragma unroll
      for (int u = 0; u < 8; ++u) A.out[u] *= alpha;
    }
    A.m += dm;
    A.first = false;
  }
#pragma unroll
  for (int u = 0; u < 8; ++u)
#pragma unroll
    for (int j = 0; j < 4; ++j) C[u][j] = __builtin_amdgcn_exp2f(C[u][j]);
}

// The same for the two tiles a quarter column owns (full packed pages only: nothing to mask).
__device__ __forceinline__ void softmax_quarter(const Ctx& x, Acc& A, float4v (&own)[2], float cz) {
  const float cst = cz * x.sc2 - A.m;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) own[i][j] = own[i][j] * x.usc[i] + cst;
  float mt = fmaxf(fmaxf(fmaxf(own[0][0], own[0][1]), fmaxf(own[0][2], own[0][3])),
                   fmaxf(fmaxf(own[1][0], own[1][1]), fmaxf(own[1][2], own[1][3])));
  mt = fmaxf(mt, ror4(mt));            // the four columns of a head ...
  mt = fmaxf(mt, ror8(mt));
  mt = max_over_lane_groups(mt);       // ... and the four lane groups: the page's maximum for this head
  if (__any(A.first || mt > 0.f)) {
    const float dm = A.first ? mt : fmaxf(mt, 0.f);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) own[i][j] -= dm;
    if (!A.first) {
      const float alpha = __builtin_amdgcn_exp2f(-dm);
      A.lz *= alpha;
#pragma unroll
      for (int u = 0; u < 8; ++u) A.out[u] *= alpha;
    }
    A.m += dm;
    A.first = false;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) own[i][j] = __builtin_amdgcn_exp2f(own[i][j]);
}

// ---------------------------------------------------------------------------------------------
// V side
// ---------------------------------------------------------------------------------------------
struct VRegs {
  uint32_t w[16];
  uint2 meta;
  __device__ __forceinline__ void x4(const Ctx& x, int j, uint32_t (&X)[4]) const {
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) X[pi] = __builtin_amdgcn_perm(swap_pair(w[4 * j + pi]), w[4 * j + pi], x.sel);
  }
  __device__ __forceinline__ uint2 meta2(const Ctx&) const { return meta; }
};
struct VLds {
  const uint8_t* base;
  __device__ __forceinline__ void x4(const Ctx& x, int j, uint32_t (&X)[4]) const {   // rows 32kg + 8j + 2pi + {0,1}
    lds_tr2(base + j * 256 + x.vtr, X[0], X[1]);
    lds_tr2(base + j * 256 + 128 + x.vtr, X[2], X[3]);
  }
  __device__ __forceinline__ uint2 meta2(const Ctx& x) const { return *(const uint2*)(base + kVOffMeta + x.lane * 8); }
};

__device__ __forceinline__ void v_load_regs(const Ctx& x, int page_index, VRegs& vb) {
  const kitty_kv_layer& L = *x.L;
  const int64_t pg = checked_page(page_id(L.page_table_v, (int64_t)x.b * L.page_table_v_stride_b + page_index), L.cache_pages_v, x.bad_page);
  const uint8_t* page = L.value_cache + pg * L.value_cache_stride_page + (int64_t)x.h * kVBytes;
  const uint8_t* meta = (const uint8_t*)L.value_meta + pg * L.value_meta_stride_page + (int64_t)x.h * kPage * 4;
  const uint32_t v_off = (32 * x.kg + (x.n & 1)) * kRowBytes + (x.n >> 1) * 4;
#pragma unroll
  for (int c = 0; c < 16; ++c) vb.w[c] = *(const uint32_t*)(page + v_off + c * 64);   // rows 32kg + 2c + (n&1)
  vb.meta = *(const uint2*)(meta + x.lane * 8);                                        // tokens 2l, 2l+1
}

// Global -> LDS loads of one V page-head, byte for byte.
__device__ __forceinline__ void dma_v(const Ctx& x, int page_index, uint32_t lds) {
  const kitty_kv_layer& L = *x.L;
  const int64_t pg = checked_page(page_id(L.page_table_v, (int64_t)x.b * L.page_table_v_stride_b + page_index), L.cache_pages_v, x.bad_page);
  const uint8_t* page = L.value_cache + pg * L.value_cache_stride_page + (int64_t)x.h * kVBytes;
  const uint8_t* meta = (const uint8_t*)L.value_meta + pg * L.value_meta_stride_page + (int64_t)x.h * kPage * 4;
  const uint32_t off16 = x.lane * 16;
  lds_dma<4, 16>(off16, page, lds);
  const uint32_t off4 = x.lane * 4;
  lds_dma<2, 4>(off4, meta, lds + kVOffMeta);
}

template <class LDS, class VSRC>
__device__ __forceinline__ void pv_packed(LDS& S, const Ctx& x, float4v (&out)[8], float4v& lz, const VSRC& vb,
                                          const float4v (&P)[8]) {
  const uint2 vm = vb.meta2(x);
  wave_lds_fence();
  S.vs_nat[x.lane] = __builtin_amdgcn_perm(vm.y, vm.x, 0x05040100u);
  S.vz_nat[x.lane] = __builtin_amdgcn_perm(vm.y, vm.x, 0x07060302u);
  wave_lds_fence();
  // sum p and sum p*zero_v ride along as one more A tile: even rows are ones, odd rows the zero
  // points, so row 0 of the product is the column's sum of p and row 1 its sum of p * zero_v
  const uint32_t* lz_rows = (x.n & 1) ? S.vz_nat : S.ones;
  // one chunk of 8 plane rows per lane group ahead, as in qk_packed
  uint32_t Xn[4];
  vb.x4(x, 0, Xn);
  uint4v spn = *(const uint4v*)&S.vs_nat[16 * x.kg];
  uint4v zrn = *(const uint4v*)&lz_rows[16 * x.kg];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint4v sp = spn, zr = zrn;
    uint32_t bp[4], p16[4], alz[4], X[4], Y[4];
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) X[pi] = Xn[pi];
    if (j < 3) {
      vb.x4(x, j + 1, Xn);
      spn = *(const uint4v*)&S.vs_nat[16 * x.kg + 4 * (j + 1)];
      zrn = *(const uint4v*)&lz_rows[16 * x.kg + 4 * (j + 1)];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) {
      const half2v p2 = {(_Float16)P[2 * pi][j], (_Float16)P[2 * pi + 1][j]};   // tokens 32kg + 8j + 2pi + {0,1}
      p16[pi] = as_u32(p2);
      alz[pi] = zr[pi];
      bp[pi] = as_u32(p2 * as_h2(sp[pi]));
      Y[pi] = X[pi] >> 10;
    }
    lz = mfma16(alz, p16, lz);
    unpack_mfma1(X, Y, bp, out);
  }
}

// PV for quarter columns: P holds the probabilities of the column's own tokens only (register j:
// tokens 32kg + 8j + 2 pi_own + {0,1}).  The B operand of chunk j is that pair times the masked
// scale table of pi_own: zero in the other three registers.  Sum p and sum p * zero_v take ONE more
// tile per page: its B registers are the four own pairs themselves, and A row 2t + 1 holds the zero
// points in the token order of a column with pi_own = t (even rows: ones), so column n finds its
// sum of p in every even row and its sum of p * zero_v in row 2 pi_own + 1.
template <class LDS>
__device__ __forceinline__ void pv_quarter(LDS& S, const Ctx& x, float4v (&out)[8], float4v& lz, const VLds& vb,
                                           const float4v (&P)[2]) {
  const uint2 vm = vb.meta2(x);   // token pair e = lane: lane group e / 16, chunk (e / 4) % 4, register e % 4
  wave_lds_fence();
  S.vs_q[x.lane & 3][x.lane] = __builtin_amdgcn_perm(vm.y, vm.x, 0x05040100u);
  S.vz_nat[(x.lane & 48) + 4 * (x.lane & 3) + ((x.lane >> 2) & 3)] = __builtin_amdgcn_perm(vm.y, vm.x, 0x07060302u);
  wave_lds_fence();
  const uint32_t* sq = &S.vs_q[x.pi_own][16 * x.kg];
  const uint32_t* lz_rows = (x.n & 1) ? &S.vz_nat[16 * x.kg + 4 * ((x.n >> 1) & 3)] : &S.ones4[0];
  uint32_t Xn[4];
  vb.x4(x, 0, Xn);
  uint4v spn = *(const uint4v*)&sq[0];
  const uint4v zr = *(const uint4v*)lz_rows;
  uint32_t p16[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const half2v p2 = {(_Float16)P[0][j], (_Float16)P[1][j]};
    p16[j] = as_u32(p2);
  }
  {
    const uint32_t alz[4] = {zr[0], zr[1], zr[2], zr[3]};
    lz = mfma16(alz, p16, lz);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint4v sp = spn;
    uint32_t bp[4], X[4], Y[4];
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) X[pi] = Xn[pi];
    if (j < 3) {
      vb.x4(x, j + 1, Xn);
      spn = *(const uint4v*)&sq[4 * (j + 1)];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) {
      bp[pi] = as_u32(as_h2(p16[j]) * as_h2(sp[pi]));
      Y[pi] = X[pi] >> 10;
    }
    unpack_mfma1(X, Y, bp, out);
  }
}

// fp16 V rows (sink, V Q-buffer, local ring), accumulators in true units.  The matrix core wants
// A[row = channel][k = token], i.e. the rows transposed: 32 tokens at a time are copied into LDS as
// [channel][token] with 16-bit stores, after which the eight k-slots of a lane are one 128-bit read.
// Which 32 tokens: k-chunk s of every lane group - tokens 32kg + 8s + {0..7}, kg = 0..3, the tokens
// behind accumulator register s of the logits - so that one staging feeds ONE full-depth matrix
// instruction per channel tile.  A tile of at most 32 tokens (the sink) has them all in lane group 0:
// there tokens 0..31 are staged once and multiplied in four steps, the other lane groups feeding zeros.
constexpr int kVtPitch = 80;                 // bytes per channel row: 32 tokens + padding
constexpr int kVtBytes = kD * kVtPitch;      // 10240
static_assert(kVtBytes <= 2 * kKTile && kVtBytes <= 10240, "the staging area reuses the K tile buffers");
// QUARTER: the tail's tiles keep whole columns; only the columns with pi_own = 0 accumulate them.
template <bool SINK, bool QUARTER>
__device__ __forceinline__ void pv_fp16(uint8_t* vt, const Ctx& x, Acc& A, int tail_first_row, int ntok,
                                        const float4v (&P)[8]) {
  const kitty_kv_layer& L = *x.L;
  const uint32_t one_or_zero = (x.n & 1) ? 0u : 0x3C003C00u;    // even rows sum p, odd rows stay 0
  const int tt = x.lane >> 1, c0 = (x.lane & 1) * 8;            // staging: position among the 32 tokens, first piece
  const bool by_chunk = ntok > 32;
  const int t_base = by_chunk ? 32 * (tt >> 3) + (tt & 7) : tt, t_step = by_chunk ? 8 : 32;
  const bool col_on = !QUARTER || x.pi_own == 0;
  // the rows of staging s + 1 are fetched while staging s is multiplied
  auto fetch = [&](int s, uint4 (&piece)[8]) {
    const int t = t_base + t_step * s;
    const bool ok = t < ntok;   // rows past the tile's end carry p = 0; zeros keep 0 * value at 0
    const __half* row = nullptr;
    if (ok) {
      if (SINK)
        row = (const __half*)((const uint8_t*)L.sink_v + (int64_t)x.b * L.sink_stride_b +
                              (int64_t)x.h * L.sink_stride_h) + (int64_t)t * kD;
      else
        row = v_tail_row(L, x.c, x.b, x.h, tail_first_row + t);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) piece[k] = ok ? ((const uint4*)row)[c0 + k] : uint4{0u, 0u, 0u, 0u};
  };
  auto stage = [&](const uint4 (&piece)[8]) {
    wave_lds_fence();
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const uint32_t w4[4] = {piece[k].x, piece[k].y, piece[k].z, piece[k].w};
      uint8_t* dst = vt + (8 * (c0 + k)) * kVtPitch + 2 * tt;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        *(uint16_t*)(dst + (2 * i) * kVtPitch) = (uint16_t)(w4[i] & 0xffffu);
        *(uint16_t*)(dst + (2 * i + 1) * kVtPitch) = (uint16_t)(w4[i] >> 16);
      }
    }
  };
  // one matrix instruction per channel tile: k-slots = 8 staged tokens at byte `at` of every channel row
  auto multiply = [&](int j, int at, bool on) {
    uint32_t bp[4], alz[4];
#pragma unroll
    for (int pi = 0; pi < 4; ++pi) {
      const half2v p2 = {(_Float16)P[2 * pi][j], (_Float16)P[2 * pi + 1][j]};   // tokens 32kg + 8j + 2pi + {0,1}
      bp[pi] = on ? as_u32(p2) : 0u;
      alz[pi] = one_or_zero;
    }
    A.lz = mfma16(alz, bp, A.lz);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const uint4v a4 = *(const uint4v*)(vt + (8 * x.n + u) * kVtPitch + at);
      const uint32_t a[4] = {a4[0], a4[1], a4[2], a4[3]};
      A.out[u] = mfma16(a, bp, A.out[u]);
    }
  };
  uint4 piece[8];
  fetch(0, piece);
  if (by_chunk) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      stage(piece);
      if (j < 3) fetch(j + 1, piece);
      wave_lds_fence();
      multiply(j, 16 * x.kg, col_on);
    }
  } else {
    stage(piece);
    wave_lds_fence();
#pragma unroll
    for (int j = 0; j < 4; ++j) multiply(j, 16 * j, col_on && x.kg == 0);
  }
  wave_lds_fence();
}

__device__ __forceinline__ void to_true_units(Acc& A) {
  if (!A.true_units) {
#pragma unroll
    for (int u = 0; u < 8; ++u) A.out[u] *= code_unscale(u);
    A.true_units = true;
  }
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}

// Every vector load of the kernel's prologue (q, counters) has landed.  The compiler does not see the
// tile loads of the streaming loops (inline assembly); what it does see is its own prologue loads,
// and it would wait for the registers they fill where they are first used - inside the loop, with
// s_waitcnt vmcnt(0), which there also waits for every tile load in flight, in every iteration.
// An explicit wait before the loop, one that the compiler's bookkeeping understands, settles them.
__device__ __forceinline__ void settle_prologue_loads() {
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0); expcnt, lgkmcnt: no wait
}

// One split of one (batch row, kv head).  crowded: the launch has more workgroups than the device
// holds at once (two per SIMD) and runs in rounds.  A workgroup's fixed cost - dispatch, prologue,
// filling and draining the tile pipeline, about two tiles' worth - then comes out of the throughput,
// so the splits are cut for few, long shares (one split for the tail, body shares of at least
// kCrowdedMinTiles tiles; a short sequence leaves its last splits without work), and the ORDER of
// the workgroups matters: the dispatcher hands them out by linear id as slots free up.  With the
// grid laid out (splits, heads, rows) the splits without work come in bursts between the busy ones,
// the slots they free are refilled late (ragged batch of 64: 1,500 of 2,048 resident on average)
// and the launch ends with whatever sequence came last.  So a crowded launch either becomes one
// round of equal shares (at most kFlatMaxB sequences, see FlatPlan below) or runs from a work
// list: decode_plan_kernel, one small workgroup ahead of the split pass, reads the sequences'
// counters and writes the items that have work, the longest first; workgroup j of the split pass
// takes item j / H_KV for kv head j % H_KV, and the workgroups past the end of the list - all at
// the end of the dispatch order - leave at once.
struct WorkItem {
  int b, h, split;
  bool crowded, valid;
  int t0, t1;    // flat shares (below): the body tiles of this item
  int n_used;    // flat shares, the tail's item: partials of the sequence that some workgroup writes
};
__device__ __forceinline__ WorkItem work_item_of_block(int h_kv, const uint32_t* plan) {
  if (!plan) return WorkItem{(int)blockIdx.z, (int)blockIdx.y, (int)blockIdx.x, false, true, 0, 0, 0};
  const uint32_t j = blockIdx.x / (uint32_t)h_kv;
  if (j >= plan[0]) return WorkItem{0, 0, 0, true, false, 0, 0, 0};
  const uint32_t item = plan[kPlanHeader + j];
  return WorkItem{(int)(item >> 16), (int)(blockIdx.x % (uint32_t)h_kv), (int)(item & 0xFFFFu), true, true, 0, 0, 0};
}
constexpr int kCrowdedMinTiles = 16;   // body tiles per split a crowded launch aims for
constexpr int kCrowdedTailCost = 12;   // what the tail's split takes, in body tiles (for the order)
// Body splits of a sequence with npp body tiles in a crowded launch (its split 0 is the tail's).
__device__ __forceinline__ int crowded_body_splits(int npp, int num_splits) {
  return npp > 0 ? min(num_splits - 1, c_div_up(npp, kCrowdedMinTiles)) : 0;
}
__device__ __forceinline__ int body_tiles_of(const SeqCounts& c) {
  return min(min(c.pv, c.pk), c_div_up(c.nbody, kPage));
}

// The work list of a crowded launch: one workgroup.  Items are sorted by what they cost, longest
// first (a counting sort over the cost in tiles), so that the last round is made of the shortest.
constexpr int kPlanBuckets = 64;
__global__ __launch_bounds__(256) void decode_plan_kernel(kitty_kv_layer L, int B, int num_splits,
                                                          uint32_t* __restrict__ plan) {
  __shared__ uint32_t s_n[kPlanBuckets], s_at[kPlanBuckets];
  if (threadIdx.x < kPlanBuckets) s_n[threadIdx.x] = 0;
  __syncthreads();
  auto bucket = [](int cost) { return kPlanBuckets - 1 - min(cost, kPlanBuckets - 1); };   // longest first
  // the shares of a sequence: nb body splits, of which the first rem have one tile more
  auto shares = [&](int b, int& nb, int& base, int& rem) {
    const int npp = body_tiles_of(load_counts(L, b));
    nb = crowded_body_splits(npp, num_splits);
    base = nb ? npp / nb : 0;
    rem = nb ? npp - base * nb : 0;
  };
  // (a thread keeps the shares of its first sequence for the second pass: with up to 256 sequences
  // the counters are read once)
  int nb0 = 0, base0 = 0, rem0 = 0;
  for (int b = threadIdx.x; b < B; b += blockDim.x) {
    int nb, base, rem;
    shares(b, nb, base, rem);
    if (b == (int)threadIdx.x) nb0 = nb, base0 = base, rem0 = rem;
    atomicAdd(&s_n[bucket(kCrowdedTailCost)], 1u);
    if (rem) atomicAdd(&s_n[bucket(base + 3)], (uint32_t)rem);
    if (nb - rem) atomicAdd(&s_n[bucket(base + 2)], (uint32_t)(nb - rem));
  }
  __syncthreads();
  if (threadIdx.x < kPlanBuckets) {   // the first wave: where each bucket starts
    static_assert(kPlanBuckets == 64, "one bucket per lane");
    const uint32_t n = s_n[threadIdx.x];
    uint32_t upto = n;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const uint32_t v = __shfl_up(upto, o);
      if ((int)threadIdx.x >= o) upto += v;
    }
    s_at[threadIdx.x] = upto - n;
    if (threadIdx.x == kPlanBuckets - 1) plan[0] = upto;
  }
  __syncthreads();
  for (int b = threadIdx.x; b < B; b += blockDim.x) {
    int nb = nb0, base = base0, rem = rem0;
    if (b != (int)threadIdx.x) shares(b, nb, base, rem);
    const uint32_t row = (uint32_t)b << 16;
    plan[kPlanHeader + atomicAdd(&s_at[bucket(kCrowdedTailCost)], 1u)] = row;
    if (rem) {
      const uint32_t at = atomicAdd(&s_at[bucket(base + 3)], (uint32_t)rem);
      for (int i = 0; i < rem; ++i) plan[kPlanHeader + at + i] = row | (uint32_t)(1 + i);
    }
    if (nb - rem) {
      const uint32_t at = atomicAdd(&s_at[bucket(base + 2)], (uint32_t)(nb - rem));
      for (int i = rem; i < nb; ++i) plan[kPlanHeader + at + i - rem] = row | (uint32_t)(1 + i);
    }
  }
}

// How many of the first splits of a (batch row, kv head) take its tail (see wave_work).
__device__ __forceinline__ int tail_splits(const SeqCounts& c, int num_splits, bool crowded) {
  if (crowded) return 1;   // one after the other costs least when nothing runs beside it for free
  const int npp = body_tiles_of(c);
  return num_splits >= 4 && npp < 12 * (num_splits - 3) ? 3 : (num_splits >= 2 ? 1 : 0);
}

// Flat shares: a crowded launch over at most kFlatMaxB sequences needs no list.  The body tiles of
// all sequences (of one kv head: the heads of a sequence are alike) form one row, sequence after
// sequence, which is cut into `chunks` pieces; workgroup (chunk c, head h) walks the sequences its
// piece touches and leaves one partial per sequence, in the slot after the slots of the pieces that
// cut the same sequence before it (slot 0 is the tail's).  The launch is one round of two
// workgroups per SIMD, in which every workgroup has the same amount of work, whatever the lengths of
// the sequences are.  Every workgroup works the cuts out for itself from the sequences' counters:
// one round trip more at its start instead of a kernel ahead of the launch.
// The tails: with at most `chunks` sequences, tail j is the LAST thing the workgroup of chunk
// floor-inverse(j * chunks / B) does (the tails lie evenly over the chunks, at most one each), and that
// chunk's piece is shorter by what a tail costs, in tiles (tc).  With more sequences than chunks the
// tails have workgroups of their own behind the others.
// No sequence may be cut into more pieces than it has slots: if the pieces are too small for the
// longest sequence (num_splits - 2 whole pieces and two part ones at most), first the tails' cost
// is left out of the account, then the pieces take the fixed size that fits the longest sequence
// and the last chunks stay empty.
constexpr int kFlatMaxB = 256;
// A tail's cost in body tiles.  By its bytes (96 KB of fp16 rows at most) it is 9; under the load of
// the streaming workgroups its scattered rows take longer (ragged batch of 64: 83.5 us with 9, 78.3
// with 12, 78.6 with 15, 80.3 with 18).  A cost per sequence, a base plus the tail's tokens over a
// divisor, did no better than one number for all (four pairs tried: +0 to +5 us).
constexpr int kFlatTailCost = 12;
struct FlatPlan {
  int total;         // body tiles of all sequences
  int chunks, B;
  int fixed;         // 0: piece c starts at bound(c) below; else at c * fixed
  int tc;            // what a tail takes off its chunk's piece
  uint64_t step_w;   // (total + tc * B) / chunks, in units of 2^-20
  uint32_t step_b;   // B / chunks in units of 2^-20; 0: the tails have workgroups of their own
};
// tails [tails_before(c), tails_before(c + 1)) belong to chunk c
__device__ __forceinline__ int flat_tails_before(const FlatPlan& p, int c) {
  return c >= p.chunks ? p.B : (int)(((uint64_t)(uint32_t)c * p.step_b) >> 20);
}
__device__ __forceinline__ int flat_bound(const FlatPlan& p, int c) {
  if (p.fixed) return min(p.total, c * p.fixed);
  if (c >= p.chunks) return p.total;
  return (int)(((uint64_t)(uint32_t)c * p.step_w) >> 20) - p.tc * flat_tails_before(p, c);
}
// the piece that holds tile `pos` of the row: the last one that starts at or before it
__device__ __forceinline__ int flat_chunk_of(const FlatPlan& p, int pos) {
  if (p.fixed) return pos / p.fixed;
  int lo = 0, hi = p.chunks;   // bound(lo) <= pos < bound(hi)
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (flat_bound(p, mid) <= pos) lo = mid; else hi = mid;
  }
  return lo;
}
// The cuts, from the row's length and the longest sequence (wave-uniform arithmetic).  Without the
// fixed size a piece has at least floor(row / chunks) - tc >= 1 tiles: the bounds rise strictly.
__device__ __forceinline__ FlatPlan flat_decide(int total, int longest, int B, int chunks, int num_splits,
                                                bool tails_apart) {
  FlatPlan p;
  p.total = total;
  p.chunks = chunks;
  p.B = B;
  p.step_b = tails_apart ? 0u : (uint32_t)(((uint64_t)(uint32_t)B << 20) / (uint32_t)chunks);
  p.tc = tails_apart ? 0 : kFlatTailCost;
  // A sequence cut into m pieces holds m - 2 whole ones: if any num_splits - 2 pieces in a row add
  // up to the longest sequence or more, no sequence has more than num_splits - 1 pieces.  They add up
  // to at least their number times the whole part of the quotient, less the tails among them.
  const int k = num_splits - 2;
  const int tails_in_k = (int)(((uint64_t)(uint32_t)k * p.step_b) >> 20) + 1;
  uint32_t row = (uint32_t)total + (uint32_t)(p.tc * B);
  uint32_t whole = row / (uint32_t)chunks;
  auto fits_with = [&](uint32_t whole_part, int tc) {
    return (int)whole_part - tc >= 1 && (int64_t)k * whole_part - (int64_t)tc * tails_in_k >= longest;
  };
  if (p.tc && !fits_with(whole, p.tc)) {
    p.tc = 0;
    row = (uint32_t)total;
    whole = row / (uint32_t)chunks;
  }
  p.fixed = fits_with(whole, p.tc) ? 0 : max(1, c_div_up(longest, k));
  const uint32_t rest = row - whole * (uint32_t)chunks;   // rest < chunks <= 2^11
  p.step_w = ((uint64_t)whole << 20) + ((rest << 20) / (uint32_t)chunks);
  return p;
}
// The chunk and the kv head of a workgroup that streams body tiles.  (The tails then lie on every
// n-th chunk, i.e. evenly over the XCDs and, as workgroups i and i + half of the launch share a SIMD,
// two to a SIMD.  Measured and dropped, ragged batch of 64: tails paired with streaming workgroups
// on a SIMD +3 %, tails in blocks of 4 / 8 / 32 consecutive chunks +1 %, all tails on two XCDs +9 %.)
__device__ __forceinline__ int flat_chunk_of_block(int H) { return blockIdx.x / H; }
__device__ __forceinline__ int flat_head_of_block(int H) { return blockIdx.x % H; }
// What a workgroup keeps in LDS of the plan: where sequence b begins in the row (b = 0 .. B), the
// row's length and the longest sequence.  It lies in the part of the second K buffer that the tail's
// staging of fp16 rows does not reach.
struct FlatTable {
  uint32_t starts[kFlatMaxB + 1];
  int total, longest;
};
constexpr int kFlatTableOff = kKTile + (10240 - kKTile);   // from the first K buffer: behind the 10240 bytes of staging
static_assert(kFlatTableOff + sizeof(FlatTable) <= 2 * kKTile, "the table fits behind the staging area");
// ends[k]: where this lane's sequence 4 * lane + k ends in the row
__device__ __forceinline__ void flat_scan(const kitty_kv_layer& L, int B, FlatTable& T, int (&ends)[4]) {
  const int lane = threadIdx.x;
  int nb[4], sum = 0, longest = 0;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int b = 4 * lane + k;
    nb[k] = b < B ? body_tiles_of(load_counts(L, min(b, B - 1))) : 0;
    sum += nb[k];
    longest = max(longest, nb[k]);
  }
  int upto = sum;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(upto, o);
    if (lane >= o) upto += v;
  }
#pragma unroll
  for (int o = 32; o; o >>= 1) longest = max(longest, __shfl_xor(longest, o));
  int at = upto - sum;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    T.starts[4 * lane + k] = (uint32_t)at;
    at += nb[k];
    ends[k] = at;
  }
  if (lane == 63) {
    T.starts[256] = (uint32_t)at;
    T.total = at;
    T.longest = longest;
  }
  wave_lds_fence();
}

// What one wave does.  DMA: packed tiles are streamed global -> LDS (G <= 8); otherwise they are
// loaded into registers.  QUARTER (needs DMA; at most 4 query heads per kv head): body pages go
// through combine_quarter / softmax_quarter / pv_quarter.
// MODE: kWaveSolo - the launch has one split, whose wave does everything; kWaveBody - a split with
// body tiles only; kWaveTail - a split with the sink and / or tiles with fp16 rows only.  The last
// two are different FUNCTIONS (the kernel calls the tail's one without inlining it), not branches of
// one: the tail's code needs every register there is and spills, and as a branch of the function
// that holds the streaming loop it costs the loop, which it never runs beside, several percent - the
// loop's code comes out with half again as many wait states and 256 registers instead of 162, and
// when the pressure is on the wrong side of the edge, with spills of its own (a reload inside the
// loop is a vector load that the hand-counted waits do not know of).
enum WaveMode { kWaveSolo, kWaveBody, kWaveTail };
template <bool BOOST, bool DMA, bool QUARTER, WaveMode MODE, bool FLAT = false, class LDS>
__device__ __forceinline__ void wave_work(const kitty_kv_layer& L, const __half* __restrict__ q, int H_Q, float scaling,
                                          float* __restrict__ ws_ml, float* __restrict__ ws_acc, int num_splits,
                                          int n_simds, const WorkItem& w, LDS& S) {
  static_assert(DMA || !QUARTER, "quarter columns are a variant of the LDS-streamed kernel");
  Ctx x;
  x.L = &L;
  x.bad_page = 0;
  x.b = w.b;
  x.h = w.h;
  const int split = w.split;
  x.lane = threadIdx.x;
  x.kg = x.lane >> 4;
  x.n = x.lane & 15;
  // A body wave's start is a chain of round trips: counters, query rows, page ids, first tiles.  The
  // query rows of a quarter-column body wave do not go through registers the compiler waits for: ONE
  // global -> LDS load (the four heads' rows, 1 KB, into the space of the q * scale table, which is
  // first written by the first page) is asked for before anything else and waited for by count after
  // the first tiles have been asked for, so that its latency lies under theirs.
  constexpr bool Q_VIA_LDS = QUARTER && MODE == kWaveBody;
  if constexpr (Q_VIA_LDS) {
    const int Gq = H_Q / L.H_KV;
    const uint8_t* qbase = (const uint8_t*)(q + ((int64_t)x.b * H_Q + (int64_t)x.h * Gq) * kD);
    lds_dma<1, 16>((uint32_t)(min(x.lane >> 4, Gq - 1) * (kD * 2) + (x.lane & 15) * 16), qbase,
                   (uint32_t)(uintptr_t)&S.qs[0][0]);   // row r of the table's space: head min(r, G - 1)
  }
  x.c = load_counts(L, x.b);
  x.lane_off = (4 * x.kg + (x.n & 1)) * kRowBytes + (x.n >> 1) * 4;
  x.sel = (x.n & 1) ? 0x03020706u : 0x05040100u;
  x.sc2 = scaling * kLog2e;
  const int G = H_Q / L.H_KV;
  constexpr bool SPLIT_COLS = DMA;   // both mean "at most 8 query heads per kv head"
  // quarter columns: column n carries head slot n % 4 (a slot past the last head repeats it; its
  // columns are never written)
  x.g = QUARTER ? min(x.n & 3, G - 1) : SPLIT_COLS ? (x.n & 7) % G : x.n % G;
  x.lo_part = SPLIT_COLS && (x.n & 8);
  x.pi_own = ((x.n >> 2) & 1) * 2 + (x.n >> 3);
  {
    const int u_own = 2 * x.pi_own;   // code_unscale wants a constant: pick from the eight
    float us[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) us[u] = code_unscale(u) * x.sc2;
    x.usc[0] = x.usc[1] = 0.f;
#pragma unroll
    for (int u = 0; u < 8; u += 2) {
      if (u == u_own) { x.usc[0] = us[u]; x.usc[1] = us[u + 1]; }
    }
  }
  x.ktr = (4 * x.kg + (x.n >> 2)) * kRowBytes + (x.n & 3) * 8;
  x.vtr = (32 * x.kg + (x.n >> 2)) * kRowBytes + (x.n & 3) * 8;

  // q of this column: operand-order pairs in registers, natural order in LDS for the slot gather
  const __half* qrow = q + ((int64_t)x.b * H_Q + (int64_t)x.h * G + x.g) * kD;
  if constexpr (!Q_VIA_LDS) {
#pragma unroll
    for (int kc = 0; kc < 4; ++kc)
#pragma unroll
      for (int pi = 0; pi < 4; ++pi) x.qpair[kc * 4 + pi] = *(const uint32_t*)(qrow + 32 * kc + krow(pi, x.kg));
  }
  // the tables of the generic QK / PV path: q in natural order for the slot gather, a zero entry
  // for "no channel", a row of ones
  auto stage_generic_tables = [&]() {
    if (x.n < G) {   // one copy per head
      const uint4* src = (const uint4*)(qrow + 32 * x.kg);
      uint4* dst = (uint4*)&S.q_nat[x.g][32 * x.kg];
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[i] = src[i];
      if (x.kg == 0) S.q_nat[x.g][128] = (_Float16)0.0f;
    }
    if (x.lane == 0) S.ks4_nat[128] = (_Float16)0.0f;
    S.ones[x.lane] = 0x3C003C00u;
    wave_lds_fence();
  };
  if constexpr (QUARTER) {
    // the generic tables share the V tile's space and are staged before the tail tiles instead
#pragma unroll
    for (int t = 0; t < 4; ++t) S.vs_q[t][x.lane] = 0u;
    if (x.lane < 4) S.ones4[x.lane] = 0x3C003C00u;
    if constexpr (!Q_VIA_LDS) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        x.q4[r] = *(const uint32_t*)(q + ((int64_t)x.b * H_Q + (int64_t)x.h * G + min(r, G - 1)) * kD + 2 * x.lane);
    }
    const int row = x.g + (x.lo_part ? 4 : 0);
    x.qs_rd = row * (kQsPitch * 4) + 8 * x.kg;
    x.qb_rd = row * 64 + 8 * x.kg;
    wave_lds_fence();
  } else {
    stage_generic_tables();
  }

  Acc A;
#pragma unroll
  for (int u = 0; u < 8; ++u) A.out[u] = float4v{0.f, 0.f, 0.f, 0.f};
  A.m = 0.f;
  A.lz = float4v{0.f, 0.f, 0.f, 0.f};
  A.first = true;
  A.true_units = false;

  // Work of one (batch row, kv head): the tiles with both sides packed ("body"), and the slow rest
  // ("tail": the sink, and the one or two tiles with fp16 rows on either side).  The tail takes the
  // FIRST splits, so that its long-latency waves start with the launch and run beside the body: one
  // split when a body split is long enough to hide it (12 tiles or more), else three (sink / first
  // tail tile / the others).  The remaining splits share the body evenly (tile counts differ by at
  // most one).  1 split: everything.
  // (Measured and dropped: no wave of its own for the tail but three splits that take one tail unit
  // each after a body share shortened by the unit's cost.  With all 16 splits of a 32k context
  // streaming, the body alone takes 4 us longer than with 15 streaming and one idle, and the gain
  // from hiding the tail is spent.)
  const int nbt = c_div_up(x.c.nbody, kPage);
  const int npp = min(min(x.c.pv, x.c.pk), nbt);
  const int n_tail = tail_splits(x.c, num_splits, w.crowded);
  int t0 = 0, t1 = 0;          // body tiles of this split: t1 - t0 of them, from tile first_tile in steps of tile_step
  int first_tile = 0, tile_step = 1;
  int u0 = nbt, u1 = nbt;      // tail tiles of this split
  bool do_sink = false;
  if constexpr (FLAT) {
    if constexpr (MODE == kWaveTail) { u0 = npp; do_sink = true; }
    else { t0 = w.t0; t1 = w.t1; }
  } else if (num_splits == 1) {
    t1 = npp; u0 = npp; do_sink = true;
  } else if (split < n_tail) {
    if (n_tail == 1) { u0 = npp; do_sink = true; }
    else if (split == 0) do_sink = true;
    else if (split == 1) { u0 = npp; u1 = min(nbt, npp + 1); }
    else u0 = min(nbt, npp + 1);
  } else {
    // even shares: the first npp % n_body splits take one tile more.  A crowded launch gives a short
    // sequence fewer, longer shares; the splits past them have nothing to do.
    const int i_body = split - n_tail;
    const int n_body = w.crowded ? crowded_body_splits(npp, num_splits) : num_splits - n_tail;
    if (i_body < n_body) {
      const int base = npp / n_body, rem = npp - base * n_body;
      t0 = i_body * base + min(i_body, rem);
      t1 = t0 + base + (i_body < rem ? 1 : 0);
      // The splits of a sequence take its tiles in turn - split i the tiles i, i + n_body, ... (as many
      // as its even share) - rather than a range each: the workgroups of a sequence then read
      // neighbouring pages, page-table entries and (scale, zero) blocks at about the same time instead of
      // fifteen places 17 pages apart.  16 sequences of 32k tokens: 60.3 against 62.6 us (61.3 against
      // 63.7 on a slower box; 60.8 against 62.0 with the pages scattered over the cache at random);
      // dealt in groups of two or four tiles: 65.5 / 68.8.  Shares of a few tiles stay ranges (1 sequence
      // of 128k tokens over 240 splits: 26.05 us in turn against 25.85), and so do a crowded launch's.
      if (!w.crowded && base >= 8) { first_tile = i_body; tile_step = n_body; }
    }
  }
  const bool tail = MODE != kWaveBody && (do_sink || u0 < u1);
  const uint8_t* qbuf_k = (const uint8_t*)L.qbuf_k + (int64_t)x.b * L.win_stride_b + (int64_t)x.h * L.win_stride_h;

  float4v C[8];
  if constexpr (MODE == kWaveTail) {
    t1 = t0;   // (a split with tail work has no body tiles; this tells the compiler)
  }
  if constexpr (MODE != kWaveTail && DMA) {
    // Tiles stream through LDS, one K tile and one V tile at a time: a buffer is asked to be filled
    // again as soon as its tile has been consumed.  Issue order
    //   K(t0) V(t0) | QK(i) -> K(i+1) -> softmax -> PV(i) -> V(i+1) | ...
    // so each tile has a lead of half an iteration.  (A second K buffer with a lead of one and a
    // half iterations was 2.6 % slower at 32k tokens x 16 sequences and 3.5 % at 128k x 1: the
    // memory system serves this many concurrent streams better with less in flight.)  The waits
    // count the instructions issued AFTER the tile that is needed; nothing is loaded past the end
    // of the range (the last iteration waits on a shorter queue).
    if (t0 < t1) {
      if constexpr (!Q_VIA_LDS) settle_prologue_loads();   // (else: no load of the prologue fills a register the loop reads)
      constexpr int nK = kDmaK<BOOST>;
      const uint32_t lk0 = (uint32_t)(uintptr_t)&S.kbuf[0][0];
      const uint32_t lv = (uint32_t)(uintptr_t)&S.vbuf[0];
      if (tile_step == 1) first_tile = t0;
      int tile = first_tile;   // of loop index i
      dma_k<BOOST>(x, tile, lk0);
      dma_v(x, tile, lv);
      if constexpr (Q_VIA_LDS) {
        // the query rows were asked for before these tiles: everything older than the tiles has landed
        wait_vmcnt<nK + kDmaV>();
        const _Float16* ql = (const _Float16*)&S.qs[0][0];
#pragma unroll
        for (int kc = 0; kc < 4; ++kc)
#pragma unroll
          for (int pi = 0; pi < 4; ++pi)
            x.qpair[kc * 4 + pi] = *(const uint32_t*)(ql + (x.n & 3) * kD + 32 * kc + krow(pi, x.kg));
#pragma unroll
        for (int r = 0; r < 4; ++r) x.q4[r] = *(const uint32_t*)(ql + r * kD + 2 * x.lane);
        wave_lds_fence();   // (the table's first write comes after these reads: LDS executes a wave's instructions in order)
      }
      // Of the two waves that share a SIMD the older one wins arbitration, and it is 8 % faster per
      // tile.  When the launch is a single round (at most two workgroups per SIMD of the device; a
      // launch of flat shares is one: 2 % on the ragged batch of 64),
      // the workgroups dispatched after every SIMD has one are the younger ones: they raise their
      // priority by one level after the first quarter of their range, which evens out the finishes.
      // (Two copies of the loop: the conditional priorities cost the other launches 1.5 %.)
      const uint32_t kSimds = (uint32_t)n_simds;
      const uint32_t n_wg = gridDim.x * gridDim.y * gridDim.z;
      const uint32_t lin_id = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
      const bool young = (FLAT || !w.crowded) && n_wg <= 2 * kSimds && lin_id >= kSimds;
      auto loop = [&](auto switch_priority) {
      constexpr bool SWITCH = decltype(switch_priority)::value;
#pragma unroll 1
      for (int i = t0; i < t1; ++i) {
        float cz;
        const bool k1 = i + 1 < t1;
        const bool fav = SWITCH && 4 * (i - t0) >= t1 - t0;
        // K(i) is followed in the queue by V(i-1) (not in the first iteration), K(i+1) if any, V(i)
        wait_vmcnt<kDmaV>();   // K(i) is followed by V(i)
        if (fav) __builtin_amdgcn_s_setprio(KITTY_PRIO_MFMA + 1); else __builtin_amdgcn_s_setprio(KITTY_PRIO_MFMA);
        if constexpr (QUARTER) qk_packed_tab<BOOST>(S, x, S.kbuf[0], C, cz);
        else qk_packed<BOOST, SPLIT_COLS>(S, x, KLds{S.kbuf[0]}, C, cz);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (k1) dma_k<BOOST>(x, tile + tile_step, lk0);
        if (fav) __builtin_amdgcn_s_setprio(KITTY_PRIO_VALU + 1); else __builtin_amdgcn_s_setprio(KITTY_PRIO_VALU);
        if constexpr (QUARTER) {
          float4v own[2];
          combine_quarter(x, C, own);
          softmax_quarter(x, A, own, cz);
          if (k1) wait_vmcnt<nK>(); else wait_vmcnt<0>();
          if (fav) __builtin_amdgcn_s_setprio(KITTY_PRIO_MFMA + 1); else __builtin_amdgcn_s_setprio(KITTY_PRIO_MFMA);
          pv_quarter(S, x, A.out, A.lz, VLds{S.vbuf}, own);
        } else {
          softmax_tile<true>(x, A, C, cz, kPage);
          if (k1) wait_vmcnt<nK>(); else wait_vmcnt<0>();
          if (fav) __builtin_amdgcn_s_setprio(KITTY_PRIO_MFMA + 1); else __builtin_amdgcn_s_setprio(KITTY_PRIO_MFMA);
          pv_packed(S, x, A.out, A.lz, VLds{S.vbuf}, C);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (k1) dma_v(x, tile + tile_step, lv);
        tile += tile_step;
      }
      };
      if (young) loop(std::true_type{}); else loop(std::false_type{});
      wait_vmcnt<0>();
    }
  } else if constexpr (MODE != kWaveTail) {
    // Register-fed software pipeline: the V words of tile i are in flight during its QK phase,
    // the K words of tile i+1 during its softmax and PV phase.
    KRegs kb;
    VRegs vb;
    if (t0 < t1) k_load_regs<BOOST>(x, t0, kb);
#pragma unroll 1
    for (int i = t0; i < t1; ++i) {
      float cz;
      v_load_regs(x, i, vb);
      qk_packed<BOOST, SPLIT_COLS>(S, x, kb, C, cz);
      // unconditional (the last iteration re-loads its own tile) so that the number of loads in
      // flight is static and the PV phase only waits for the V words, not for this prefetch
      k_load_regs<BOOST>(x, min(i + 1, t1 - 1), kb);
      softmax_tile<true>(x, A, C, cz, kPage);
      pv_packed(S, x, A.out, A.lz, vb, C);
    }
  }
  if (MODE != kWaveBody && tail) {
    if constexpr (QUARTER) stage_generic_tables();   // the V tile is idle from here on
    to_true_units(A);
    KRegs kb;
    VRegs vb;
#pragma unroll 1
    for (int i = u0; i < u1; ++i) {
      float cz = 0.f;
      const int ntok = min(kPage, x.c.nbody - i * kPage);
      if (i < x.c.pk) {
        k_load_regs<BOOST>(x, i, kb);
        qk_packed<BOOST, SPLIT_COLS>(S, x, kb, C, cz);
        softmax_tile<true>(x, A, C, cz, ntok);
      } else {
        qk_fp16(S, x, qbuf_k, ntok, C);
        softmax_tile<false>(x, A, C, 0.f, ntok);
      }
      if (i < x.c.pv) {
        // a packed V page under fp16 keys (only reachable with hand-made counters): accumulate in
        // code units on the side, then fold in
        float4v tmp[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) tmp[u] = float4v{0.f, 0.f, 0.f, 0.f};
        v_load_regs(x, i, vb);
        if (QUARTER && x.pi_own != 0) {
#pragma unroll
          for (int u = 0; u < 8; ++u) C[u] = float4v{0.f, 0.f, 0.f, 0.f};
        }
        pv_packed(S, x, tmp, A.lz, vb, C);
#pragma unroll
        for (int u = 0; u < 8; ++u) A.out[u] += tmp[u] * code_unscale(u);
      } else {
        pv_fp16<false, QUARTER>(&S.kbuf[0][0], x, A, (i - x.c.pv) * kPage, ntok, C);
      }
    }
    if (do_sink && x.c.sink > 0) {
      const uint8_t* sink_k = (const uint8_t*)L.sink_k + (int64_t)x.b * L.sink_stride_b + (int64_t)x.h * L.sink_stride_h;
      qk_fp16(S, x, sink_k, x.c.sink, C);
      softmax_tile<false>(x, A, C, 0.f, x.c.sink);
      pv_fp16<true, QUARTER>(&S.kbuf[0][0], x, A, 0, x.c.sink, C);
    }
  }
  to_true_units(A);

  report_bad_page(L, x.b, x.bad_page);
  // ---- partial of this split: columns n < G are the G heads -----------------------------------
  float l = A.lz[0], z = A.lz[1];
  if constexpr (QUARTER) {
    // the four columns of a head hold partial sums over their own tokens (the tail's tiles went to
    // pi_own = 0 alone); sum p * zero_v of a column sits in row 2 pi_own + 1, which this lane holds
    // if its lane group is even (pi_own 0, 1) or odd (pi_own 2, 3) accordingly
    l += ror4(l);
    l += ror8(l);
    z = (x.pi_own & 1) ? A.lz[3] : A.lz[1];
    z = ((x.pi_own >> 1) == (x.kg & 1)) ? z : 0.f;
    z += ror4(z);
    z += ror8(z);
    z += __shfl_xor(z, 16);
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float v = A.out[u][j];
        v += ror4(v);
        v += ror8(v);
        A.out[u][j] = v;
      }
  }
  if (x.n < G) {
    const int64_t row = ((int64_t)x.b * H_Q + (int64_t)x.h * G + x.n) * num_splits + split;
    if (x.kg == 0) {
      ws_ml[row * 2] = A.first ? -INFINITY : A.m;
      ws_ml[row * 2 + 1] = l;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j) ws_acc[row * kD + 32 * x.kg + 8 * j + u] = A.out[u][j] + z;
  }
  if constexpr (MODE == kWaveTail) {
    // a crowded launch has no workgroups for the splits without work: the tail's split marks their
    // partials as empty (the merge pass then does not read their accumulator rows)
    if (w.crowded) {
      const int s0 = FLAT ? w.n_used : 1 + crowded_body_splits(npp, num_splits);
      const int n_empty = num_splits - s0;
      for (int i = x.lane; i < G * n_empty; i += 64) {
        const int g = i / n_empty, s = s0 + i - g * n_empty;
        const int64_t row = ((int64_t)x.b * H_Q + (int64_t)x.h * G + g) * num_splits + s;
        ws_ml[row * 2] = -INFINITY;
        ws_ml[row * 2 + 1] = 0.f;
      }
    }
  }
}

// The kernel's arguments, as one struct: the tail's function reads them where they lie.
struct KernArgs {
  kitty_kv_layer L;
  const __half* q;
  int H_Q;
  float scaling;
  float* ws_ml;
  float* ws_acc;
  int num_splits, n_simds;
  const uint32_t* plan;   // the work list of a crowded launch (see WorkItem), else NULL
  int B, flat_chunks;     // flat shares (see FlatPlan): sequences, chunks (workgroups per kv head that stream body tiles)
  bool flat_tails_apart;  // flat shares: the tails have workgroups of their own
};

__device__ __forceinline__ const KernArgs& kernel_args_of(const KernArgs* p) {   // the address as a scalar again
  const uint64_t v = (uint64_t)(uintptr_t)p;
  const uint64_t u = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(v >> 32)) << 32) |
                     (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  return *(const KernArgs*)(const __attribute__((address_space(4))) KernArgs*)(uintptr_t)u;
}

// The tail's function: a call, not a branch (see wave_work).  Arguments of a function arrive in
// vector registers, which the compiler takes for different from lane to lane - every branch on them
// a divergent one, every load through them a vector load.  So the function gets addresses, made
// scalars again on arrival: of the kernel's argument block (the intrinsic that names it is only
// valid in the kernel itself) and of the wave's LDS.  This one ends the wave: nothing of the
// caller's needs saving.
template <bool BOOST, bool DMA, bool QUARTER>
__device__ __attribute__((noinline, noreturn)) void tail_wave(const KernArgs* kernel_args,
                                                               __attribute__((address_space(3))) WaveLds<DMA, QUARTER>* lds) {
  const KernArgs& a = kernel_args_of(kernel_args);
  const WorkItem w = work_item_of_block(a.L.H_KV, a.plan);
  wave_work<BOOST, DMA, QUARTER, kWaveTail>(a.L, a.q, a.H_Q, a.scaling, a.ws_ml, a.ws_acc, a.num_splits, 0, w,
                                             *(WaveLds<DMA, QUARTER>*)lds);
  __builtin_amdgcn_endpgm();
}
// A crowded launch with flat shares (see FlatPlan): workgroups [0, flat_chunks * H_KV) stream body
// tiles - chunk = id / H_KV of head id % H_KV - and then take the chunk's tail, if it has one; the
// workgroups behind them (flat_tails_apart) take the tail of one (sequence, head) each.  The tail's
// function marks the sequence's unused partials as empty and ends the wave.
template <bool BOOST, bool QUARTER>
__device__ __attribute__((noinline, noreturn)) void flat_tail_wave(const KernArgs* kernel_args,
                                                                    __attribute__((address_space(3))) WaveLds<true, QUARTER>* lds) {
  const KernArgs& a = kernel_args_of(kernel_args);
  WaveLds<true, QUARTER>& S = *(WaveLds<true, QUARTER>*)lds;
  const FlatTable& T = *(const FlatTable*)(&S.kbuf[0][0] + kFlatTableOff);
  const int H = a.L.H_KV, id = blockIdx.x, n_body = a.flat_chunks * H;
  const FlatPlan P = flat_decide(__builtin_amdgcn_readfirstlane(T.total), __builtin_amdgcn_readfirstlane(T.longest), a.B,
                                 a.flat_chunks, a.num_splits, a.flat_tails_apart);
  const int b = id >= n_body ? (id - n_body) / H : flat_tails_before(P, flat_chunk_of_block(H));
  const int s = __builtin_amdgcn_readfirstlane((int)T.starts[b]), e = __builtin_amdgcn_readfirstlane((int)T.starts[b + 1]);
  const int pieces = e > s ? flat_chunk_of(P, e - 1) - flat_chunk_of(P, s) + 1 : 0;
  const WorkItem w{b, id >= n_body ? id % H : flat_head_of_block(H), 0, true, true, 0, 0, 1 + pieces};
  wave_work<BOOST, true, QUARTER, kWaveTail, true>(a.L, a.q, a.H_Q, a.scaling, a.ws_ml, a.ws_acc, a.num_splits, 0, w, S);
  __builtin_amdgcn_endpgm();
}
template <bool BOOST, bool QUARTER>
__global__ __launch_bounds__(64, 2) void decode_mfma_flat_kernel(KernArgs a) {
  __shared__ WaveLds<true, QUARTER> S;
  static_assert(sizeof(S.kbuf) == 2 * kKTile, "the plan's table lies in the second K buffer");
  FlatTable& T = *(FlatTable*)(&S.kbuf[0][0] + kFlatTableOff);
  const int H = a.L.H_KV;
  int ends[4];
  flat_scan(a.L, a.B, T, ends);
  auto tail = [&]() {
    flat_tail_wave<BOOST, QUARTER>(
        (const KernArgs*)(const __attribute__((address_space(4))) KernArgs*)__builtin_amdgcn_kernarg_segment_ptr(),
        (__attribute__((address_space(3))) WaveLds<true, QUARTER>*)&S);
  };
  if ((int)blockIdx.x >= a.flat_chunks * H) tail();
  const FlatPlan P = flat_decide(__builtin_amdgcn_readfirstlane(T.total), __builtin_amdgcn_readfirstlane(T.longest), a.B,
                                 a.flat_chunks, a.num_splits, a.flat_tails_apart);
  const int c = flat_chunk_of_block(H), h = flat_head_of_block(H);
  const int lo = flat_bound(P, c), hi = flat_bound(P, c + 1);
  const bool has_tail = !a.flat_tails_apart && flat_tails_before(P, c + 1) > flat_tails_before(P, c);
  if (lo < hi) {
    // the first sequence of the piece: as many sequences end at or before its first tile
    int b = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) b += __popcll(__ballot(4 * (int)threadIdx.x + k < a.B && ends[k] <= lo));
    int slot = -1;   // of the first sequence: found by search; the others begin inside the piece
#pragma unroll 1
    for (; b < a.B; ++b) {
      const int s = __builtin_amdgcn_readfirstlane((int)T.starts[b]), e = __builtin_amdgcn_readfirstlane((int)T.starts[b + 1]);
      if (s >= hi) break;
      if (e <= s) continue;
      if (slot < 0) slot = min(1 + c - flat_chunk_of(P, s), a.num_splits - 1); else slot = 1;   // (the plan keeps it below num_splits; the workspace ends there)
      const WorkItem w{b, h, slot, true, true, max(lo, s) - s, min(hi, e) - s, 0};
      wave_work<BOOST, true, QUARTER, kWaveBody, true>(a.L, a.q, a.H_Q, a.scaling, a.ws_ml, a.ws_acc, a.num_splits,
                                                       a.n_simds, w, S);
    }
  }
  if (has_tail) tail();
}

// SOLO: the launch has one split.  Otherwise the first tail_splits() splits of a (batch row, kv head)
// go through tail_wave and the others stream the body.
template <bool BOOST, bool DMA, bool QUARTER, bool SOLO>
__global__ __launch_bounds__(64, 2) void decode_mfma_kernel(KernArgs a) {
  __shared__ WaveLds<DMA, QUARTER> S;
  const WorkItem w = work_item_of_block(a.L.H_KV, a.plan);
  if (!w.valid) return;
  if constexpr (SOLO) {
    wave_work<BOOST, DMA, QUARTER, kWaveSolo>(a.L, a.q, a.H_Q, a.scaling, a.ws_ml, a.ws_acc, a.num_splits, a.n_simds, w, S);
  } else {
    if (w.split < tail_splits(load_counts(a.L, w.b), a.num_splits, w.crowded)) {
      tail_wave<BOOST, DMA, QUARTER>(
          (const KernArgs*)(const __attribute__((address_space(4))) KernArgs*)__builtin_amdgcn_kernarg_segment_ptr(),
          (__attribute__((address_space(3))) WaveLds<DMA, QUARTER>*)&S);
    }
    wave_work<BOOST, DMA, QUARTER, kWaveBody>(a.L, a.q, a.H_Q, a.scaling, a.ws_ml, a.ws_acc, a.num_splits, a.n_simds, w, S);
  }
}

}  // namespace

bool decode_mfma_supported(const kitty_kv_layer& L, int H_Q) {
  return (L.D_BOOSTED == 32 || L.D_BOOSTED == 0) && L.D == kD && L.PAGE_SIZE == kPage && H_Q / L.H_KV <= 16;
}

// ev_start / ev_stop (both or neither): events attached to the kernel's own dispatch, which then hold
// the moments the kernel began and ended on the device (what a kernel trace reports) rather than the
// moments the host enqueued around it.
namespace {
struct LaunchArgs {
  KernArgs k;
  int B;
  hipStream_t stream;
  hipEvent_t ev_start, ev_stop;
};
template <bool BOOST, bool QUARTER>
void launch_flat(const LaunchArgs& a) {
  const dim3 grid((uint32_t)((a.k.flat_chunks + (a.k.flat_tails_apart ? a.B : 0)) * a.k.L.H_KV)), block(64);
  if (a.ev_start)
    hipExtLaunchKernelGGL((decode_mfma_flat_kernel<BOOST, QUARTER>), grid, block, 0, a.stream, a.ev_start, a.ev_stop, 0, a.k);
  else
    hipLaunchKernelGGL((decode_mfma_flat_kernel<BOOST, QUARTER>), grid, block, 0, a.stream, a.k);
}
template <bool BOOST, bool DMA, bool QUARTER, bool SOLO>
void launch_one(const LaunchArgs& a) {
  if constexpr (DMA && !SOLO) {
    if (a.k.flat_chunks > 0) return launch_flat<BOOST, QUARTER>(a);
  }
  const bool crowded = a.k.plan != nullptr;
  const dim3 grid = crowded ? dim3((uint32_t)(a.B * a.k.L.H_KV * a.k.num_splits), 1, 1)
                            : dim3(a.k.num_splits, a.k.L.H_KV, a.B);
  const dim3 block(64);
  // a crowded launch is two kernels: the events take in both
  if (crowded) {
    uint32_t* plan = const_cast<uint32_t*>(a.k.plan);
    if (a.ev_start)
      hipExtLaunchKernelGGL(decode_plan_kernel, dim3(1), dim3(256), 0, a.stream, a.ev_start, nullptr, 0, a.k.L, a.B,
                            a.k.num_splits, plan);
    else
      hipLaunchKernelGGL(decode_plan_kernel, dim3(1), dim3(256), 0, a.stream, a.k.L, a.B, a.k.num_splits, plan);
  }
  if (a.ev_start)
    hipExtLaunchKernelGGL((decode_mfma_kernel<BOOST, DMA, QUARTER, SOLO>), grid, block, 0, a.stream,
                          crowded ? nullptr : a.ev_start, a.ev_stop, 0, a.k);
  else
    hipLaunchKernelGGL((decode_mfma_kernel<BOOST, DMA, QUARTER, SOLO>), grid, block, 0, a.stream, a.k);
}
template <bool BOOST, bool DMA, bool QUARTER>
void launch_variant(const LaunchArgs& a) {
  if (a.k.num_splits == 1) launch_one<BOOST, DMA, QUARTER, true>(a);
  else launch_one<BOOST, DMA, QUARTER, false>(a);
}
}  // namespace

void launch_decode_mfma(const kitty_kv_layer& L, const void* q, int B, int H_Q, float scaling, float* ws_ml,
                        float* ws_acc, uint32_t* ws_plan, int num_splits, int n_simds, hipStream_t stream,
                        hipEvent_t ev_start, hipEvent_t ev_stop) {
  const int64_t n_wg = (int64_t)B * L.H_KV * num_splits;
  const bool crowded = num_splits > 1 && n_wg > 2 * (int64_t)n_simds && n_wg <= INT32_MAX;
  const int G = H_Q / L.H_KV;
  const bool boost = L.D_BOOSTED == 32, dma = G <= 8, quarter = G <= 4;
  // flat shares: a launch of one round - two workgroups per SIMD, of which the tails take theirs and
  // the body at least half
  const bool flat = crowded && dma && B <= kFlatMaxB && num_splits >= 3;
  const int all_slots = std::min(2048, std::max(1, 2 * n_simds / L.H_KV));
  const bool tails_apart = B > all_slots;
  const int flat_chunks = !flat ? 0 : !tails_apart ? all_slots : std::max(1, std::max(2 * n_simds - B * L.H_KV, n_simds) / L.H_KV);
  const LaunchArgs a{KernArgs{L, (const __half*)q, H_Q, scaling, ws_ml, ws_acc, num_splits, n_simds,
                              crowded && !flat ? ws_plan : nullptr, B, flat_chunks, tails_apart},
                     B, stream, ev_start, ev_stop};
  if (boost && quarter) launch_variant<true, true, true>(a);
  else if (boost && dma) launch_variant<true, true, false>(a);
  else if (boost) launch_variant<true, false, false>(a);
  else if (quarter) launch_variant<false, true, true>(a);
  else if (dma) launch_variant<false, true, false>(a);
  else launch_variant<false, false, false>(a);
}

}  // namespace kitty
