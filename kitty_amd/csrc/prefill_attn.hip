// Chunked-prefill attention: T_q new tokens attend, causally among themselves, to everything the
// cache already holds (sink rows, packed pages, fp16 windows) and to the new chunk's own keys
// and values.  The reference has no such kernel (its prefill runs dense flash attention on an
// empty cache, benchmark_kitty.py:302, and kitty_attention.py:411 asserts t_query == 1); the
// arithmetic is the same as decode: softmax(q . k^ * scaling) . v^ with
// k^ = fp16(code) * scale + zero evaluated in fp16 (kitty_attention.py:162-165, 317-320).
//
// The work is a dense contraction (G * T_q query rows per KV head), so it runs on the matrix
// cores, flash-attention style.  One workgroup of 4 wavefronts owns 256 query rows of one
// (batch row, KV head): PB = 256 / G consecutive chunk positions times the G query heads of the
// group; wavefront w owns rows 64w .. 64w+63.  The workgroup walks the sequence in 128-token
// tiles.  Each tile is brought into LDS once, as fp16, by all 256 threads: packed pages are
// dequantized on the way (exactly the reference's two fp16 roundings), fp16 rows are copied.
// Two tile buffers alternate: while tile t is multiplied, tile t+1 is converted into the other
// buffer and the packed bytes of tile t+2 are in flight; one barrier per tile.
//
// Matrix-core formulation (v_mfma_f32_16x16x32_f16; lane = 16 kg + n holds A[n][8 k-slots],
// B[8 k-slots][n], C[4kg .. 4kg+3][n]):
//   S^T[pos][row]  = sum_ch  K[pos][ch]  * Q[row][ch]      A = keys,   B = queries (registers)
//   O^T[cp][row]   = sum_pos V[pos][cp]  * P^T[pos][row]   A = values, B = probabilities
// The accumulator of the first product is, lane for lane, the B operand of the second: k-slot j
// of lane group kg stands for position 16 (j / 4) + 4 kg + j % 4 of a 32-position sub-tile.
//
// LDS layouts, chosen so that dequantization writes 128-bit rows and the matrix-core operands
// come out of `ds_read_b64_tr_b16` (a 16-lane block reads 4 rows x 16 columns and lane i
// receives column i of the 4 rows):
//   K tile: [channel][position]       V tile: [position][channel slot]      row pitch 288 bytes
// "position" and "channel slot" are the order in which codes fall out of a plane word when it is
// masked with 0x00030003 << 2u: slot 2u + e of a 16-block is element u + 8e.  Keys and values use
// the same token permutation, the output undoes the channel permutation.
#include "decode_common.h"

// wave priority while a wave issues the PV MFMAs (the other wave of the SIMD fills the gaps)
#define KITTY_PV_PRIO 2

namespace kitty {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));

constexpr int kPitch = 288;                   // bytes per LDS row: 128 fp16 + 32 bytes of padding
constexpr int kTile = kPage * kPitch;         // 36864 bytes, one K or V tile
constexpr int kLdsBytes = 4 * kTile;          // K and V, two buffers each
constexpr int kRows = 256;                    // query rows per workgroup
constexpr int kWaves = 8;                     // two per SIMD: one does vector work while the other feeds the matrix pipe
constexpr int kThreads = 64 * kWaves;
constexpr int kNT = kRows / (16 * kWaves);    // 16-row column tiles per wave
constexpr int kParts = kThreads / 128;        // threads that share one row of a tile while staging it
constexpr int kW = 8 / kParts;                // 16-code words of a packed row per thread
constexpr int kPartBytes = 256 / kParts;      // bytes of an fp16 row per thread
constexpr float kLog2e = 1.4426950408889634f;

enum SrcKind : int { SRC_PACKED = 0, SRC_ROWS = 1, SRC_VTAIL = 2 };

// where the keys and the values of one 128-token tile come from
struct TileSrc {
  int k_kind, v_kind;
  const uint8_t* k_ptr;   // packed: the page-head;  rows: first row
  const uint8_t* k_meta;
  const uint8_t* v_ptr;
  const uint8_t* v_meta;
  int64_t k_stride, v_stride;   // rows: bytes between tokens
  int v_u0;                     // v-tail: index of the tile's first token in [Q_Buffer_V | ring]
  int ntok;                     // valid tokens
  int chunk_t0;                 // >= 0: tile of the new chunk starting at this chunk position
};

// what issue() leaves in flight for a packed tile (fp16 rows are few and are copied by finish())
struct Stage {
  uint32_t klo[kW], khi[kW], v[kW];
  uint32_t kmeta, vmeta;
};

__device__ __forceinline__ int slot_of(int e) {   // element (token or channel) -> LDS slot
  return (e & ~15) | ((e & 7) << 1) | ((e >> 3) & 1);
}

__device__ __forceinline__ half4 lds_tr(const uint8_t* p) {
  short4v r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)p);
  return __builtin_bit_cast(half4, r);
}

// matrix-core A operand: k-slots 0..3 from the 4 LDS rows at p, k-slots 4..7 from 16 rows further
__device__ __forceinline__ half8 load_a(const uint8_t* p) {
  const half4 a0 = lds_tr(p), a1 = lds_tr(p + 16 * kPitch);
  return __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Maximum over the four lane groups (lanes l, l^16, l^32, l^48) with the row-swap instructions of
// gfx950: two vector instructions per step, where a shuffle would be a round trip through LDS.
// v_permlane16_swap exchanges rows 1 and 3 of its first operand with rows 0 and 2 of its second.
__device__ __forceinline__ float max_over_lane_groups(float v) {
  const unsigned b = __builtin_bit_cast(unsigned, v);
  const auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  const unsigned r0 = r[0], r1 = r[1];   // as scalars first: a bit_cast of r[1] itself reads element 0
  const float m = vmax(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
  const unsigned c = __builtin_bit_cast(unsigned, m);
  const auto q = __builtin_amdgcn_permlane32_swap(c, c, false, false);
  const unsigned q0 = q[0], q1 = q[1];
  return vmax(__builtin_bit_cast(float, q0), __builtin_bit_cast(float, q1));
}

__device__ __forceinline__ float xor_lanes(float v, int mask) { return __shfl_xor(v, mask); }

// fp16(code) * scale + zero with both roundings, for two codes at a time; `c` holds the codes as
// integers in its two halves.
__device__ __forceinline__ uint32_t dequant_pair(uint32_t c, half2v scale, half2v zero) {
#pragma clang fp contract(off)
  const half2v magic = {(_Float16)1024.f, (_Float16)1024.f};
  half2v f = __builtin_bit_cast(half2v, c | 0x64006400u) - magic;   // exact: 1024 + code - 1024
  half2v m = f * scale;
  half2v r = m + zero;
  return __builtin_bit_cast(uint32_t, r);
}

template <bool BOOST>
struct Prefill {
  const kitty_kv_layer& L;
  const SeqCounts c;
  const int b, h, tid;
  const uint8_t* k_new;
  const uint8_t* v_new;
  int64_t new_stride_t;
  int kv_chunk;      // chunk tokens this workgroup can see
  int n_body;        // body tiles
  int n_tiles;       // sink + body + chunk tiles actually walked
  int first_body, first_chunk;
  mutable int bad_page = 0;   // a page id outside the cache was met (checked_page)
  // Page ids reach tile() through LDS, checked: kIdChunk body tiles at a time, the K and V ids are
  // read by one thread each, range-checked (checked_page) and left as 32-bit numbers in one of two
  // chunk buffers; the chunk after the current one is staged when the walk is half way through the
  // current one, and the barrier that ends every iteration of the walk publishes it.  Reading and
  // checking the ids where they are used - a load whose value the next instructions need, in every
  // iteration of every workgroup - cost this kernel 10 %.
  static constexpr int kIdChunk = 64;
  int32_t (*page_ids)[2][kIdChunk];   // [chunk & 1][K, V][body tile % kIdChunk]

  __device__ __forceinline__ void stage_page_ids(int chunk) const {
    if (tid < 2 * kIdChunk) {
      const int side = tid / kIdChunk, i = chunk * kIdChunk + tid % kIdChunk;
      if (i < (side ? c.pv : c.pk)) {
        const int64_t pg = side ? L.page_table_v[(int64_t)b * L.page_table_v_stride_b + i]
                                : L.page_table_k[(int64_t)b * L.page_table_k_stride_b + i];
        page_ids[chunk & 1][side][tid % kIdChunk] =
            (int32_t)checked_page(pg, side ? L.cache_pages_v : L.cache_pages_k, bad_page);
      }
    }
  }
  // (every lane reads the same word and keeps it in a vector register: made a scalar again with
  // v_readfirstlane, with the tile addresses then computed on the scalar unit, the kernel is 4 % slower)
  __device__ __forceinline__ int64_t staged_page(int side, int i) const {
    return page_ids[(i / kIdChunk) & 1][side][i % kIdChunk];
  }

  __device__ TileSrc tile(int t) const {
    TileSrc s;
    s.chunk_t0 = -1;
    s.k_meta = s.v_meta = nullptr;
    s.v_u0 = 0;
    const int64_t win = (int64_t)b * L.win_stride_b + (int64_t)h * L.win_stride_h;
    if (t < first_body) {   // the sink rows
      const int64_t off = (int64_t)b * L.sink_stride_b + (int64_t)h * L.sink_stride_h;
      s.k_kind = s.v_kind = SRC_ROWS;
      s.k_ptr = (const uint8_t*)L.sink_k + off;
      s.v_ptr = (const uint8_t*)L.sink_v + off;
      s.k_stride = s.v_stride = kD * 2;
      s.ntok = c.sink;
    } else if (t < first_chunk) {
      const int i = t - first_body;
      s.ntok = min(kPage, c.nbody - i * kPage);
      if (i < c.pk) {
        const int64_t pg = staged_page(0, i);
        s.k_kind = SRC_PACKED;
        s.k_ptr = L.key_cache + pg * L.key_cache_stride_page + (int64_t)h * k_head_bytes(L.D_BOOSTED);
        s.k_meta = (const uint8_t*)L.key_meta + pg * L.key_meta_stride_page + (int64_t)h * kD * 4;
      } else {
        s.k_kind = SRC_ROWS;
        s.k_ptr = (const uint8_t*)L.qbuf_k + win;
        s.k_stride = kD * 2;
      }
      if (i < c.pv) {
        const int64_t pg = staged_page(1, i);
        s.v_kind = SRC_PACKED;
        s.v_ptr = L.value_cache + pg * L.value_cache_stride_page + (int64_t)h * kVBytes;
        s.v_meta = (const uint8_t*)L.value_meta + pg * L.value_meta_stride_page + (int64_t)h * kPage * 4;
      } else {
        s.v_kind = SRC_VTAIL;
        s.v_ptr = nullptr;
        s.v_u0 = (i - c.pv) * kPage;
      }
      s.v_stride = 0;
    } else {
      const int t0 = (t - first_chunk) * kPage;
      s.k_kind = s.v_kind = SRC_ROWS;
      s.k_ptr = k_new + (int64_t)t0 * new_stride_t;
      s.v_ptr = v_new + (int64_t)t0 * new_stride_t;
      s.k_stride = s.v_stride = new_stride_t;
      s.ntok = min(kPage, kv_chunk - t0);
      s.chunk_t0 = t0;
    }
    return s;
  }

  // ---- stage 1: global loads of a packed tile into registers ----------------------------------
  __device__ __forceinline__ void issue(const TileSrc& s, Stage& g) const {
    const int e = tid / kParts, part = tid % kParts;   // element (channel or token) and its part of the row
    if (s.k_kind == SRC_PACKED) {
      const uint32_t* lo = (const uint32_t*)(s.k_ptr + e * kRowBytes + part * (4 * kW));
#pragma unroll
      for (int w = 0; w < kW; ++w) g.klo[w] = lo[w];
      g.kmeta = *(const uint32_t*)(s.k_meta + e * 4);
#pragma unroll
      for (int w = 0; w < kW; ++w) g.khi[w] = 0u;
      if (BOOST) {
        const int slot = s.k_ptr[kLoBytes + L.D_BOOSTED * kRowBytes + e];
        if (slot < L.D_BOOSTED) {
          const uint32_t* hi = (const uint32_t*)(s.k_ptr + kLoBytes + slot * kRowBytes + part * (4 * kW));
#pragma unroll
          for (int w = 0; w < kW; ++w) g.khi[w] = hi[w];
        }
      }
    }
    if (s.v_kind == SRC_PACKED) {
      const uint32_t* vv = (const uint32_t*)(s.v_ptr + e * kRowBytes + part * (4 * kW));
#pragma unroll
      for (int w = 0; w < kW; ++w) g.v[w] = vv[w];
      g.vmeta = *(const uint32_t*)(s.v_meta + e * 4);
    }
  }

  // ---- stage 2: registers -> fp16 tile in LDS -----------------------------------------------
  __device__ __forceinline__ void finish(const TileSrc& s, const Stage& g, uint8_t* kt, uint8_t* vt) const {
    const int e = tid / kParts, part = tid % kParts;
    if (s.k_kind == SRC_PACKED) {
      // thread = one channel, 16 kW tokens: plane words of 16 tokens each
      const half2v m2 = __builtin_bit_cast(half2v, g.kmeta);
      const half2v scale = {m2[0], m2[0]}, zero = {m2[1], m2[1]};
      const uint32_t k01 = dequant_pair(0x00010000u, scale, zero), k23 = dequant_pair(0x00030002u, scale, zero);
      uint8_t* row = kt + e * kPitch + part * kPartBytes;
#pragma unroll
      for (int w = 0; w < kW; ++w) {
        uint32_t o[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          uint32_t code = (g.klo[w] >> (2 * u)) & 0x00030003u;
          if (BOOST) {
            code |= ((g.khi[w] >> (2 * u)) & 0x00030003u) << 2;
            o[u] = dequant_pair(code, scale, zero);
          } else {   // four values per channel: the table of the V side below
            o[u] = __builtin_amdgcn_perm(k23, k01, code * 0x0202u + 0x01000100u);
          }
        }
        *(uint4*)(row + w * 32) = uint4{o[0], o[1], o[2], o[3]};
        *(uint4*)(row + w * 32 + 16) = uint4{o[4], o[5], o[6], o[7]};
      }
    } else if (e < s.ntok) {
      // thread = one token, 16 kW channels: transpose into [channel][slot] with 16-bit stores
      uint8_t* col = kt + (part * 16 * kW) * kPitch + slot_of(e) * 2;
      const uint4* src = (const uint4*)(s.k_ptr + (int64_t)e * s.k_stride + part * kPartBytes);
#pragma unroll
      for (int i = 0; i < 2 * kW; ++i) {
        const uint4 x = src[i];
        const uint32_t w4[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          *(uint16_t*)(col + (8 * i + 2 * j) * kPitch) = (uint16_t)(w4[j] & 0xffffu);
          *(uint16_t*)(col + (8 * i + 2 * j + 1) * kPitch) = (uint16_t)(w4[j] >> 16);
        }
      }
    }
    uint8_t* vrow = vt + slot_of(e) * kPitch + part * kPartBytes;
    if (s.v_kind == SRC_PACKED) {
      // thread = one token, 16 kW channels: words of 16 channels each
      // All of a token's codes share one (scale, zero) and take four values: the four dequantized
      // numbers are computed once (same instructions as dequant_pair, so the same two roundings)
      // and every pair of codes picks its two with a byte permute, selector bytes (2c, 2c+1).
      const half2v m2 = __builtin_bit_cast(half2v, g.vmeta);
      const half2v scale = {m2[0], m2[0]}, zero = {m2[1], m2[1]};
      const uint32_t t01 = dequant_pair(0x00010000u, scale, zero), t23 = dequant_pair(0x00030002u, scale, zero);
#pragma unroll
      for (int w = 0; w < kW; ++w) {
        uint32_t o[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const uint32_t codes = (g.v[w] >> (2 * u)) & 0x00030003u;
          o[u] = __builtin_amdgcn_perm(t23, t01, codes * 0x0202u + 0x01000100u);
        }
        *(uint4*)(vrow + w * 32) = uint4{o[0], o[1], o[2], o[3]};
        *(uint4*)(vrow + w * 32 + 16) = uint4{o[4], o[5], o[6], o[7]};
      }
    } else {
      // 16 channels at a time: slot 2u + e' takes channel u + 8e'; dead rows must be finite
      const bool ok = e < s.ntok;
      const uint4* src = nullptr;
      if (ok)
        src = s.v_kind == SRC_VTAIL
                  ? (const uint4*)((const uint8_t*)v_tail_row(L, c, b, h, s.v_u0 + e) + part * kPartBytes)
                  : (const uint4*)(s.v_ptr + (int64_t)e * s.v_stride + part * kPartBytes);
      const uint4 zero4 = uint4{0u, 0u, 0u, 0u};
#pragma unroll
      for (int w = 0; w < kW; ++w) {
        const uint4 a = ok ? src[2 * w] : zero4, bb = ok ? src[2 * w + 1] : zero4;   // channels 0..7, 8..15
        const uint32_t a4[4] = {a.x, a.y, a.z, a.w}, b4[4] = {bb.x, bb.y, bb.z, bb.w};
        uint32_t o[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          o[2 * j] = __builtin_amdgcn_perm(b4[j], a4[j], 0x05040100u);
          o[2 * j + 1] = __builtin_amdgcn_perm(b4[j], a4[j], 0x07060302u);
        }
        *(uint4*)(vrow + w * 32) = uint4{o[0], o[1], o[2], o[3]};
        *(uint4*)(vrow + w * 32 + 16) = uint4{o[4], o[5], o[6], o[7]};
      }
    }
  }
};

// One wavefront's state: 16 kNT query rows (kNT column tiles of 16) against the tiles in LDS.
struct WaveAcc {
  float4v o[8][kNT];    // O^T: [channel-slot tile][row tile]
  float m[kNT], l[kNT];   // running max (log2 units) per row tile column, per-lane partial sums
  bool first;
};

// One 128-token tile in (kt, vt) against this wavefront's rows, in sub-tiles of 32 positions (the
// logits of a sub-tile fit 16 registers).  Software-pipelined: the QK^T MFMAs of sub-tile s+1 are
// issued between the exponentials of sub-tile s, so that a wave's instruction stream mixes matrix
// and vector work instead of alternating long runs of each.
// limit[nt]: tokens of the tile with index < limit are visible to the row of column tile nt.
struct TileAttend {
  const uint8_t* kb;   // K tile + this lane's corner of a transposing read
  const uint8_t* vb;   // V tile + the same corner
  const half8 (&q)[4][kNT];
  WaveAcc& A;
  const float sc2;
  const bool masked;
  const int (&limit)[kNT];
  const int kg;

  __device__ __forceinline__ void qk_issue(int sub, float4v (&S)[2][kNT]) const {
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int nt = 0; nt < kNT; ++nt) S[mt][nt] = float4v{0.f, 0.f, 0.f, 0.f};
    const uint8_t* kbase = kb + sub * 64;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const half8 a = load_a(kbase + (32 * c) * kPitch + mt * 32);
#pragma unroll
        for (int nt = 0; nt < kNT; ++nt) S[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, q[c][nt], S[mt][nt], 0, 0, 0);
      }
  }

  // scale, mask, column maxima, and the (rare, wave-uniform) move of the running maxima
  __device__ __forceinline__ void softmax_head(int sub, float4v (&S)[2][kNT]) const {
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) S[mt][nt] = S[mt][nt] * sc2 - A.m[nt];
    if (masked) {   // one wave-uniform branch: partial tiles and the chunk's own tiles only
#pragma unroll
      for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int tok = 32 * sub + 16 * mt + 2 * kg + (i >> 1) + 8 * (i & 1);
            if (tok >= limit[nt]) S[mt][nt][i] = -INFINITY;
          }
      asm volatile("" ::: "memory");   // keep this a branch, not selects on every tile
    }
    // this lane's maxima; a logit above the running maximum of its row (the logits are relative to
    // it) shows in the lane that holds it, so the maxima over the four lane groups are only formed
    // when some row's maximum really moves
    float mt_[kNT];
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt) {
      float mx = vmax3(vmax3(S[0][nt][0], S[0][nt][1], S[0][nt][2]), S[0][nt][3], S[1][nt][0]);
      mt_[nt] = vmax3(vmax3(mx, S[1][nt][1], S[1][nt][2]), S[1][nt][3], mx);
    }
    bool move = A.first;
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt) move = move || mt_[nt] > 0.f;
    if (__any(move)) {
#pragma unroll
      for (int nt = 0; nt < kNT; ++nt) {
        const float col = max_over_lane_groups(mt_[nt]);
        const float dm = A.first ? col : fmaxf(col, 0.f);
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) S[mt][nt][i] -= dm;
        if (!A.first) {
          const float alpha = __builtin_amdgcn_exp2f(-dm);
          A.l[nt] *= alpha;
#pragma unroll
          for (int ct = 0; ct < 8; ++ct) A.o[ct][nt] *= alpha;
        }
        A.m[nt] += dm;
      }
      A.first = false;
    }
  }

  // exponentials, row sums, fp16 probabilities
  __device__ __forceinline__ void softmax_tail(float4v (&S)[2][kNT], half8 (&p)[kNT]) const {
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt) {
      float sum = 0.f;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float e = __builtin_amdgcn_exp2f(S[mt][nt][i]);
          S[mt][nt][i] = e;
          sum += e;
        }
      A.l[nt] += sum;
      const float4v x0 = S[0][nt], x1 = S[1][nt];
      p[nt] = half8{(_Float16)x0[0], (_Float16)x0[1], (_Float16)x0[2], (_Float16)x0[3],
                    (_Float16)x1[0], (_Float16)x1[1], (_Float16)x1[2], (_Float16)x1[3]};
    }
  }

  __device__ __forceinline__ void pv(int sub, const half8 (&p)[kNT]) const {
    const uint8_t* vbase = vb + (32 * sub) * kPitch;
#pragma unroll
    for (int ct = 0; ct < 8; ++ct) {
      const half8 a = load_a(vbase + ct * 32);
#pragma unroll
      for (int nt = 0; nt < kNT; ++nt) A.o[ct][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, p[nt], A.o[ct][nt], 0, 0, 0);
    }
  }

  __device__ __forceinline__ void run(int nsub) const {
    float4v Sc[2][kNT], Sn[2][kNT];
    half8 p[kNT];
    qk_issue(0, Sc);
#pragma unroll 1
    for (int sub = 0; sub + 1 < nsub; ++sub) {
      softmax_head(sub, Sc);
      // one basic block: 16 operand reads + 16 kNT MFMAs of the next sub-tile between the vector work
      softmax_tail(Sc, p);
      qk_issue(sub + 1, Sn);
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);     // one LDS read
        __builtin_amdgcn_sched_group_barrier(0x008, kNT, 0);   // its MFMAs
        __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);     // a few vector instructions
      }
      __builtin_amdgcn_s_setprio(KITTY_PV_PRIO);
      pv(sub, p);
      __builtin_amdgcn_s_setprio(0);
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < kNT; ++nt) Sc[mt][nt] = Sn[mt][nt];
    }
    softmax_head(nsub - 1, Sc);
    softmax_tail(Sc, p);
    pv(nsub - 1, p);
  }
};

template <bool BOOST>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(kWaves / 4, kWaves / 4))) void prefill_attn_kernel(
    kitty_kv_layer L, const uint8_t* __restrict__ q, int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_t,
    const uint8_t* __restrict__ k_new, const uint8_t* __restrict__ v_new, int64_t new_stride_b,
    int64_t new_stride_h, int64_t new_stride_t, int H_Q, int Tq, float scaling, __half* __restrict__ out) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int32_t s_page_ids[2][2][Prefill<BOOST>::kIdChunk];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, kg = lane >> 4, n = lane & 15;
  const int b = blockIdx.z, h = blockIdx.y;
  const int G = H_Q / L.H_KV;
  const int PB = kRows / G;                              // chunk positions per workgroup
  const int blk = (int)gridDim.x - 1 - (int)blockIdx.x;   // longest causal extent first
  const int p0 = blk * PB;

  const SeqCounts cnt = load_counts(L, b);
  Prefill<BOOST> P{L, cnt, b, h, tid,
                   k_new + (int64_t)b * new_stride_b + (int64_t)h * new_stride_h,
                   v_new + (int64_t)b * new_stride_b + (int64_t)h * new_stride_h,
                   new_stride_t, min(Tq, p0 + PB), 0, 0, 0, 0};
  P.page_ids = s_page_ids;
  P.n_body = c_div_up(cnt.nbody, kPage);
  P.first_body = cnt.sink > 0 ? 1 : 0;
  P.first_chunk = P.first_body + P.n_body;
  P.n_tiles = P.first_chunk + c_div_up(P.kv_chunk, kPage);

  // this lane's query rows: column n of row tile nt is row 16 kNT w + 16 nt + n
  half8 qreg[4][kNT];
  int qpos[kNT];
#pragma unroll
  for (int nt = 0; nt < kNT; ++nt) {
    const int r = 16 * kNT * w + 16 * nt + n;
    const int g = r / PB, pos = p0 + r % PB;
    const bool ok = g < G && pos < Tq;
    qpos[nt] = ok ? pos : -1;
    const uint8_t* row = q + (int64_t)b * q_stride_b + (int64_t)(h * G + (ok ? g : 0)) * q_stride_h +
                         (int64_t)(ok ? pos : 0) * q_stride_t;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      // k-slots 0..3 = channels 32c + 4kg .., k-slots 4..7 = channels 32c + 16 + 4kg ..
      uint2 x0 = *(const uint2*)(row + (32 * c + 4 * kg) * 2);
      uint2 x1 = *(const uint2*)(row + (32 * c + 16 + 4 * kg) * 2);
      if (!ok) x0 = x1 = uint2{0u, 0u};
      const uint4 x = uint4{x0.x, x0.y, x1.x, x1.y};
      qreg[c][nt] = __builtin_bit_cast(half8, x);
    }
  }

  WaveAcc A;
#pragma unroll
  for (int ct = 0; ct < 8; ++ct)
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt) A.o[ct][nt] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int nt = 0; nt < kNT; ++nt) A.m[nt] = 0.f, A.l[nt] = 0.f;
  A.first = true;
  const float sc2 = scaling * kLog2e;

  // Software pipeline over tiles: tile t is multiplied from LDS buffer t & 1 while tile t+1 is
  // turned into fp16 in the other buffer from registers loaded one iteration earlier, and the
  // packed bytes of tile t+2 are on their way.  The waves of a SIMD take the two jobs in opposite
  // order (waves 0..3 convert first, waves 4..7 multiply first), so that one does vector work
  // while the other keeps the matrix pipe busy.  One barrier per tile.
  const int nt_ = P.n_tiles;
  const bool convert_first = w < kWaves / 2;
  Stage ga, gb;                       // tile t+1, tile t+2
  P.stage_page_ids(0);
  __syncthreads();
  TileSrc cur = P.tile(0), nxt = cur, nn = cur;
  P.issue(cur, ga);
  P.finish(cur, ga, lds, lds + 2 * kTile);
  if (nt_ > 1) {
    nxt = P.tile(1);
    P.issue(nxt, ga);
  }
  __syncthreads();
#pragma unroll 1
  for (int t = 0; t < nt_; ++t) {
    const int buf = t & 1;
    const bool more = t + 1 < nt_;
    if (t + 2 < nt_) {
      nn = P.tile(t + 2);
      P.issue(nn, gb);
    }
    {   // half way through a chunk of page ids: stage the next one (tile() is at body tile t + 2 - first_body)
      const int i = t + 2 - P.first_body;
      if (i >= 0 && i % Prefill<BOOST>::kIdChunk == Prefill<BOOST>::kIdChunk / 2) P.stage_page_ids(i / Prefill<BOOST>::kIdChunk + 1);
    }
    uint8_t* kn = lds + (buf ^ 1) * kTile;
    uint8_t* vn = lds + (2 + (buf ^ 1)) * kTile;
    if (more && convert_first) P.finish(nxt, ga, kn, vn);
    int limit[kNT];
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt)
      limit[nt] = cur.chunk_t0 >= 0 ? min(cur.ntok, qpos[nt] - cur.chunk_t0 + 1) : cur.ntok;
    const bool masked = cur.chunk_t0 >= 0 || cur.ntok < kPage;
    {
      // the lane's corner inside a 16-lane transposing read: row n / 4 of 4, columns 4 (n % 4) ..;
      // made opaque so that every read's offset stays a small immediate on these two bases
      uint32_t ok_ = buf * kTile + (4 * kg + (n >> 2)) * kPitch + (n & 3) * 8;
      uint32_t ov_ = ok_ + 2 * kTile;
      asm volatile("" : "+v"(ok_), "+v"(ov_));
      const TileAttend T{lds + ok_, lds + ov_, qreg, A, sc2, masked, limit, kg};
      T.run((cur.ntok + 31) >> 5);
    }
    if (more && !convert_first) P.finish(nxt, ga, kn, vn);
    cur = nxt;
    nxt = nn;
    ga = gb;
    __syncthreads();
  }

  // normalise and store: O^T[ct][nt][i] is channel slot 16 ct + 4 kg + i of row 16 kNT w + 16 nt + n
#pragma unroll
  for (int nt = 0; nt < kNT; ++nt) {
    float l = A.l[nt];
    l += xor_lanes(l, 16);
    l += xor_lanes(l, 32);
    if (qpos[nt] < 0) continue;
    const float inv = 1.f / l;
    const int r = 16 * kNT * w + 16 * nt + n;
    const int g_ = r / PB;
    __half* orow = out + (((int64_t)b * Tq + qpos[nt]) * H_Q + (h * G + g_)) * kD;
#pragma unroll
    for (int ct = 0; ct < 8; ++ct) {
      const float4v o = A.o[ct][nt] * inv;
      // slots 4kg + {0, 2} are channels 2kg, 2kg + 1; slots 4kg + {1, 3} are channels 2kg + 8, 2kg + 9
      *(__half2*)(orow + 16 * ct + 2 * kg) = __floats2half2_rn(o[0], o[2]);
      *(__half2*)(orow + 16 * ct + 2 * kg + 8) = __floats2half2_rn(o[1], o[3]);
    }
  }
  report_bad_page(L, b, P.bad_page);   // by whichever thread met one
}

}  // namespace

int prefill_lds_bytes() { return kLdsBytes; }

void launch_prefill_attn(const kitty_kv_layer& L, const void* q, int64_t q_stride_b, int64_t q_stride_h,
                         int64_t q_stride_t, const void* k_new, const void* v_new, int64_t new_stride_b,
                         int64_t new_stride_h, int64_t new_stride_t, int B, int H_Q, int Tq, float scaling,
                         void* out, hipStream_t stream) {
  const int G = H_Q / L.H_KV;
  const int PB = kRows / G;
  dim3 grid(c_div_up(Tq, PB), L.H_KV, B), block(kThreads);
#define KITTY_LAUNCH_PREFILL(BOOST)                                                                              \
  do {                                                                                                           \
    /* more LDS than the default per-workgroup limit; per device, so set on every launch */                      \
    (void)hipFuncSetAttribute((const void*)prefill_attn_kernel<BOOST>,                                           \
                              hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);                            \
    hipLaunchKernelGGL((prefill_attn_kernel<BOOST>), grid, block, kLdsBytes, stream, L, (const uint8_t*)q,       \
                       q_stride_b, q_stride_h, q_stride_t, (const uint8_t*)k_new, (const uint8_t*)v_new,         \
                       new_stride_b, new_stride_h, new_stride_t, H_Q, Tq, scaling, (__half*)out);                \
  } while (0)
  if (L.D_BOOSTED > 0)
    KITTY_LAUNCH_PREFILL(true);
  else
    KITTY_LAUNCH_PREFILL(false);
#undef KITTY_LAUNCH_PREFILL
}

}  // namespace kitty
