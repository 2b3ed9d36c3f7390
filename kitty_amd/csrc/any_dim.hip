// The quantized-KV path for head dimensions other than 128 (64 and 256).
//
// The reference takes the head dimension from the model's config and promotes a quarter of the key
// channels (kitty.py:39-44); its kernels take D as a parameter (kitty_quant_pack.py:42-45, 180-181;
// kitty_attention.py:59-62, 253-254).  The tuned kernels of this library are written for D = 128, the
// size of every model the reference names.  The kernels here cover the other sizes with the same
// arithmetic and the same storage format - plain vector-ALU code, one template parameter for D:
//
//   quant_k_any_kernel / quant_v_any_kernel   quantize-and-pack, boost selection fused or given
//   attn_any_kernel<D, false, ROWS>           decode attention, split pass (the reference's order of
//                                             operations: fp16 dequantization with both roundings)
//   attn_any_kernel<D, true, 16>              chunked-prefill attention, one pass
//   merge_any_kernel                          the merge pass of split-K
//
// Wire format for general D (PAGE = 128 tokens): a K page-head is 32 D bytes of low plane (channel d at
// 32 d), 32 d_boost bytes of high plane (slot s at 32 (D + s)) and D bytes of slot map; a V page-head is
// 128 rows of D / 4 bytes; metadata as for D = 128 with D resp. 128 (scale, zero) pairs per head.
#include "decode_common.h"
#include "quant_arith.h"

namespace kitty {
namespace {

constexpr int kMaxRows = 16;   // query rows per workgroup at most: the group's heads (decode), heads x positions (prefill)

// ---------------------------------------------------------------------------------------------
// quantize and pack
// ---------------------------------------------------------------------------------------------
// One K page of one head: thread d owns channel d and walks the page's 128 tokens twice (the second
// pass finds the rows in the cache).  MODE 0: slot map given.  1: selection fused.  2: selection only.
template <int D, int MODE>
__global__ __launch_bounds__(256) void quant_k_any_kernel(
    const uint8_t* __restrict__ key, int64_t stride_b, int64_t stride_h, int64_t stride_t, int t_offset, int d_boost,
    const uint8_t* __restrict__ slot_map_in, uint8_t* __restrict__ slot_map_out, int pages,
    const int64_t* __restrict__ page_table, int64_t pt_stride_b, int page_offset, uint8_t* __restrict__ cache,
    int64_t cache_stride_page, uint8_t* __restrict__ meta, int64_t meta_stride_page, int64_t cache_pages,
    int32_t* __restrict__ status) {
  static_assert(D <= 256, "one thread per channel");
  const int p = blockIdx.x, h = blockIdx.y, b = blockIdx.z, H = gridDim.y;
  const uint8_t* src = key + (int64_t)b * stride_b + (int64_t)h * stride_h + (int64_t)(t_offset + p * kPage) * stride_t;
  const int64_t slot_off = (((int64_t)b * H + h) * pages + p) * D;
  uint8_t* dst = nullptr;
  uint8_t* mdst = nullptr;
  if (MODE != 2) {
    const int64_t pg = page_table[(int64_t)b * pt_stride_b + page_offset + p];
    if (pg < 0 || pg >= cache_pages) {   // never write outside the cache; leave a record instead
      if (status && threadIdx.x == 0) status[b * KITTY_STATUS_FIELDS + KITTY_STATUS_BAD_PAGE_WRITE] = 1;
      return;
    }
    dst = cache + pg * cache_stride_page + (int64_t)h * k_head_bytes_d(D, d_boost);
    mdst = meta + pg * meta_stride_page + (int64_t)h * D * 4;
  }
  __shared__ uint32_t s_key[D];   // score << 8 | (D - 1 - channel): larger sorts first
  const int d = threadIdx.x;
  const bool on = d < D;
  float mn = INFINITY, mx = -INFINITY;
  unsigned long long sum = 0;     // exact: every |x| * 2^24 is an integer below 2^40
  bool saturated = false;
  if (on) {
    for (int t = 0; t < kPage; ++t) {
      const float x = h2f(*(const uint16_t*)(src + (int64_t)t * stride_t + 2 * d));
      mn = fminf(mn, x);
      mx = fmaxf(mx, x);
      if (MODE != 0) {
        const float v = fabsf(x) * 0x1p24f;
        if (v < 0x1p41f) sum += (unsigned long long)v;
        else saturated = true;      // inf or NaN among the inputs
      }
    }
  }
  uint32_t slot;
  if (MODE != 0) {
    // score = mean |x| rounded once to fp16; rank = number of channels that sort before this one
    // (higher score first, then lower channel index)
    if (on) s_key[d] = ((uint32_t)(saturated ? 0x7C00 : mean_abs_fp16_bits(sum)) << 8) | (uint32_t)(D - 1 - d);
    __syncthreads();
    int rank = 0;
    if (on) {
      const uint32_t mine = s_key[d];
      for (int e = 0; e < D; ++e) rank += s_key[e] > mine;
    }
    slot = (uint32_t)(rank < d_boost ? rank : d_boost);
    if (on && slot_map_out) slot_map_out[slot_off + d] = (uint8_t)slot;
    if (MODE == 2) return;
  } else {
    slot = on ? slot_map_in[slot_off + d] : 0u;
  }
  if (!on) return;
  const float qmax = slot < (uint32_t)d_boost ? 15.0f : 3.0f;
  float scale = (mx - mn) / qmax;
  scale = scale < 1e-6f ? 1e-6f : scale;
  const Divisor k = make_divisor(scale);
  *(__half2*)(mdst + d * 4) = __halves2half2(__float2half_rn(scale), __float2half_rn(mn));
  uint32_t lo[8], hi[8];
#pragma unroll
  for (int w = 0; w < 8; ++w) {
    lo[w] = hi[w] = 0u;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float x = h2f(*(const uint16_t*)(src + (int64_t)(16 * w + i) * stride_t + 2 * d));
      const uint32_t c = (uint32_t)code_of(x - mn, k, qmax + 0.5f);
      lo[w] |= (c & 3u) << (2 * i);
      hi[w] |= (c >> 2) << (2 * i);
    }
  }
  uint4* lo_row = (uint4*)(dst + d * kRowBytes);
  lo_row[0] = uint4{lo[0], lo[1], lo[2], lo[3]};
  lo_row[1] = uint4{lo[4], lo[5], lo[6], lo[7]};
  if (slot < (uint32_t)d_boost) {
    uint4* hi_row = (uint4*)(dst + (D + slot) * kRowBytes);
    hi_row[0] = uint4{hi[0], hi[1], hi[2], hi[3]};
    hi_row[1] = uint4{hi[4], hi[5], hi[6], hi[7]};
  }
  dst[kRowBytes * (D + d_boost) + d] = (uint8_t)slot;
}

// One V page of one head: thread t owns token t and walks its D channels twice.
template <int D>
__global__ __launch_bounds__(128) void quant_v_any_kernel(
    const uint8_t* __restrict__ value, int64_t stride_b, int64_t stride_h, int64_t stride_t, int t_offset,
    const int64_t* __restrict__ page_table, int64_t pt_stride_b, int page_offset, uint8_t* __restrict__ cache,
    int64_t cache_stride_page, uint8_t* __restrict__ meta, int64_t meta_stride_page, int64_t cache_pages,
    int32_t* __restrict__ status) {
  const int p = blockIdx.x, h = blockIdx.y, b = blockIdx.z, t = threadIdx.x;
  const int64_t pg = page_table[(int64_t)b * pt_stride_b + page_offset + p];
  if (pg < 0 || pg >= cache_pages) {
    if (status && t == 0) status[b * KITTY_STATUS_FIELDS + KITTY_STATUS_BAD_PAGE_WRITE] = 1;
    return;
  }
  const uint8_t* row = value + (int64_t)b * stride_b + (int64_t)h * stride_h + (int64_t)(t_offset + p * kPage + t) * stride_t;
  uint8_t* dst = cache + pg * cache_stride_page + (int64_t)h * v_head_bytes_d(D) + t * (D / 4);
  uint8_t* mdst = meta + pg * meta_stride_page + ((int64_t)h * kPage + t) * 4;
  float mn = INFINITY, mx = -INFINITY;
  for (int c = 0; c < D / 8; ++c) {
    const uint4 w = ((const uint4*)row)[c];
    const uint32_t w4[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = h2f((uint16_t)(w4[i] & 0xffffu)), bb = h2f((uint16_t)(w4[i] >> 16));
      mn = fminf(mn, fminf(a, bb));
      mx = fmaxf(mx, fmaxf(a, bb));
    }
  }
  float scale = (mx - mn) / 3.0f;
  scale = scale < 1e-6f ? 1e-6f : scale;
  const Divisor k = make_divisor(scale);
  for (int c = 0; c < D / 16; ++c) {   // 16 channels per word of codes: channel e in bits 2 (e % 16)
    uint32_t packed = 0u;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint4 w = ((const uint4*)row)[2 * c + j];
      const uint32_t w4[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t c0 = (uint32_t)code_of(h2f((uint16_t)(w4[i] & 0xffffu)) - mn, k, 3.5f);
        const uint32_t c1 = (uint32_t)code_of(h2f((uint16_t)(w4[i] >> 16)) - mn, k, 3.5f);
        packed |= (c0 | (c1 << 2)) << (4 * (4 * j + i));
      }
    }
    ((uint32_t*)dst)[c] = packed;
  }
  *(__half2*)mdst = __halves2half2(__float2half_rn(scale), __float2half_rn(mn));
}

// ---------------------------------------------------------------------------------------------
// attention
// ---------------------------------------------------------------------------------------------
// fp16(code) * scale + zero with BOTH operations rounded to fp16 (kitty_attention.py:162-165, 317-320 as
// eager torch and the Triton interpreter evaluate them).
__device__ inline float dequant_two(uint32_t code, __half scale, __half zero) {
#pragma clang fp contract(off)
  const _Float16 s = static_cast<__half_raw>(scale).data;
  const _Float16 z = static_cast<__half_raw>(zero).data;
  const _Float16 c = (_Float16)(float)code;
  const _Float16 prod = c * s;
  const _Float16 r = prod + z;
  return (float)r;
}

// Up to 16 query rows of one (batch row, kv head) against a range of 128-token tiles.
// Decode (PREFILL false): grid (splits, H_KV, B); the rows are the G heads of the group; the partial
// (running max in log2 units, running sum, un-normalised output) goes to the split-K workspace.
// Prefill: grid (blocks of 16 / G chunk positions, H_KV, B); row r is head r / PB at chunk position
// p0 + r % PB; after the layer's own tiles come the chunk's rows, causally; the normalised output
// goes to out [B, T_q, H_Q, D].
// Logits: thread = (token, half of the channels).  Output: thread = (channel, 1 / (256 / D) of the tile's
// tokens).  Logits and probabilities stay fp32.
template <int D, bool PREFILL, int ROWS>
__global__ __launch_bounds__(256) void attn_any_kernel(
    kitty_kv_layer L, const uint8_t* __restrict__ q, int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_t,
    const uint8_t* __restrict__ k_new, const uint8_t* __restrict__ v_new, int64_t new_stride_b,
    int64_t new_stride_h, int64_t new_stride_t, int H_Q, int Tq, float scaling, float* __restrict__ ws_ml,
    float* __restrict__ ws_acc, int num_splits, __half* __restrict__ out) {
  constexpr int kParts = 256 / D;   // token parts of the output phase
  constexpr int kPartTok = kPage / kParts;
  static_assert(D == 64 || D == 128 || D == 256, "head dimensions with a whole number of token parts");
  const int h = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int G = H_Q / L.H_KV;
  const int DB = L.D_BOOSTED;
  const SeqCounts c = load_counts(L, b);
  const int PB = PREFILL ? max(1, ROWS / G) : 1;
  const int R = PREFILL ? G * PB : G;
  const int p0 = PREFILL ? (int)blockIdx.x * PB : 0;
  const int kv_chunk = PREFILL ? min(Tq, p0 + PB) : 0;           // chunk tokens this workgroup can see
  const int n_tiles = c.ntiles + (kv_chunk + kPage - 1) / kPage;
  int tile_begin = 0, tile_end = n_tiles;
  if (!PREFILL) {
    const int per = (c.ntiles + num_splits - 1) / num_splits;
    tile_begin = (int)blockIdx.x * per;
    tile_end = min(c.ntiles, tile_begin + per);
  }
  int bad_page = 0;

  __shared__ __attribute__((aligned(16))) float s_q[D][ROWS];        // [channel][row]: a thread reads the rows of a channel at once
  __shared__ __attribute__((aligned(16))) uint8_t s_codes[kRowBytes * 2 * D + D];   // a K page-head with d_boost up to D
  __shared__ __half2 s_meta[D > kPage ? D : kPage];
  __shared__ __attribute__((aligned(16))) float s_p[kPage][ROWS];    // [token][row]
  __shared__ union {
    float part[2][ROWS][kPage];        // logits: [half of the channels][row][token]
    float o[kParts][ROWS][D];          // the output's partial sums at the end
  } s_u;
  __shared__ float s_m[ROWS], s_l[ROWS], s_alpha[ROWS];
  __shared__ int s_pos[ROWS];          // prefill: chunk position of a row, -1 = no such row

  if (tid < ROWS) {
    s_m[tid] = -INFINITY;
    s_l[tid] = 0.f;
    int pos = 0;
    if (PREFILL) pos = (tid < R && p0 + tid % PB < Tq) ? p0 + tid % PB : -1;
    s_pos[tid] = pos;
  }
  for (int i = tid; i < R * D; i += 256) {
    const int r = i / D, d = i % D;
    const int g = PREFILL ? r / PB : r, pos = PREFILL ? min(p0 + r % PB, Tq - 1) : 0;
    const uint8_t* row = q + (int64_t)b * q_stride_b + (int64_t)(h * G + g) * q_stride_h + (int64_t)pos * q_stride_t;
    s_q[d][r] = __half2float(((const __half*)row)[d]);
  }
  float acc_o[ROWS];
#pragma unroll
  for (int g = 0; g < ROWS; ++g) acc_o[g] = 0.f;
  __syncthreads();

  const int t = tid & 127, half = tid >> 7;
  const int od = tid % D, opart = tid / D;
  const int64_t sink_base = (int64_t)b * L.sink_stride_b + (int64_t)h * L.sink_stride_h;
  const int64_t win_base = (int64_t)b * L.win_stride_b + (int64_t)h * L.win_stride_h;
  const uint8_t* kc = PREFILL ? k_new + (int64_t)b * new_stride_b + (int64_t)h * new_stride_h : nullptr;
  const uint8_t* vc = PREFILL ? v_new + (int64_t)b * new_stride_b + (int64_t)h * new_stride_h : nullptr;

  for (int tile = tile_begin; tile < tile_end; ++tile) {
    const bool chunk = tile >= c.ntiles;                       // a tile of the new chunk (prefill only)
    const int chunk_t0 = chunk ? (tile - c.ntiles) * kPage : 0;
    const int body = tile - 1;                                  // -1 = sink
    const int ntok = chunk ? min(kPage, kv_chunk - chunk_t0) : tile == 0 ? c.sink : min(kPage, c.nbody - body * kPage);
    const bool k_packed = !chunk && tile > 0 && body < c.pk;
    const bool v_packed = !chunk && tile > 0 && body < c.pv;

    // ---- logits -----------------------------------------------------------------------------
    float acc[ROWS];
#pragma unroll
    for (int g = 0; g < ROWS; ++g) acc[g] = 0.f;
    if (k_packed) {
      const int64_t pg = checked_page(page_id(L.page_table_k, (int64_t)b * L.page_table_k_stride_b + body), L.cache_pages_k, bad_page);
      const uint8_t* src = L.key_cache + pg * L.key_cache_stride_page + (int64_t)h * k_head_bytes_d(D, DB);
      for (int i = tid; i < k_head_bytes_d(D, DB) / 16; i += 256) ((uint4*)s_codes)[i] = ((const uint4*)src)[i];
      if (tid < D)
        s_meta[tid] = *(const __half2*)((const uint8_t*)L.key_meta + pg * L.key_meta_stride_page +
                                        ((int64_t)h * D + tid) * 4);
      __syncthreads();
      const int sh = 2 * (t & 3);
      const uint8_t* idx = s_codes + kRowBytes * (D + DB);
      for (int d = half * (D / 2); d < (half + 1) * (D / 2); ++d) {
        uint32_t code = (s_codes[d * kRowBytes + (t >> 2)] >> sh) & 3u;
        const uint32_t slot = idx[d];
        if (slot < (uint32_t)DB) code |= ((s_codes[(D + slot) * kRowBytes + (t >> 2)] >> sh) & 3u) << 2;
        const __half2 m = s_meta[d];
        const float x = dequant_two(code, __low2half(m), __high2half(m));
#pragma unroll
        for (int g = 0; g < ROWS; ++g)
          if (g < R) acc[g] += s_q[d][g] * x;
      }
    } else if (t < ntok) {
      const __half* row = chunk      ? (const __half*)(kc + (int64_t)(chunk_t0 + t) * new_stride_t)
                          : tile == 0 ? (const __half*)((const uint8_t*)L.sink_k + sink_base) + (int64_t)t * D
                                      : (const __half*)((const uint8_t*)L.qbuf_k + win_base) + (int64_t)t * D;
      for (int d = half * (D / 2); d < (half + 1) * (D / 2); ++d) {
        const float x = __half2float(row[d]);
#pragma unroll
        for (int g = 0; g < ROWS; ++g)
          if (g < R) acc[g] += s_q[d][g] * x;
      }
    }
#pragma unroll
    for (int g = 0; g < ROWS; ++g)
      if (g < R) s_u.part[half][g][t] = acc[g];
    __syncthreads();

    // ---- online softmax: one wave per query row ------------------------------------------------
    for (int g = wave; g < R; g += 4) {
      // tokens of the tile this row sees: all of them, or (the chunk's own tiles) those up to its position
      int lim = ntok;
      if (PREFILL) lim = s_pos[g] < 0 ? 0 : chunk ? min(ntok, s_pos[g] - chunk_t0 + 1) : ntok;
      float v0 = -INFINITY, v1 = -INFINITY;
      if (lane < lim) v0 = (s_u.part[0][g][lane] + s_u.part[1][g][lane]) * scaling;
      if (lane + 64 < lim) v1 = (s_u.part[0][g][lane + 64] + s_u.part[1][g][lane + 64]) * scaling;
      float mxv = fmaxf(v0, v1);
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) mxv = fmaxf(mxv, __shfl_xor(mxv, o));
      const float m_old = s_m[g];
      const float m_new = fmaxf(m_old, mxv);
      const float p0v = (v0 == -INFINITY) ? 0.f : __expf(v0 - m_new);
      const float p1v = (v1 == -INFINITY) ? 0.f : __expf(v1 - m_new);
      float sum = p0v + p1v;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
      const float alpha = (m_old == -INFINITY) ? 0.f : __expf(m_old - m_new);
      s_p[lane][g] = p0v;
      s_p[lane + 64][g] = p1v;
      if (lane == 0) { s_m[g] = m_new; s_l[g] = s_l[g] * alpha + sum; s_alpha[g] = alpha; }
    }
    // ---- stage V ---------------------------------------------------------------------------
    if (v_packed) {
      const int64_t pg = checked_page(page_id(L.page_table_v, (int64_t)b * L.page_table_v_stride_b + body), L.cache_pages_v, bad_page);
      const uint8_t* src = L.value_cache + pg * L.value_cache_stride_page + (int64_t)h * v_head_bytes_d(D);
      for (int i = tid; i < v_head_bytes_d(D) / 16; i += 256) ((uint4*)s_codes)[i] = ((const uint4*)src)[i];
      if (tid < kPage)
        s_meta[tid] = *(const __half2*)((const uint8_t*)L.value_meta + pg * L.value_meta_stride_page +
                                        ((int64_t)h * kPage + tid) * 4);
    }
    __syncthreads();

    // ---- out += P V : thread = (channel, part of the tile's tokens) ---------------------------
    {
#pragma unroll
      for (int g = 0; g < ROWS; ++g)
        if (g < R) acc_o[g] *= s_alpha[g];
      const int t0 = opart * kPartTok, t1 = min(ntok, (opart + 1) * kPartTok);
      for (int tt = t0; tt < t1; ++tt) {
        float x;
        if (v_packed) {
          const uint32_t code = (s_codes[tt * (D / 4) + (od >> 2)] >> (2 * (od & 3))) & 3u;
          const __half2 m = s_meta[tt];
          x = dequant_two(code, __low2half(m), __high2half(m));
        } else if (chunk) {
          x = __half2float(((const __half*)(vc + (int64_t)(chunk_t0 + tt) * new_stride_t))[od]);
        } else if (tile == 0) {
          x = __half2float(((const __half*)((const uint8_t*)L.sink_v + sink_base))[(int64_t)tt * D + od]);
        } else {
          x = __half2float(v_tail_row(L, c, b, h, (body - c.pv) * kPage + tt, D)[od]);
        }
#pragma unroll
        for (int g = 0; g < ROWS; ++g)
          if (g < R) acc_o[g] += s_p[tt][g] * x;   // (a masked token has probability 0)
      }
    }
    __syncthreads();
  }

  if (tid == 0) report_bad_page(L, b, bad_page);
#pragma unroll
  for (int g = 0; g < ROWS; ++g)
    if (g < R) s_u.o[opart][g][od] = acc_o[g];
  __syncthreads();
  for (int i = tid; i < R * D; i += 256) {
    const int g = i / D, d = i % D;
    float o = 0.f;
#pragma unroll
    for (int pp = 0; pp < kParts; ++pp) o += s_u.o[pp][g][d];
    if (PREFILL) {
      const int pos = s_pos[g];
      if (pos >= 0) {
        const float l = s_l[g];
        out[(((int64_t)b * Tq + pos) * H_Q + (h * G + g / PB)) * D + d] = __float2half_rn(l > 0.f ? o / l : 0.f);
      }
    } else {
      const int64_t row = ((int64_t)b * H_Q + (int64_t)h * G + g) * num_splits + blockIdx.x;
      ws_acc[row * D + d] = o;
      if (d == 0) { ws_ml[row * 2] = s_m[g] * 1.44269504088896f; ws_ml[row * 2 + 1] = s_l[g]; }
    }
  }
}

// out[b, 0, hq, :] = sum_s acc_s * 2^(m_s - m) / sum_s l_s * 2^(m_s - m); one block per query head, one
// thread per channel.
template <int D>
__global__ __launch_bounds__(D) void merge_any_kernel(const float* __restrict__ ws_ml, const float* __restrict__ ws_acc,
                                                       __half* __restrict__ out, int num_splits) {
  const int64_t head = (int64_t)blockIdx.y * gridDim.x + blockIdx.x;
  const int64_t row0 = head * num_splits;
  const int d = threadIdx.x;
  float m = -INFINITY;
  for (int s = 0; s < num_splits; ++s) m = fmaxf(m, ws_ml[(row0 + s) * 2]);
  float l = 0.f, o = 0.f;
  for (int s = 0; s < num_splits; ++s) {
    const float ms = ws_ml[(row0 + s) * 2];
    if (ms == -INFINITY) continue;   // an empty split
    const float w = exp2f(ms - m);
    l += ws_ml[(row0 + s) * 2 + 1] * w;
    o += ws_acc[(row0 + s) * D + d] * w;
  }
  out[head * D + d] = __float2half_rn(l > 0.f ? o / l : 0.f);
}

template <int D>
void quant_k_any(int mode, const void* key, int64_t sb, int64_t sh, int64_t st, int B, int H, int t_offset, int pages,
                 int d_boost, const uint8_t* slot_in, uint8_t* slot_out, const int64_t* page_table, int64_t pt_stride,
                 int page_offset, uint8_t* cache, int64_t cache_stride, void* meta, int64_t meta_stride,
                 int64_t cache_pages, int32_t* status, hipStream_t stream) {
  const dim3 grid(pages, H, B), block(256);
#define KITTY_QK_ANY(MODE)                                                                                        \
  hipLaunchKernelGGL((quant_k_any_kernel<D, MODE>), grid, block, 0, stream, (const uint8_t*)key, sb, sh, st,        \
                     t_offset, d_boost, slot_in, slot_out, pages, page_table, pt_stride, page_offset, cache,        \
                     cache_stride, (uint8_t*)meta, meta_stride, cache_pages, status)
  if (mode == 0) KITTY_QK_ANY(0);
  else if (mode == 1) KITTY_QK_ANY(1);
  else KITTY_QK_ANY(2);
#undef KITTY_QK_ANY
}

}  // namespace

// mode 0: slot map given; 1: selection fused into the quantizer; 2: selection only (slot_out).
void launch_quant_k_any(int D, int mode, const void* key, int64_t sb, int64_t sh, int64_t st, int B, int H,
                        int t_offset, int pages, int d_boost, const uint8_t* slot_in, uint8_t* slot_out,
                        const int64_t* page_table, int64_t pt_stride, int page_offset, uint8_t* cache,
                        int64_t cache_stride, void* meta, int64_t meta_stride, int64_t cache_pages, int32_t* status,
                        hipStream_t stream) {
  if (D == 64)
    quant_k_any<64>(mode, key, sb, sh, st, B, H, t_offset, pages, d_boost, slot_in, slot_out, page_table, pt_stride,
                    page_offset, cache, cache_stride, meta, meta_stride, cache_pages, status, stream);
  else
    quant_k_any<256>(mode, key, sb, sh, st, B, H, t_offset, pages, d_boost, slot_in, slot_out, page_table, pt_stride,
                     page_offset, cache, cache_stride, meta, meta_stride, cache_pages, status, stream);
}

void launch_quant_v_any(int D, const void* value, int64_t sb, int64_t sh, int64_t st, int B, int H, int t_offset,
                        int pages, const int64_t* page_table, int64_t pt_stride, int page_offset, uint8_t* cache,
                        int64_t cache_stride, void* meta, int64_t meta_stride, int64_t cache_pages, int32_t* status,
                        hipStream_t stream) {
  const dim3 grid(pages, H, B), block(128);
  if (D == 64)
    hipLaunchKernelGGL((quant_v_any_kernel<64>), grid, block, 0, stream, (const uint8_t*)value, sb, sh, st, t_offset,
                       page_table, pt_stride, page_offset, cache, cache_stride, (uint8_t*)meta, meta_stride,
                       cache_pages, status);
  else
    hipLaunchKernelGGL((quant_v_any_kernel<256>), grid, block, 0, stream, (const uint8_t*)value, sb, sh, st, t_offset,
                       page_table, pt_stride, page_offset, cache, cache_stride, (uint8_t*)meta, meta_stride,
                       cache_pages, status);
}

void launch_decode_any(const kitty_kv_layer& L, const void* q, int B, int H_Q, float scaling, float* ws_ml,
                       float* ws_acc, int num_splits, hipStream_t stream) {
  const dim3 grid(num_splits, L.H_KV, B), block(256);
  const int64_t qb = (int64_t)H_Q * L.D * 2, qh = (int64_t)L.D * 2;
  const int G = H_Q / L.H_KV;
  // the kernel is instantiated for 4, 8 and 16 query rows: a group of 4 heads does not pay for 16
#define KITTY_ATTN_ANY(DD, RR)                                                                                       \
  hipLaunchKernelGGL((attn_any_kernel<DD, false, RR>), grid, block, 0, stream, L, (const uint8_t*)q, qb, qh,         \
                     (int64_t)0, nullptr, nullptr, (int64_t)0, (int64_t)0, (int64_t)0, H_Q, 1, scaling, ws_ml,       \
                     ws_acc, num_splits, nullptr)
  if (L.D == 64) {
    if (G <= 4) KITTY_ATTN_ANY(64, 4);
    else if (G <= 8) KITTY_ATTN_ANY(64, 8);
    else KITTY_ATTN_ANY(64, 16);
  } else {
    if (G <= 4) KITTY_ATTN_ANY(256, 4);
    else if (G <= 8) KITTY_ATTN_ANY(256, 8);
    else KITTY_ATTN_ANY(256, 16);
  }
#undef KITTY_ATTN_ANY
}

void launch_merge_any(int D, const float* ws_ml, const float* ws_acc, void* out, int B, int H_Q, int num_splits,
                      hipStream_t stream) {
  const dim3 grid(H_Q, B);
  if (D == 64)
    hipLaunchKernelGGL((merge_any_kernel<64>), grid, dim3(64), 0, stream, ws_ml, ws_acc, (__half*)out, num_splits);
  else
    hipLaunchKernelGGL((merge_any_kernel<256>), grid, dim3(256), 0, stream, ws_ml, ws_acc, (__half*)out, num_splits);
}

void launch_prefill_any(const kitty_kv_layer& L, const void* q, int64_t q_stride_b, int64_t q_stride_h,
                        int64_t q_stride_t, const void* k_new, const void* v_new, int64_t new_stride_b,
                        int64_t new_stride_h, int64_t new_stride_t, int B, int H_Q, int Tq, float scaling, void* out,
                        hipStream_t stream) {
  const int G = H_Q / L.H_KV;
  const int PB = kMaxRows / G > 0 ? kMaxRows / G : 1;
  const dim3 grid((Tq + PB - 1) / PB, L.H_KV, B), block(256);
  if (L.D == 64)
    hipLaunchKernelGGL((attn_any_kernel<64, true, kMaxRows>), grid, block, 0, stream, L, (const uint8_t*)q, q_stride_b,
                       q_stride_h, q_stride_t, (const uint8_t*)k_new, (const uint8_t*)v_new, new_stride_b,
                       new_stride_h, new_stride_t, H_Q, Tq, scaling, nullptr, nullptr, 1, (__half*)out);
  else
    hipLaunchKernelGGL((attn_any_kernel<256, true, kMaxRows>), grid, block, 0, stream, L, (const uint8_t*)q, q_stride_b,
                       q_stride_h, q_stride_t, (const uint8_t*)k_new, (const uint8_t*)v_new, new_stride_b,
                       new_stride_h, new_stride_t, H_Q, Tq, scaling, nullptr, nullptr, 1, (__half*)out);
}

}  // namespace kitty
