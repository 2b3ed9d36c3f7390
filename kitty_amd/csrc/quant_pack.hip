// Quantize-and-pack kernels for gfx950: one workgroup per (page, kv-head, batch row).
//
// K pages: per-channel asymmetric quantization over the page's 128 tokens, 2 bits per code with
// the boosted channels carrying 2 more bits in a second plane; the boost selection (mean |K| per
// channel, top-d_boost) can run fused in the same pass over the tile.
// V pages: per-token asymmetric 2-bit quantization over the 128 channels.
//
// Arithmetic contract (shared with the reference's Triton kernels, kitty_quant_pack.py:75-82,
// 106-112, 201-204, 227-230): min/max, range, scale = range / qmax (IEEE fp32 divide, floored at
// 1e-6), (x - min) / scale in fp32, floor(. + 0.5), clamp to [0, qmax]; the stored scale is the
// fp32 scale rounded to fp16, the stored zero point is the minimum itself.
#include "kitty_common.h"

using namespace kitty;

namespace {

// fp16 bit pattern of (S * 2^-31) rounded to nearest even, S = sum over 128 tokens of |x| * 2^24,
// i.e. the mean of |x| rounded once.  Positive fp16 patterns order like their values.
__device__ inline uint16_t mean_abs_fp16_bits(uint64_t S) {
  if (S == 0) return 0;
  int msb = 63 - __clzll((long long)S);
  int E = msb - 31;
  if (E >= -14) {
    int shift = msb - 10;
    uint64_t q;
    if (shift > 0) {
      q = S >> shift;
      uint64_t rem = S & ((1ull << shift) - 1), half = 1ull << (shift - 1);
      if (rem > half || (rem == half && (q & 1))) q++;
    } else {
      q = S << (-shift);
    }
    if (q == 2048) { q = 1024; E++; }
    if (E > 15) return 0x7C00;
    return (uint16_t)(((uint32_t)(E + 15) << 10) | (uint32_t)(q & 1023));
  }
  uint64_t q = S >> 7, rem = S & 127;
  if (rem > 64 || (rem == 64 && (q & 1))) q++;
  return (uint16_t)q;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// 16 bytes of the source, which is read exactly once: a non-temporal load (a read-only stream
// reaches 6.5 TB/s with them on this part, 5.9 TB/s without)
__device__ __forceinline__ uint4 nt_load16(const uint8_t* p) {
  const u32x4 v = __builtin_nontemporal_load((const u32x4*)p);
  return uint4{v.x, v.y, v.z, v.w};
}

__device__ inline float h2f(uint16_t bits) { return __half2float(__ushort_as_half(bits)); }

// IEEE fp32 division by a divisor that is shared by a whole group.  This is the correctly rounded
// sequence the compiler emits for `/` (reciprocal, one Newton step, quotient, two residual
// corrections) without its range scaling and special-case fix-up, which cannot trigger here: the
// divisor is a scale in [1e-6, 4.4e4], the dividend x - min is 0 or in [2^-24, 1.4e5].  The
// reciprocal part depends on the divisor only and is computed once per group.  Bit-identical to
// `/` on that domain except that -0 / d gives +0, which the + 0.5 that follows erases.
struct Divisor {
  float d, r;
};
__device__ __forceinline__ Divisor make_divisor(float d) {
  float r = __builtin_amdgcn_rcpf(d);
  const float e = __builtin_fmaf(-d, r, 1.0f);
  r = __builtin_fmaf(e, r, r);
  return {d, r};
}
__device__ __forceinline__ float div_by(float n, Divisor k) {
  float q = n * k.r;
  float rem = __builtin_fmaf(-k.d, q, n);
  q = __builtin_fmaf(rem, k.r, q);
  rem = __builtin_fmaf(-k.d, q, n);
  return __builtin_fmaf(rem, k.r, q);
}
// floor(min(x / scale + 0.5, qmax + 0.5)) as a float: the code.  x >= 0, so the lower clamp of
// the reference never acts, and clamping before the floor gives the same integer.
__device__ __forceinline__ float code_of(float x_minus_min, Divisor k, float qlim) {
  return __builtin_floorf(fminf(div_by(x_minus_min, k) + 0.5f, qlim));
}
// The same codes for N values of one group at a time, mostly without the division:
//   t = fma(x, r, c0),  c0 = fma(-min, r, 0.5),  r = the refined reciprocal of the scale.
// Against the reference's fl(fl((x - min) / scale) + 0.5) this differs by the roundings of x - min,
// of the quotient and of the sum (1e-6 each for quotients below 16.5), the reciprocal's last bit
// (2e-6), the rounding of c0 (1.9e-6 while |min * r| <= 32) and its own (1e-6): under 8e-6.  So
// unless t lies within 2^-16 of an integer, floor(t) is the reference's code; the reference's upper
// clamp never changes a floor for finite inputs (the largest quotient is qmax * (1 + 2^-24)).  If any
// lane of the wave has such a t among its N, or a group whose c0 is NaN (fast_offset returns that
// when |min * r| > 32 or the scale is not finite), the wave redoes these N values with the exact
// division: about one group in seventy on gaussian data.
__device__ __forceinline__ float fast_offset(float mn, Divisor k) {
  const float c0 = __builtin_fmaf(-mn, k.r, 0.5f);
  return (fabsf(mn * k.r) <= 32.0f && k.d < 3.0e38f) ? c0 : __builtin_nanf("");
}
template <int N>
__device__ __forceinline__ void codes_of(const float (&x)[N], float mn, float c0, Divisor k, float qlim, float (&c)[N]) {
  float fmn = 1.0f, fmx = 0.0f;
#pragma unroll
  for (int r = 0; r < N; ++r) {
    const float t = __builtin_fmaf(x[r], k.r, c0);
    c[r] = __builtin_floorf(t);
    const float f = t - c[r];
    fmn = fminf(fmn, f);
    fmx = fmaxf(fmx, f);
  }
  constexpr float kEps = 1.52587890625e-05f;   // 2^-16
  // (min / max skip NaNs, so the group's NaN offset is tested by itself)
  if (__any(!(c0 == c0 && fmn >= kEps && fmx <= 1.0f - kEps))) {
#pragma unroll
    for (int r = 0; r < N; ++r) c[r] = code_of(x[r] - mn, k, qlim);
  }
}
// Bits {1,0} (SHIFT = 0) or {3,2} (SHIFT = 2) of the 8 nibbles of n, packed into 16 bits.
template <int SHIFT>
__device__ __forceinline__ uint32_t gather_fields(uint32_t n) {
  uint32_t x = SHIFT ? (n >> SHIFT) : n;
  x = ((x >> 2) & 0x0C0C0C0Cu) | (x & ~0x0C0C0C0Cu);   // nibble pairs -> low nibble of each byte
  x = ((x >> 4) & 0x00F000F0u) | (x & ~0x00F000F0u);   // byte pairs -> low byte of each half
  x = ((x >> 8) & 0x0000FF00u) | (x & ~0x0000FF00u);   // halves -> low half
  return x & 0xffffu;
}

// One K page of one head.  MODE 0: slot map given.  MODE 1: selection fused, then quantize.
// MODE 2: selection only.  src: the page's first token row of this head; slot_in / slot_out: 128
// bytes (or NULL); dst: the page-head in the cache, meta_dst: its 128 (scale, zero) pairs.
// Called by all 256 threads of a workgroup.
template <int MODE>
__device__ __forceinline__ void quant_k_page(const uint8_t* __restrict__ src_page, int64_t stride_t, int d_boost,
                                             const uint8_t* __restrict__ slot_in, uint8_t* __restrict__ slot_out,
                                             uint8_t* __restrict__ dst, uint8_t* __restrict__ meta_dst) {
  const int tid = threadIdx.x;
  const int tg = tid >> 4;   // tokens tg*8 .. tg*8+7
  const int c8 = tid & 15;   // channels c8*8 .. c8*8+7

  // LDS layouts are chosen so that the 64 lanes of an access fall on 64 different banks.  Per-channel
  // tables are indexed by pos(channel) = (channel % 8) * 16 + channel / 8: the 16 lanes that share a
  // token group work on channels 8 apart and so read / write consecutive entries.  Rows of partials
  // (one per token group) are 144 entries apart, which moves each of the four token groups of a
  // wave to its own quarter (floats) or half (doubles, two passes) of the banks.
  constexpr int kPitch = kD + 16;
  __shared__ __attribute__((aligned(16))) float s_pmin[16][kPitch];   // later: the low plane on its way out
  __shared__ float s_pmax[16][kPitch];
  __shared__ double s_psum[MODE == 0 ? 1 : 16][kPitch];
  __shared__ float4 s_q[kD];   // [pos]: min, scale, refined reciprocal of the scale, qmax + 0.5
  __shared__ float s_c0[kD];   // [pos]: the fast path's offset (fast_offset)
  __shared__ __attribute__((aligned(16))) uint32_t s_key[kD];   // score << 8 | (127 - channel): larger sorts first
  __shared__ __attribute__((aligned(16))) uint8_t s_idx[kD];    // slot by channel, as it is stored
  __shared__ uint8_t s_idx_p[kD];                               // [pos]
  static_assert(sizeof(s_pmin) >= kD * 32, "the low plane reuses the minima");
  uint8_t* const s_lo = (uint8_t*)&s_pmin[0][0];

  const uint8_t* src = src_page + (int64_t)(tg * 8) * stride_t + c8 * 16;
  uint4 rows[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) rows[r] = nt_load16(src + (int64_t)r * stride_t);

  // this thread's 8 tokens x 8 channels as floats, and per channel the partial min / max (/ sum
  // of |x|: exact in fp64, every term is a multiple of 2^-24 below 2^16)
  float xs[8][8];   // [channel j][token r]
#pragma unroll
  for (int j = 0; j < 8; ++j) {
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const uint32_t w = ((const uint32_t*)&rows[r])[j >> 1];
      xs[j][r] = h2f((j & 1) ? (uint16_t)(w >> 16) : (uint16_t)(w & 0xffffu));
    }
    float mn = xs[j][0], mx = xs[j][0];
    double sum = 0.0;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      mn = fminf(mn, xs[j][r]);
      mx = fmaxf(mx, xs[j][r]);
      if (MODE != 0) sum += (double)fabsf(xs[j][r]);
    }
    s_pmin[tg][j * 16 + c8] = mn;
    s_pmax[tg][j * 16 + c8] = mx;
    if (MODE != 0) s_psum[tg][j * 16 + c8] = sum;
  }
  __syncthreads();

  // Second stage on lane pairs: lanes 2c and 2c+1 each fold 8 of channel c's 16 partials, then
  // exchange; with selection they also split the 128 comparisons of the ranking.
  // (the pair's channel follows the table order, so that its reads are consecutive too)
  const int pos = tid >> 1, hf = tid & 1;
  const int ch = (pos & 15) * 8 + (pos >> 4);
  float ch_min = s_pmin[hf][pos], ch_max = s_pmax[hf][pos];
#pragma unroll
  for (int i = 2; i < 16; i += 2) {
    ch_min = fminf(ch_min, s_pmin[i + hf][pos]);
    ch_max = fmaxf(ch_max, s_pmax[i + hf][pos]);
  }
  ch_min = fminf(ch_min, __shfl_xor(ch_min, 1));
  ch_max = fmaxf(ch_max, __shfl_xor(ch_max, 1));
  if (MODE != 0) {
    double sum = 0.0;
#pragma unroll
    for (int i = 0; i < 16; i += 2) sum += s_psum[i + hf][pos];
    sum += __shfl_xor(sum, 1);
    // an integer below 2^47 (or inf / nan for non-finite inputs, which saturate)
    if (hf == 0)
      s_key[ch] = ((uint32_t)mean_abs_fp16_bits(sum < 1.8e19 ? (uint64_t)(sum * 16777216.0) : ~0ull) << 8) |
                  (uint32_t)(kD - 1 - ch);
    __syncthreads();
    // rank = number of channels that sort before this one: higher score, or equal score and
    // lower channel index
    const uint32_t mine = s_key[ch];
    int rank = 0;
#pragma unroll 8
    for (int d = hf * (kD / 2); d < (hf + 1) * (kD / 2); d += 4) {
      const uint4 o = *(const uint4*)&s_key[d];
      rank += (o.x > mine) + (o.y > mine) + (o.z > mine) + (o.w > mine);
    }
    rank += __shfl_xor(rank, 1);
    const uint8_t slot = (uint8_t)(rank < d_boost ? rank : d_boost);
    if (hf == 0) {
      s_idx[ch] = slot;
      s_idx_p[pos] = slot;
      if (slot_out) slot_out[ch] = slot;
    }
    if (MODE == 2) return;
    if (hf == 0) {
      const float qmax = slot < d_boost ? 15.0f : 3.0f;
      float scale = (ch_max - ch_min) / qmax;
      scale = scale < 1e-6f ? 1e-6f : scale;
      const Divisor k = make_divisor(scale);
      s_q[pos] = float4{ch_min, k.d, k.r, qmax + 0.5f};
      s_c0[pos] = fast_offset(ch_min, k);
      *(__half2*)(meta_dst + ch * 4) = __halves2half2(__float2half_rn(scale), __float2half_rn(ch_min));
    }
  } else if (hf == 0) {
    const uint8_t slot = slot_in[ch];
    s_idx[ch] = slot;
    s_idx_p[pos] = slot;
    const float qmax = slot < d_boost ? 15.0f : 3.0f;
    float scale = (ch_max - ch_min) / qmax;
    scale = scale < 1e-6f ? 1e-6f : scale;
    const Divisor k = make_divisor(scale);
    s_q[pos] = float4{ch_min, k.d, k.r, qmax + 0.5f};
    s_c0[pos] = fast_offset(ch_min, k);
    *(__half2*)(meta_dst + ch * 4) = __halves2half2(__float2half_rn(scale), __float2half_rn(ch_min));
  }
  __syncthreads();   // the tables are complete, and nobody reads the partial minima any more (s_lo takes their place)

#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int d = c8 * 8 + j, dp = j * 16 + c8;
    const float4 qp = s_q[dp];
    const Divisor k = {qp.y, qp.z};
    // the 8 codes (0..15) as one word of nibbles, built in floating point (exact: 16 bits per half)
    float c[8];
    codes_of<8>(xs[j], qp.x, s_c0[dp], k, qp.w, c);
    const float h0 = __builtin_fmaf(__builtin_fmaf(__builtin_fmaf(c[3], 16.f, c[2]), 16.f, c[1]), 16.f, c[0]);
    const float h1 = __builtin_fmaf(__builtin_fmaf(__builtin_fmaf(c[7], 16.f, c[6]), 16.f, c[5]), 16.f, c[4]);
    const uint32_t nib = (uint32_t)h0 | ((uint32_t)h1 << 16);
    // plane row d, tokens 8 tg ..: byte d * 32 + 2 tg, with the row's 16-byte pieces and its three
    // row-in-octet bits flipped by c8 so that the 16 rows written at once (8 apart) spread over the banks
    *(uint16_t*)(s_lo + ((d * 32 + tg * 2) ^ (c8 << 4))) = (uint16_t)gather_fields<0>(nib);
    const uint8_t slot = s_idx_p[dp];
    if (slot < d_boost) *(uint16_t*)(dst + kLoBytes + slot * kRowBytes + tg * 2) = (uint16_t)gather_fields<2>(nib);
  }
  __syncthreads();
  ((uint4*)dst)[tid] = *(const uint4*)(s_lo + ((tid * 16) ^ (((tid >> 4) & 15) << 4)));   // piece tid of the plane: row tid / 2, c8 = row / 8
  if (tid < kD / 4) ((uint32_t*)(dst + kRowBytes * (kD + d_boost)))[tid] = ((const uint32_t*)s_idx)[tid];
}

template <int MODE>
__global__ __launch_bounds__(256) void quant_pack_k_kernel(
    const uint8_t* __restrict__ key, int64_t stride_b, int64_t stride_h, int64_t stride_t,
    int t_offset, int d_boost,
    const uint8_t* __restrict__ slot_map_in, uint8_t* __restrict__ slot_map_out, int pages,
    const int64_t* __restrict__ page_table, int64_t pt_stride_b, int page_offset,
    uint8_t* __restrict__ cache, int64_t cache_stride_page,
    uint8_t* __restrict__ meta, int64_t meta_stride_page, int64_t cache_pages) {
  const int p = blockIdx.x, h = blockIdx.y, b = blockIdx.z, H = gridDim.y;
  const uint8_t* src = key + (int64_t)b * stride_b + (int64_t)h * stride_h + (int64_t)(t_offset + p * kPage) * stride_t;
  const int64_t slot_off = (((int64_t)b * H + h) * pages + p) * kD;
  uint8_t* dst = nullptr;
  uint8_t* mdst = nullptr;
  if (MODE != 2) {
    const int64_t pg = page_table[(int64_t)b * pt_stride_b + page_offset + p];
    if (pg < 0 || pg >= cache_pages) return;   // never write outside the cache
    dst = cache + pg * cache_stride_page + (int64_t)h * k_head_bytes(d_boost);
    mdst = meta + pg * meta_stride_page + (int64_t)h * kD * 4;
  }
  quant_k_page<MODE>(src, stride_t, d_boost, slot_map_in ? slot_map_in + slot_off : nullptr,
                     slot_map_out ? slot_map_out + slot_off : nullptr, dst, mdst);
}

// One V page of one head: 256 threads, 8 consecutive lanes share a token (16 channels each), 4
// tokens per thread.  src: the page's first token row of this head.
__device__ __forceinline__ void quant_v_page(const uint8_t* __restrict__ src_page, int64_t stride_t,
                                             uint8_t* __restrict__ dst, uint8_t* __restrict__ mdst) {
  const int tid = threadIdx.x;
  const int cg = tid & 7;
  const uint8_t* src = src_page + cg * 32;
  uint4 la[4], lc[4];   // all eight loads of the thread are in flight before the first is used
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = (tid >> 3) + 32 * i;
    la[i] = nt_load16(src + (int64_t)t * stride_t);
    lc[i] = nt_load16(src + (int64_t)t * stride_t + 16);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = (tid >> 3) + 32 * i;
    const uint4 a = la[i], c = lc[i];
    const uint32_t w[8] = {a.x, a.y, a.z, a.w, c.x, c.y, c.z, c.w};
    float x[16];
    float mn = INFINITY, mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      x[2 * k] = h2f((uint16_t)(w[k] & 0xffffu));
      x[2 * k + 1] = h2f((uint16_t)(w[k] >> 16));
      mn = fminf(mn, fminf(x[2 * k], x[2 * k + 1]));
      mx = fmaxf(mx, fmaxf(x[2 * k], x[2 * k + 1]));
    }
#pragma unroll
    for (int o = 1; o < 8; o <<= 1) {
      mn = fminf(mn, __shfl_xor(mn, o));
      mx = fmaxf(mx, __shfl_xor(mx, o));
    }
    float scale = (mx - mn) / 3.0f;
    scale = scale < 1e-6f ? 1e-6f : scale;
    const Divisor kd = make_divisor(scale);
    float code[16];
    codes_of<16>(x, mn, fast_offset(mn, kd), kd, 3.5f, code);
    // 16 codes (0..3), 2 bits each, built in floating point in two exact 16-bit halves
    float h0 = 0.f, h1 = 0.f;
#pragma unroll
    for (int k = 7; k >= 0; --k) {
      h0 = __builtin_fmaf(h0, 4.f, code[k]);
      h1 = __builtin_fmaf(h1, 4.f, code[8 + k]);
    }
    const uint32_t packed = (uint32_t)h0 | ((uint32_t)h1 << 16);
    __builtin_nontemporal_store(packed, (uint32_t*)(dst + t * kRowBytes + cg * 4));   // written once, read much later
    if (cg == 0) *(__half2*)(mdst + t * 4) = __halves2half2(__float2half_rn(scale), __float2half_rn(mn));
  }
}

__global__ __launch_bounds__(256) void quant_pack_v_kernel(
    const uint8_t* __restrict__ value, int64_t stride_b, int64_t stride_h, int64_t stride_t,
    int t_offset,
    const int64_t* __restrict__ page_table, int64_t pt_stride_b, int page_offset,
    uint8_t* __restrict__ cache, int64_t cache_stride_page,
    uint8_t* __restrict__ meta, int64_t meta_stride_page, int64_t cache_pages) {
  const int p = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int64_t pg = page_table[(int64_t)b * pt_stride_b + page_offset + p];
  if (pg < 0 || pg >= cache_pages) return;
  quant_v_page(value + (int64_t)b * stride_b + (int64_t)h * stride_h + (int64_t)(t_offset + p * kPage) * stride_t,
               stride_t, cache + pg * cache_stride_page + (int64_t)h * kVBytes,
               meta + pg * meta_stride_page + (int64_t)h * kPage * 4);
}

// ---------------------------------------------------------------------------------------------
// Decode-time append and flush with per-sequence counters on the device (int32 [B][8], the
// KITTY_CNT_* fields).  The state machine is KittyCache.update's decode branch (kitty.py:97-123)
// and quantize_decode (kitty.py:194-236), per sequence instead of per batch.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void append_token_kernel(kitty_kv_layer L, const uint8_t* __restrict__ k_new,
                                                           const uint8_t* __restrict__ v_new, int64_t stride_b,
                                                           int64_t stride_h) {
  const int b = blockIdx.x;
  int32_t* cnt = const_cast<int32_t*>(L.seq_counts) + b * KITTY_SEQ_COUNT_FIELDS;
  if (cnt[KITTY_CNT_FLAGS] & KITTY_SEQ_INACTIVE) return;   // the whole block: nobody reaches the barrier
  const int sink = cnt[KITTY_CNT_SINK], rk = cnt[KITTY_CNT_QBUF_K], rv = cnt[KITTY_CNT_QBUF_V];
  const int lv = cnt[KITTY_CNT_LOCAL_V], off = cnt[KITTY_CNT_LOCAL_OFF] & (kPage - 1);
  const bool to_sink = sink < L.S;
  // a full Q-buffer means the caller skipped a flush: drop the token rather than write out of bounds
  const bool ok = to_sink || (rk < kPage && (lv < kPage || rv < kPage));
  __syncthreads();   // every thread has read the counters before thread 0 rewrites them
  if (ok) {
    for (int i = threadIdx.x; i < L.H_KV * 32; i += blockDim.x) {
      const int h = i >> 5, part = (i & 31) * 8;   // 8 bytes = 4 channels
      const uint2 kk = *(const uint2*)(k_new + (int64_t)b * stride_b + (int64_t)h * stride_h + part);
      const uint2 vv = *(const uint2*)(v_new + (int64_t)b * stride_b + (int64_t)h * stride_h + part);
      if (to_sink) {
        const int64_t o = (int64_t)b * L.sink_stride_b + (int64_t)h * L.sink_stride_h + (int64_t)sink * (kD * 2) + part;
        *(uint2*)((uint8_t*)L.sink_k + o) = kk;
        *(uint2*)((uint8_t*)L.sink_v + o) = vv;
      } else {
        const int64_t w = (int64_t)b * L.win_stride_b + (int64_t)h * L.win_stride_h + part;
        *(uint2*)((uint8_t*)L.qbuf_k + w + (int64_t)rk * (kD * 2)) = kk;
        if (lv < kPage) {
          *(uint2*)((uint8_t*)L.local_v + w + (int64_t)lv * (kD * 2)) = vv;
        } else {   // ring full: its oldest row moves to the V Q-buffer, the new one takes the slot
          uint2* slot = (uint2*)((uint8_t*)L.local_v + w + (int64_t)off * (kD * 2));
          *(uint2*)((uint8_t*)L.qbuf_v + w + (int64_t)rv * (kD * 2)) = *slot;
          *slot = vv;
        }
      }
    }
    if (threadIdx.x == 0) {
      if (to_sink) {
        cnt[KITTY_CNT_SINK] = sink + 1;
      } else {
        cnt[KITTY_CNT_QBUF_K] = rk + 1;
        if (lv < kPage) {
          cnt[KITTY_CNT_LOCAL_V] = lv + 1;
        } else {
          cnt[KITTY_CNT_QBUF_V] = rv + 1;
          cnt[KITTY_CNT_LOCAL_OFF] = (off + 1) & (kPage - 1);
        }
      }
    }
  }
}

// blockIdx.z = 0: the K Q-buffer of (b, h) if it is full; 1: the V Q-buffer.
__global__ __launch_bounds__(256) void flush_full_kernel(kitty_kv_layer L, int64_t cache_pages) {
  const int h = blockIdx.x, b = blockIdx.y;
  const int32_t* cnt = L.seq_counts + b * KITTY_SEQ_COUNT_FIELDS;
  const int64_t w = (int64_t)b * L.win_stride_b + (int64_t)h * L.win_stride_h;
  if (cnt[KITTY_CNT_FLAGS] & KITTY_SEQ_INACTIVE) return;
  if (blockIdx.z == 0) {
    const int pk = cnt[KITTY_CNT_PAGES_K];
    if (cnt[KITTY_CNT_QBUF_K] != kPage || pk < 0 || pk >= L.MAX_PAGE) return;
    const int64_t pg = L.page_table_k[(int64_t)b * L.page_table_k_stride_b + pk];
    if (pg < 0 || pg >= cache_pages) return;
    quant_k_page<1>((const uint8_t*)L.qbuf_k + w, kD * 2, L.D_BOOSTED, nullptr, nullptr,
                    const_cast<uint8_t*>(L.key_cache) + pg * L.key_cache_stride_page + (int64_t)h * k_head_bytes(L.D_BOOSTED),
                    (uint8_t*)L.key_meta + pg * L.key_meta_stride_page + (int64_t)h * kD * 4);
  } else {
    const int pv = cnt[KITTY_CNT_PAGES_V];
    if (cnt[KITTY_CNT_QBUF_V] != kPage || pv < 0 || pv >= L.MAX_PAGE) return;
    const int64_t pg = L.page_table_v[(int64_t)b * L.page_table_v_stride_b + pv];
    if (pg < 0 || pg >= cache_pages) return;
    quant_v_page((const uint8_t*)L.qbuf_v + w, kD * 2,
                 const_cast<uint8_t*>(L.value_cache) + pg * L.value_cache_stride_page + (int64_t)h * kVBytes,
                 (uint8_t*)L.value_meta + pg * L.value_meta_stride_page + (int64_t)h * kPage * 4);
  }
}

// after flush_full_kernel: the flushed Q-buffers are empty, their pages count.  The conditions are
// those under which flush_full_kernel wrote the page.
__global__ void advance_counts_kernel(kitty_kv_layer L, int B, int64_t cache_pages) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  int32_t* cnt = const_cast<int32_t*>(L.seq_counts) + b * KITTY_SEQ_COUNT_FIELDS;
  if (cnt[KITTY_CNT_FLAGS] & KITTY_SEQ_INACTIVE) return;
  const int pk = cnt[KITTY_CNT_PAGES_K], pv = cnt[KITTY_CNT_PAGES_V];
  if (cnt[KITTY_CNT_QBUF_K] == kPage && pk >= 0 && pk < L.MAX_PAGE) {
    const int64_t pg = L.page_table_k[(int64_t)b * L.page_table_k_stride_b + pk];
    if (pg >= 0 && pg < cache_pages) {
      cnt[KITTY_CNT_PAGES_K] = pk + 1;
      cnt[KITTY_CNT_QBUF_K] = 0;
    }
  }
  if (cnt[KITTY_CNT_QBUF_V] == kPage && pv >= 0 && pv < L.MAX_PAGE) {
    const int64_t pg = L.page_table_v[(int64_t)b * L.page_table_v_stride_b + pv];
    if (pg >= 0 && pg < cache_pages) {
      cnt[KITTY_CNT_PAGES_V] = pv + 1;
      cnt[KITTY_CNT_QBUF_V] = 0;
    }
  }
}

int check_src(const void* p, int64_t sb, int64_t sh, int64_t st, int B, int H, int T, int D, int t_offset,
              int pages, int page_size) {
  KITTY_REQUIRE(p != nullptr, KITTY_E_NULL, "source tensor is NULL");
  KITTY_REQUIRE(D == kD && page_size == kPage, KITTY_E_SHAPE,
                "kernels are built for head_dim 128 and page_size 128, got D=%d page_size=%d", D, page_size);
  KITTY_REQUIRE(B >= 0 && H >= 1 && pages >= 0 && t_offset >= 0, KITTY_E_RANGE,
                "bad B=%d H=%d pages=%d t_offset=%d", B, H, pages, t_offset);
  KITTY_REQUIRE((int64_t)t_offset + (int64_t)pages * page_size <= (int64_t)T, KITTY_E_RANGE,
                "pages [%d, %d) tokens exceed the source length %d", t_offset, t_offset + pages * page_size, T);
  KITTY_REQUIRE(B <= 65535 && H <= 65535, KITTY_E_RANGE, "B and H must fit a grid dimension");
  KITTY_REQUIRE(((uintptr_t)p % 16) == 0 && sb % 16 == 0 && sh % 16 == 0 && st % 16 == 0 && st >= D * 2,
                KITTY_E_ALIGN, "source needs 16-byte aligned base and strides with D contiguous");
  return 0;
}

int check_dst(const int64_t* page_table, int page_offset, const void* cache, int64_t cache_stride,
              const void* meta, int64_t meta_stride, int64_t cache_pages, int64_t need_cache,
              int64_t need_meta) {
  KITTY_REQUIRE(page_table && cache && meta, KITTY_E_NULL, "page_table / cache / metadata is NULL");
  KITTY_REQUIRE(page_offset >= 0 && cache_pages >= 0, KITTY_E_RANGE, "bad page_offset or cache_pages");
  KITTY_REQUIRE(cache_stride >= need_cache && meta_stride >= need_meta, KITTY_E_RANGE,
                "page stride too small: cache %lld < %lld or metadata %lld < %lld", (long long)cache_stride,
                (long long)need_cache, (long long)meta_stride, (long long)need_meta);
  KITTY_REQUIRE(((uintptr_t)cache % 16) == 0 && cache_stride % 16 == 0 && ((uintptr_t)meta % 4) == 0 &&
                    meta_stride % 4 == 0,
                KITTY_E_ALIGN, "cache needs 16-byte, metadata 4-byte alignment");
  return 0;
}

}  // namespace

extern "C" int kitty_select_boost_k(const void* key, int64_t stride_b, int64_t stride_h, int64_t stride_t,
                                    int B, int H, int T, int D, int t_offset, int pages, int page_size, int d_boost,
                                    uint8_t* slot_map, void* stream) {
  if (int rc = check_src(key, stride_b, stride_h, stride_t, B, H, T, D, t_offset, pages, page_size)) return rc;
  KITTY_REQUIRE(slot_map != nullptr, KITTY_E_NULL, "slot_map is NULL");
  KITTY_REQUIRE(d_boost >= 0 && d_boost <= D, KITTY_E_SHAPE, "d_boost must be in [0, %d], got %d", D, d_boost);
  if (B == 0 || pages == 0) return 0;
  hipLaunchKernelGGL(quant_pack_k_kernel<2>, dim3(pages, H, B), dim3(256), 0, (hipStream_t)stream,
                     (const uint8_t*)key, stride_b, stride_h, stride_t, t_offset, d_boost, nullptr, slot_map,
                     pages, nullptr, 0, 0, nullptr, 0, nullptr, 0, 0);
  return check_launch("kitty_select_boost_k");
}

extern "C" int kitty_quant_pack_k(const void* key, int64_t stride_b, int64_t stride_h, int64_t stride_t,
                                  int B, int H, int T, int D, int t_offset, int pages, int page_size, int d_boost,
                                  const uint8_t* slot_map,
                                  const int64_t* page_table, int64_t page_table_stride_b, int page_offset,
                                  uint8_t* cache, int64_t cache_stride_page,
                                  void* meta, int64_t meta_stride_page, int64_t cache_pages, void* stream) {
  if (int rc = check_src(key, stride_b, stride_h, stride_t, B, H, T, D, t_offset, pages, page_size)) return rc;
  // the slot map is a uint8 with d_boost as the "not boosted" marker, and the high plane has
  // d_boost rows: keep rows 4-byte friendly
  KITTY_REQUIRE(d_boost >= 0 && d_boost <= D, KITTY_E_SHAPE, "d_boost must be in [0, %d], got %d", D, d_boost);
  KITTY_REQUIRE((k_head_bytes(d_boost) % 16) == 0, KITTY_E_ALIGN,
                "d_boost=%d gives a per-head page size that is not a multiple of 16 bytes", d_boost);
  if (int rc = check_dst(page_table, page_offset, cache, cache_stride_page, meta, meta_stride_page, cache_pages,
                         (int64_t)H * k_head_bytes(d_boost), (int64_t)H * kD * 4))
    return rc;
  if (B == 0 || pages == 0) return 0;
  dim3 grid(pages, H, B), block(256);
  if (slot_map)
    hipLaunchKernelGGL(quant_pack_k_kernel<0>, grid, block, 0, (hipStream_t)stream, (const uint8_t*)key, stride_b,
                       stride_h, stride_t, t_offset, d_boost, slot_map, nullptr, pages, page_table,
                       page_table_stride_b, page_offset, cache, cache_stride_page, (uint8_t*)meta,
                       meta_stride_page, cache_pages);
  else
    hipLaunchKernelGGL(quant_pack_k_kernel<1>, grid, block, 0, (hipStream_t)stream, (const uint8_t*)key, stride_b,
                       stride_h, stride_t, t_offset, d_boost, nullptr, nullptr, pages, page_table,
                       page_table_stride_b, page_offset, cache, cache_stride_page, (uint8_t*)meta,
                       meta_stride_page, cache_pages);
  return check_launch("kitty_quant_pack_k");
}

extern "C" int kitty_quant_pack_v(const void* value, int64_t stride_b, int64_t stride_h, int64_t stride_t,
                                  int B, int H, int T, int D, int t_offset, int pages, int page_size,
                                  const int64_t* page_table, int64_t page_table_stride_b, int page_offset,
                                  uint8_t* cache, int64_t cache_stride_page,
                                  void* meta, int64_t meta_stride_page, int64_t cache_pages, void* stream) {
  if (int rc = check_src(value, stride_b, stride_h, stride_t, B, H, T, D, t_offset, pages, page_size)) return rc;
  if (int rc = check_dst(page_table, page_offset, cache, cache_stride_page, meta, meta_stride_page, cache_pages,
                         (int64_t)H * kVBytes, (int64_t)H * kPage * 4))
    return rc;
  if (B == 0 || pages == 0) return 0;
  hipLaunchKernelGGL(quant_pack_v_kernel, dim3(pages, H, B), dim3(256), 0, (hipStream_t)stream,
                     (const uint8_t*)value, stride_b, stride_h, stride_t, t_offset, page_table,
                     page_table_stride_b, page_offset, cache, cache_stride_page, (uint8_t*)meta, meta_stride_page,
                     cache_pages);
  return check_launch("kitty_quant_pack_v");
}

namespace {
int check_append_layer(const kitty_kv_layer* layer, int B) {
  KITTY_REQUIRE(layer != nullptr, KITTY_E_NULL, "layer is NULL");
  const kitty_kv_layer& L = *layer;
  KITTY_REQUIRE(L.seq_counts != nullptr, KITTY_E_NULL, "this entry point needs per-sequence counters (seq_counts)");
  KITTY_REQUIRE(L.D == kD && L.PAGE_SIZE == kPage, KITTY_E_SHAPE,
                "kernels are built for head_dim 128 and page_size 128, got D=%d page_size=%d", L.D, L.PAGE_SIZE);
  KITTY_REQUIRE(L.H_KV >= 1 && L.H_KV <= 65535 && B >= 1 && B <= 65535, KITTY_E_RANGE, "bad H_KV=%d or B=%d", L.H_KV, B);
  KITTY_REQUIRE(L.S >= 0 && L.S <= kPage && L.MAX_PAGE >= 0 && L.D_BOOSTED >= 0 && L.D_BOOSTED <= kD &&
                    k_head_bytes(L.D_BOOSTED) % 16 == 0,
                KITTY_E_SHAPE, "bad S=%d, MAX_PAGE=%d or D_BOOSTED=%d", L.S, L.MAX_PAGE, L.D_BOOSTED);
  KITTY_REQUIRE(L.key_cache && L.key_meta && L.value_cache && L.value_meta && L.page_table_k && L.page_table_v &&
                    L.sink_k && L.sink_v && L.qbuf_k && L.qbuf_v && L.local_v,
                KITTY_E_NULL, "a cache tensor pointer is NULL");
  KITTY_REQUIRE(((uintptr_t)L.key_cache % 16) == 0 && L.key_cache_stride_page % 16 == 0 &&
                    ((uintptr_t)L.value_cache % 16) == 0 && L.value_cache_stride_page % 16 == 0 &&
                    ((uintptr_t)L.key_meta % 4) == 0 && L.key_meta_stride_page % 4 == 0 &&
                    ((uintptr_t)L.value_meta % 4) == 0 && L.value_meta_stride_page % 4 == 0 &&
                    ((uintptr_t)L.sink_k % 16) == 0 && ((uintptr_t)L.sink_v % 16) == 0 &&
                    ((uintptr_t)L.qbuf_k % 16) == 0 && ((uintptr_t)L.qbuf_v % 16) == 0 &&
                    ((uintptr_t)L.local_v % 16) == 0 && L.sink_stride_b % 16 == 0 && L.sink_stride_h % 16 == 0 &&
                    L.win_stride_b % 16 == 0 && L.win_stride_h % 16 == 0 && ((uintptr_t)L.seq_counts % 4) == 0,
                KITTY_E_ALIGN, "cache tensors need 16-byte alignment");
  KITTY_REQUIRE(L.key_cache_stride_page >= (int64_t)L.H_KV * k_head_bytes(L.D_BOOSTED) &&
                    L.value_cache_stride_page >= (int64_t)L.H_KV * kVBytes &&
                    L.key_meta_stride_page >= (int64_t)L.H_KV * kD * 4 &&
                    L.value_meta_stride_page >= (int64_t)L.H_KV * kPage * 4,
                KITTY_E_RANGE, "a page stride is smaller than one page");
  return 0;
}
}  // namespace

extern "C" int kitty_append_token(const kitty_kv_layer* layer, const void* k_new, const void* v_new,
                                  int64_t stride_b, int64_t stride_h, int B, void* stream) {
  if (int rc = check_append_layer(layer, B)) return rc;
  KITTY_REQUIRE(k_new && v_new, KITTY_E_NULL, "k_new / v_new is NULL");
  KITTY_REQUIRE(((uintptr_t)k_new % 8) == 0 && ((uintptr_t)v_new % 8) == 0 && stride_b % 8 == 0 && stride_h % 8 == 0,
                KITTY_E_ALIGN, "k_new / v_new need 8-byte aligned bases and strides");
  hipLaunchKernelGGL(append_token_kernel, dim3(B), dim3(256), 0, (hipStream_t)stream, *layer, (const uint8_t*)k_new,
                     (const uint8_t*)v_new, stride_b, stride_h);
  return check_launch("kitty_append_token");
}

extern "C" int kitty_flush_full(const kitty_kv_layer* layer, int B, int64_t cache_pages, void* stream) {
  if (int rc = check_append_layer(layer, B)) return rc;
  KITTY_REQUIRE(cache_pages >= 0, KITTY_E_RANGE, "bad cache_pages");
  hipLaunchKernelGGL(flush_full_kernel, dim3(layer->H_KV, B, 2), dim3(256), 0, (hipStream_t)stream, *layer, cache_pages);
  hipLaunchKernelGGL(advance_counts_kernel, dim3((B + 63) / 64), dim3(64), 0, (hipStream_t)stream, *layer, B,
                     cache_pages);
  return check_launch("kitty_flush_full");
}
