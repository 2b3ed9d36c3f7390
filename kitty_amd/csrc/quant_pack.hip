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
#include "half_ops.h"
#include "quant_arith.h"

namespace kitty {
// head dimensions other than 128 (any_dim.hip)
void launch_quant_k_any(int D, int mode, const void* key, int64_t sb, int64_t sh, int64_t st, int B, int H,
                        int t_offset, int pages, int d_boost, const uint8_t* slot_in, uint8_t* slot_out,
                        const int64_t* page_table, int64_t pt_stride, int page_offset, uint8_t* cache,
                        int64_t cache_stride, void* meta, int64_t meta_stride, int64_t cache_pages, int32_t* status,
                        hipStream_t stream);
void launch_quant_v_any(int D, const void* value, int64_t sb, int64_t sh, int64_t st, int B, int H, int t_offset,
                        int pages, const int64_t* page_table, int64_t pt_stride, int page_offset, uint8_t* cache,
                        int64_t cache_stride, void* meta, int64_t meta_stride, int64_t cache_pages, int32_t* status,
                        hipStream_t stream);
}  // namespace kitty

using namespace kitty;

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// 16 bytes of the source, which is read exactly once: a non-temporal load (a read-only stream
// reaches 6.5 TB/s with them on this part, 5.9 TB/s without)
__device__ __forceinline__ uint4 nt_load16(const uint8_t* p) {
  const u32x4 v = __builtin_nontemporal_load((const u32x4*)p);
  return uint4{v.x, v.y, v.z, v.w};
}

__device__ __forceinline__ void nt_store16(uint8_t* p, const uint4& v) {
  __builtin_nontemporal_store(u32x4{v.x, v.y, v.z, v.w}, (u32x4*)p);
}

// The codes of the 8 values of one group (half `hi` of the words w[0..7]) as bytes of two words,
// mostly without the division.  The reference floors T = fl(fl(fl(x - min) / scale) + 0.5).  Here
//   a = fma(x, r, cA),  b = fma(x, r, cB),  cA = fma(-min, r, -2^-16),  cB = fma(-min, r, +2^-16),
// r = the refined reciprocal of the scale.  Against T - 0.5 -+ 2^-16 these differ by the reference's
// roundings of x - min, of the quotient and of the sum (1e-6 each for quotients below 16.5), the
// reciprocal's last bit (2e-6), the rounding of cA / cB (1.9e-6 while |min * r| <= 32) and their own
// (1e-6): under 8e-6, so a < T - 0.5 < b.  v_cvt_pk_u8_f32 rounds to the nearest integer (ties to even)
// and saturates at 0 and 255.  If it gives the same integer n for a and for b, then n - 0.5 <= a and
// b <= n + 0.5, hence n < T < n + 1: n is the reference's code (its upper clamp never changes a floor
// for finite inputs: the largest quotient is qmax * (1 + 2^-24)).  If the two differ for any of a
// lane's 8 values in any lane of the wave, or the group's offsets are NaN (fast_offsets returns that
// when |min * r| > 32 or the scale is not finite), the wave redoes these 8 values with the exact
// division: about one group in seventy on gaussian data.
__device__ __forceinline__ float2 fast_offsets(float mn, Divisor k) {
  constexpr float kEps = 1.52587890625e-05f;   // 2^-16
  const float nan = __builtin_nanf("");
  const bool ok = fabsf(mn * k.r) <= 32.0f && k.d < 3.0e38f;
  return ok ? float2{__builtin_fmaf(-mn, k.r, -kEps), __builtin_fmaf(-mn, k.r, kEps)} : float2{nan, nan};
}
__device__ __forceinline__ void codes_of(const uint32_t (&w)[8], int hi, float mn, float2 cab, Divisor k, float qlim,
                                         uint32_t& c0123, uint32_t& c4567) {
  uint32_t a[2] = {0, 0}, b[2] = {0, 0};
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const float x = (float)half_of(w[r], hi);
    a[r >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(x, k.r, cab.x), r & 3, a[r >> 2]);
    b[r >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(x, k.r, cab.y), r & 3, b[r >> 2]);
  }
  if (__any(!(cab.x == cab.x) || a[0] != b[0] || a[1] != b[1])) {
    a[0] = a[1] = 0;
#pragma unroll
    for (int r = 0; r < 8; ++r)
      a[r >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(code_of((float)half_of(w[r], hi) - mn, k, qlim), r & 3, a[r >> 2]);
  }
  c0123 = a[0];
  c4567 = a[1];
}
// Bits {1,0} (SHIFT = 0) or {3,2} (SHIFT = 2) of the 8 code bytes of (c0123, c4567), packed into 16
// bits: a dot product of the four masked bytes with (1, 4, 16, 64) lines their fields up.
template <int SHIFT>
__device__ __forceinline__ uint32_t gather_fields(uint32_t c0123, uint32_t c4567) {
  constexpr uint32_t kMask = 0x03030303u << SHIFT, kWeights = 0x40100401u;
  const uint32_t lo = __builtin_amdgcn_udot4(c0123 & kMask, kWeights, 0u, false);
  const uint32_t hi = __builtin_amdgcn_udot4(c4567 & kMask, kWeights, 0u, false);
  return ((hi << 8) + lo) >> SHIFT;
}

// One K page of one head.  MODE 0: slot map given.  MODE 1: selection fused, then quantize.
// MODE 2: selection only.  row_of(t): the 256-byte row of token t (0..127) of this head; slot_in /
// slot_out: 128 bytes (or NULL); dst: the page-head in the cache, meta_dst: its 128 (scale, zero)
// pairs.  Called by all 256 threads of a workgroup.
struct StridedRows {   // the rows of a page that lies in one tensor
  const uint8_t* base;
  int64_t stride_t;
  __device__ __forceinline__ const uint8_t* operator()(int t) const { return base + (int64_t)t * stride_t; }
  // row t0 + r, r a constant: the product with the lane's t0 is formed once for all r
  __device__ __forceinline__ const uint8_t* operator()(int t0, int r) const {
    return base + (int64_t)t0 * stride_t + (int64_t)r * stride_t;
  }
};
template <int MODE, class ROWS>
__device__ __forceinline__ void quant_k_page(const ROWS row_of, int d_boost,
                                             const uint8_t* __restrict__ slot_in, uint8_t* __restrict__ slot_out,
                                             uint8_t* __restrict__ dst, uint8_t* __restrict__ meta_dst) {
  const int tid = threadIdx.x;
  const int tg = tid >> 4;   // tokens tg*8 .. tg*8+7
  const int c8 = tid & 15;   // channels c8*8 .. c8*8+7

  // LDS layouts are chosen so that the 64 lanes of an access fall on 64 different banks.  Per-channel
  // tables are indexed by pos(channel) = (channel % 8) * 16 + channel / 8: the 16 lanes that share a
  // token group work on channels 8 apart and so read / write consecutive entries.  Rows of partials
  // are 80 words (minima / maxima: one per token group, a word of two fp16 channels) or 144 floats
  // (sums: one per pair of token groups) apart, which moves each of the four token groups of a wave to
  // its own quarter of the banks.  All of it stays under 20 KB, so that eight workgroups share a CU:
  // the kernel needs that many to keep the vector units busy across its five barriers.
  constexpr int kPitchW = kD / 2 + 16, kPitch = kD + 16;
  __shared__ __attribute__((aligned(16))) uint32_t s_pmin[16][kPitchW];   // later: the low plane on its way out
  __shared__ __attribute__((aligned(16))) uint32_t s_pmax[16][kPitchW];   // later: the high plane on its way out
  __shared__ float s_psum[MODE == 0 ? 1 : 8][kPitch];
  // [pos]: min, scale, refined reciprocal of the scale, qmax + 0.5; before the ranking its first half
  // holds s_exact, [pos]: the exact sum of |x| * 2^24 where fp32 leaves a doubt
  __shared__ float4 s_q[kD];
  unsigned long long* const s_exact = (unsigned long long*)s_q;
  __shared__ uint8_t s_doubt[MODE == 0 ? 1 : kD];              // [pos]
  __shared__ int s_any_doubt;
  __shared__ float2 s_cab[kD];   // [pos]: the fast path's two offsets (fast_offsets)
  // score << 8 | (127 - channel): larger sorts first; after the ranking s_meta, the (scale, zero) pairs by
  // channel, as they are stored
  __shared__ __attribute__((aligned(16))) uint32_t s_key[kD];
  uint32_t* const s_meta = s_key;
  __shared__ __attribute__((aligned(16))) uint8_t s_idx[kD];    // slot by channel, as it is stored
  __shared__ uint8_t s_idx_p[kD];                               // [pos]
  // A given slot map need not use every slot; the high-plane rows of unused slots keep their old bytes
  // (the fused selection fills slots 0 .. d_boost - 1, all of them).
  __shared__ __attribute__((aligned(4))) uint8_t s_slot_used[MODE == 0 ? 256 : 4];
  static_assert(sizeof(s_pmin) >= kD * 32 && sizeof(s_pmax) >= kD * 32, "the planes reuse the minima and maxima");
  uint8_t* const s_lo = (uint8_t*)&s_pmin[0][0];
  uint8_t* const s_hi = (uint8_t*)&s_pmax[0][0];   // 32 bytes per slot

  // this thread's 8 tokens x 8 channels: word q of row r holds channels 2q and 2q + 1 of token r
  uint32_t w[4][8];
  {
    uint4 rows[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) rows[r] = nt_load16(row_of(tg * 8, r) + c8 * 16);
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      w[0][r] = rows[r].x;
      w[1][r] = rows[r].y;
      w[2][r] = rows[r].z;
      w[3][r] = rows[r].w;
    }
  }

  // per channel the partial min / max (packed fp16, exact) and the partial sum of |x| in fp32 (good
  // enough to rank nearly every channel, see below)
  if (MODE != 0 && tid == 0) s_any_doubt = 0;
  if (MODE == 0 && tid < 64) ((uint32_t*)s_slot_used)[tid] = 0;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    uint32_t mn = w[q][0], mx = w[q][0];
#pragma unroll
    for (int r = 1; r < 8; ++r) {
      mn = pk_min_f16(mn, w[q][r]);
      mx = pk_max_f16(mx, w[q][r]);
    }
    s_pmin[tg][q * 16 + c8] = mn;
    s_pmax[tg][q * 16 + c8] = mx;
    if (MODE != 0) {
#pragma unroll
      for (int hi = 0; hi < 2; ++hi) {
        // added as a tree: every term goes through three additions here and a fourth with the
        // neighbouring token group's sum (lane l ^ 16), whose even member keeps the result
        const float own = ((abs_sum_f16(w[q][0], w[q][1], hi) + abs_sum_f16(w[q][2], w[q][3], hi)) +
                           (abs_sum_f16(w[q][4], w[q][5], hi) + abs_sum_f16(w[q][6], w[q][7], hi)));
        const unsigned bits = __builtin_bit_cast(unsigned, own);
        const auto both = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
        const unsigned b0 = both[0], b1 = both[1];   // as scalars first: a bit_cast of both[1] itself reads element 0
        if ((tg & 1) == 0)
          s_psum[tg >> 1][(2 * q + hi) * 16 + c8] = __builtin_bit_cast(float, b0) + __builtin_bit_cast(float, b1);
      }
    }
  }
  __syncthreads();

  // Second stage on lane pairs: lanes 2c and 2c+1 each fold 8 of channel c's 16 partials, then
  // exchange; with selection they also split the 128 comparisons of the ranking.
  // (the pair's channel follows the table order, so that its reads are consecutive too)
  const int pos = tid >> 1, hf = tid & 1;
  const int ch = (pos & 15) * 8 + (pos >> 4);
  float ch_min, ch_max;
  {
    const int word = (pos >> 5) * 16 + (pos & 15);   // the word that holds this channel, in half (pos >> 4) & 1
    uint32_t mn = s_pmin[hf][word], mx = s_pmax[hf][word];
#pragma unroll
    for (int i = 2; i < 16; i += 2) {
      mn = pk_min_f16(mn, s_pmin[i + hf][word]);
      mx = pk_max_f16(mx, s_pmax[i + hf][word]);
    }
    mn = pk_min_f16(mn, (uint32_t)__shfl_xor((int)mn, 1));
    mx = pk_max_f16(mx, (uint32_t)__shfl_xor((int)mx, 1));
    const int sh = (pos & 16);   // 16 for the upper half
    ch_min = widen_f16(mn >> sh, 0);
    ch_max = widen_f16(mx >> sh, 0);
  }
  if (MODE != 0) {
    // The score is the mean of |x| over the page, rounded ONCE to fp16.  In the fp32 sum of the 128
    // non-negative terms every term went through 7 additions (3 in its thread, 1 with the next token
    // group, 2 in this fold, 1 between the lanes), each with a relative error of at most 2^-24, so the exact mean lies within
    // 7.01 * 2^-24 (relative) of sum / 128.  The ends of the interval tested are that mean times
    // 1 -+ 10 * 2^-24 (both factors are fp32 numbers; the products round once more).  If both ends
    // round to the same fp16 number, that is the score; otherwise (one channel in about 600: the
    // interval contains a midpoint between two fp16 numbers; one page-head in five has such a
    // channel), or when the mean is so small that fp16 has no normal number for it, the channel's
    // 16 threads add their terms exactly - every |x| is a multiple of 2^-24 below 2^16 - into a
    // 64-bit integer.
    float sum = (s_psum[hf][pos] + s_psum[2 + hf][pos]) + (s_psum[4 + hf][pos] + s_psum[6 + hf][pos]);
    sum += __shfl_xor(sum, 1);
    if (hf == 0) {
      uint32_t score = 0;
      bool doubt = false;
      if (!(sum < 3.0e38f)) {
        score = 0x7C00;   // inf or NaN among the inputs: saturates
      } else if (sum != 0.f) {
        const float mean = sum * (1.0f / kPage);
        const uint16_t lo = __half_as_ushort(__float2half_rn(mean * (1.0f - 0x1.4p-21f)));
        const uint16_t hi = __half_as_ushort(__float2half_rn(mean * (1.0f + 0x1.4p-21f)));
        doubt = lo != hi || mean < 0x1p-13f;
        score = lo;
      }
      s_doubt[pos] = doubt;
      if (doubt) {
        s_exact[pos] = 0;
        s_any_doubt = 1;
      } else {
        s_key[ch] = (score << 8) | (uint32_t)(kD - 1 - ch);
      }
    }
    __syncthreads();
    if (s_any_doubt) {   // the same for every thread of the workgroup
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (s_doubt[j * 16 + c8]) {
          // |x| * 2^24 is an integer below 2^40: its bits from 2^20 up and the rest, added apart
          uint32_t up = 0, low = 0;
#pragma unroll
          for (int r = 0; r < 8; ++r) {
            const float v = (float)__builtin_fabsf16(half_of(w[j >> 1][r], j & 1)) * 0x1p24f;
            const float u = floorf(v * 0x1p-20f);
            up += (uint32_t)u;
            low += (uint32_t)__builtin_fmaf(u, -0x1p20f, v);
          }
          atomicAdd(&s_exact[j * 16 + c8], ((unsigned long long)up << 20) + low);
        }
      }
      __syncthreads();
      if (hf == 0 && s_doubt[pos])
        s_key[ch] = ((uint32_t)mean_abs_fp16_bits(s_exact[pos]) << 8) | (uint32_t)(kD - 1 - ch);
      __syncthreads();
    }
    // rank = number of channels that sort before this one: higher score, or equal score and lower
    // channel index.  Each wave ranks 32 channels: a lane holds two of the 128 keys, a channel's key is
    // read into every lane, and the lanes whose keys are larger are counted - one compare per 64 pairs
    // of keys, the counting on the scalar unit.
    {
      const int lane = tid & 63, first = (tid >> 6) * (kD / 4);
      const uint32_t k0 = s_key[lane], k1 = s_key[lane + 64];
#pragma unroll
      for (int i = 0; i < kD / 16; ++i) {
        const uint4 t = *(const uint4*)&s_key[first + 4 * i];
        const uint32_t key[4] = {t.x, t.y, t.z, t.w};
        uint32_t slots = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int rank = __popcll(__ballot(k0 > key[e])) + __popcll(__ballot(k1 > key[e]));
          slots |= (uint32_t)(rank < d_boost ? rank : d_boost) << (8 * e);
        }
        ((uint32_t*)s_idx)[(first >> 2) + i] = slots;   // the same word from every lane
      }
    }
    __syncthreads();
    const uint8_t slot = s_idx[ch];
    if (hf == 0) {
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
      s_cab[pos] = fast_offsets(ch_min, k);
      s_meta[ch] = __builtin_bit_cast(uint32_t, __halves2half2(__float2half_rn(scale), __float2half_rn(ch_min)));
    }
  } else if (hf == 0) {
    const uint8_t slot = slot_in[ch];
    s_idx[ch] = slot;
    s_idx_p[pos] = slot;
    if (slot < d_boost) s_slot_used[slot] = 1;
    const float qmax = slot < d_boost ? 15.0f : 3.0f;
    float scale = (ch_max - ch_min) / qmax;
    scale = scale < 1e-6f ? 1e-6f : scale;
    const Divisor k = make_divisor(scale);
    s_q[pos] = float4{ch_min, k.d, k.r, qmax + 0.5f};
    s_cab[pos] = fast_offsets(ch_min, k);
    s_meta[ch] = __builtin_bit_cast(uint32_t, __halves2half2(__float2half_rn(scale), __float2half_rn(ch_min)));
  }
  __syncthreads();   // the tables are complete, and nobody reads the partial minima and maxima any more (s_lo, s_hi take their place)

#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int d = c8 * 8 + j, dp = j * 16 + c8;
    const float4 qp = s_q[dp];
    const Divisor k = {qp.y, qp.z};
    uint32_t c0123, c4567;   // the 8 codes (0..15), a byte each
    codes_of(w[j >> 1], j & 1, qp.x, s_cab[dp], k, qp.w, c0123, c4567);
    // plane row d, tokens 8 tg ..: byte d * 32 + 2 tg, with the row's 16-byte pieces and its three
    // row-in-octet bits flipped by c8 so that the 16 rows written at once (8 apart) spread over the banks
    *(uint16_t*)(s_lo + ((d * 32 + tg * 2) ^ (c8 << 4))) = (uint16_t)gather_fields<0>(c0123, c4567);
    const uint8_t slot = s_idx_p[dp];
    if (slot < d_boost) *(uint16_t*)(s_hi + slot * kRowBytes + tg * 2) = (uint16_t)gather_fields<2>(c0123, c4567);
  }
  __syncthreads();
  // everything leaves in contiguous pieces: the low plane by all threads (16 bytes each), the high plane by the
  // first lanes (16 bytes each), the slot map by the second wave and the (scale, zero) pairs by the last two
  // (4 bytes each: the metadata's alignment is only that)
  // the planes are written once and read much later: non-temporal stores
  nt_store16(dst + tid * 16, *(const uint4*)(s_lo + ((tid * 16) ^ (((tid >> 4) & 15) << 4))));   // piece tid of the plane: row tid / 2, c8 = row / 8
  if (tid < 2 * d_boost && (MODE != 0 || s_slot_used[tid >> 1])) nt_store16(dst + kLoBytes + tid * 16, ((const uint4*)s_hi)[tid]);
  const int t1 = tid - 64, t2 = tid - 128;
  if (t1 >= 0 && t1 < kD / 4) ((uint32_t*)(dst + kRowBytes * (kD + d_boost)))[t1] = ((const uint32_t*)s_idx)[t1];
  if (t2 >= 0) ((uint32_t*)meta_dst)[t2] = s_meta[t2];
}

template <int MODE>
__global__ __launch_bounds__(256) void quant_pack_k_kernel(
    const uint8_t* __restrict__ key, int64_t stride_b, int64_t stride_h, int64_t stride_t,
    int t_offset, int d_boost,
    const uint8_t* __restrict__ slot_map_in, uint8_t* __restrict__ slot_map_out, int pages,
    const int64_t* __restrict__ page_table, int64_t pt_stride_b, int page_offset,
    uint8_t* __restrict__ cache, int64_t cache_stride_page,
    uint8_t* __restrict__ meta, int64_t meta_stride_page, int64_t cache_pages, int32_t* __restrict__ status) {
  const int p = blockIdx.x, h = blockIdx.y, b = blockIdx.z, H = gridDim.y;
  const uint8_t* src = key + (int64_t)b * stride_b + (int64_t)h * stride_h + (int64_t)(t_offset + p * kPage) * stride_t;
  const int64_t slot_off = (((int64_t)b * H + h) * pages + p) * kD;
  uint8_t* dst = nullptr;
  uint8_t* mdst = nullptr;
  if (MODE != 2) {
    const int64_t pg = page_table[(int64_t)b * pt_stride_b + page_offset + p];
    if (pg < 0 || pg >= cache_pages) {   // never write outside the cache; leave a record instead
      if (status && threadIdx.x == 0) status[b * KITTY_STATUS_FIELDS + KITTY_STATUS_BAD_PAGE_WRITE] = 1;
      return;
    }
    dst = cache + pg * cache_stride_page + (int64_t)h * k_head_bytes(d_boost);
    mdst = meta + pg * meta_stride_page + (int64_t)h * kD * 4;
  }
  quant_k_page<MODE>(StridedRows{src, stride_t}, d_boost, slot_map_in ? slot_map_in + slot_off : nullptr,
                     slot_map_out ? slot_map_out + slot_off : nullptr, dst, mdst);
}

// The 16 codes (0..3) of one lane's 16 channels of a token - both halves of w[0..7], in the order low
// half of w[0], high half of w[0], low half of w[1] .. - as bytes of four words: the two roundings of codes_of above, the exact division
// where they disagree.
__device__ __forceinline__ void codes_of_row(const uint32_t (&w)[8], float mn, float2 cab, Divisor k, uint32_t (&c)[4]) {
  uint32_t b[4] = {0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < 4; ++i) c[i] = 0;
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const float x = (float)half_of(w[e >> 1], e & 1);
    c[e >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(x, k.r, cab.x), e & 3, c[e >> 2]);
    b[e >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(x, k.r, cab.y), e & 3, b[e >> 2]);
  }
  if (__any(!(cab.x == cab.x) || c[0] != b[0] || c[1] != b[1] || c[2] != b[2] || c[3] != b[3])) {
#pragma unroll
    for (int i = 0; i < 4; ++i) c[i] = 0;
#pragma unroll
    for (int e = 0; e < 16; ++e)
      c[e >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(code_of((float)half_of(w[e >> 1], e & 1) - mn, k, 3.5f), e & 3, c[e >> 2]);
  }
}

// One V page of one head: 256 threads, 8 consecutive lanes share a token, 4 tokens per thread.  A lane
// holds channels 8 cg .. 8 cg + 7 and 64 + 8 cg .. 64 + 8 cg + 7 of its tokens: each load instruction
// then reads whole 128-byte half rows, 16 bytes per lane.  row_of(t): the 256-byte row of token t of this head.
template <class ROWS>
__device__ __forceinline__ void quant_v_page(const ROWS row_of, uint8_t* __restrict__ dst, uint8_t* __restrict__ mdst) {
  const int tid = threadIdx.x;
  const int cg = tid & 7;
  uint4 la[4], lc[4];   // all eight loads of the thread are in flight before the first is used
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint8_t* src = row_of((tid >> 3) + 32 * i) + cg * 16;
    la[i] = nt_load16(src);
    lc[i] = nt_load16(src + kD);
  }
  // The lane's codes make bytes 2 cg, 2 cg + 1 and 16 + 2 cg, 17 + 2 cg of the token's 32-byte row.  Lanes
  // 2 m and 2 m + 1 swap one of the two pairs, so that the even lane has bytes 4 m .. 4 m + 3 and the odd
  // lane bytes 16 + 4 m .. 19 + 4 m: one 4-byte store per lane.
  const bool odd = cg & 1;
  const uint32_t pick = odd ? 0x03020706u : 0x05040100u;   // odd: (partner's upper pair, own upper pair); even: (own lower, partner's lower)
  const int out_off = odd ? 14 + 2 * cg : 2 * cg;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = (tid >> 3) + 32 * i;
    const uint4 a = la[i], c = lc[i];
    const uint32_t w[8] = {a.x, a.y, a.z, a.w, c.x, c.y, c.z, c.w};
    // The token's minimum and maximum in packed fp16 (exact): over the lane's 8 words, then with the
    // maximum negated beside the minimum in one word, so that one packed minimum per step serves both,
    // over the word's own halves and over the 8 lanes that share the token.
    uint32_t mnw = w[0], mxw = w[0];
#pragma unroll
    for (int k = 1; k < 8; ++k) {
      mnw = pk_min_f16(mnw, w[k]);
      mxw = pk_max_f16(mxw, w[k]);
    }
    const uint32_t nmx = mxw ^ 0x80008000u;
    uint32_t m = pk_min_f16(__builtin_amdgcn_perm(nmx, mnw, 0x05040100u),    // (mnw.lo, nmx.lo)
                            __builtin_amdgcn_perm(nmx, mnw, 0x07060302u));   // (mnw.hi, nmx.hi)
    // lanes l ^ 1, l ^ 2, then 7 - l of the group of 8 (whose quads agree by then): data-parallel moves,
    // no trip through the LDS crossbar
    m = pk_min_f16(m, (uint32_t)__builtin_amdgcn_mov_dpp((int)m, 0xB1 /* quad_perm [1,0,3,2] */, 0xf, 0xf, true));
    m = pk_min_f16(m, (uint32_t)__builtin_amdgcn_mov_dpp((int)m, 0x4E /* quad_perm [2,3,0,1] */, 0xf, 0xf, true));
    m = pk_min_f16(m, (uint32_t)__builtin_amdgcn_mov_dpp((int)m, 0x141 /* row_half_mirror */, 0xf, 0xf, true));
    const float mn = widen_f16(m, 0), mx = -widen_f16(m, 1);
    float scale = (mx - mn) / 3.0f;
    scale = scale < 1e-6f ? 1e-6f : scale;
    const Divisor kd = make_divisor(scale);
    uint32_t code[4];
    codes_of_row(w, mn, fast_offsets(mn, kd), kd, code);
    // 16 codes, 2 bits each: a dot product of four code bytes with (1, 4, 16, 64) is a byte of the row
    constexpr uint32_t kWeights = 0x40100401u;
    const uint32_t own = __builtin_amdgcn_udot4(code[0], kWeights, 0u, false) |
                         (__builtin_amdgcn_udot4(code[1], kWeights, 0u, false) << 8) |
                         (__builtin_amdgcn_udot4(code[2], kWeights, 0u, false) << 16) |
                         (__builtin_amdgcn_udot4(code[3], kWeights, 0u, false) << 24);
    const uint32_t partner = (uint32_t)__builtin_amdgcn_mov_dpp((int)own, 0xB1 /* quad_perm [1,0,3,2] */, 0xf, 0xf, true);
    const uint32_t packed = __builtin_amdgcn_perm(partner, own, pick);
    __builtin_nontemporal_store(packed, (uint32_t*)(dst + t * kRowBytes + out_off));   // written once, read much later
    if (cg == 0) *(__half2*)(mdst + t * 4) = __halves2half2(__float2half_rn(scale), __float2half_rn(mn));
  }
}

__global__ __launch_bounds__(256) void quant_pack_v_kernel(
    const uint8_t* __restrict__ value, int64_t stride_b, int64_t stride_h, int64_t stride_t,
    int t_offset,
    const int64_t* __restrict__ page_table, int64_t pt_stride_b, int page_offset,
    uint8_t* __restrict__ cache, int64_t cache_stride_page,
    uint8_t* __restrict__ meta, int64_t meta_stride_page, int64_t cache_pages, int32_t* __restrict__ status) {
  const int p = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int64_t pg = page_table[(int64_t)b * pt_stride_b + page_offset + p];
  if (pg < 0 || pg >= cache_pages) {
    if (status && threadIdx.x == 0) status[b * KITTY_STATUS_FIELDS + KITTY_STATUS_BAD_PAGE_WRITE] = 1;
    return;
  }
  quant_v_page(StridedRows{value + (int64_t)b * stride_b + (int64_t)h * stride_h + (int64_t)(t_offset + p * kPage) * stride_t,
                           stride_t},
               cache + pg * cache_stride_page + (int64_t)h * kVBytes,
               meta + pg * meta_stride_page + (int64_t)h * kPage * 4);
}

// ---------------------------------------------------------------------------------------------
// Decode-time append and flush with per-sequence counters on the device (int32 [B][8], the
// KITTY_CNT_* fields).  The state machine is KittyCache.update's decode branch (kitty.py:97-123)
// and quantize_decode (kitty.py:194-236), per sequence instead of per batch.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void bump_status(const kitty_kv_layer& L, int b, int field, int by) {
  if (L.status) L.status[b * KITTY_STATUS_FIELDS + field] += by;   // one writer per sequence and launch
}

// k * cos + rotate_half(k) * sin for 4 channels starting at c, as fp16 tensor arithmetic evaluates it:
// each product and the sum rounded to fp16 (the product of two fp16 numbers is exact in fp32, and so
// is the sum of two, up to one rounding that rounding again to fp16 never alters).  Contraction is
// switched off: left on, the compiler folds the second product and the sum into one fp16 FMA, which
// skips a rounding the tensor expression has.
__device__ __forceinline__ uint2 rope4(uint2 own, uint2 partner, uint2 cs, uint2 sn, bool upper) {
#pragma clang fp contract(off)
  const uint32_t o[2] = {own.x, own.y}, q[2] = {partner.x, partner.y}, c[2] = {cs.x, cs.y}, s[2] = {sn.x, sn.y};
  uint32_t r[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    uint16_t out[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const float x = h2f((uint16_t)(o[i] >> (16 * k))), y = h2f((uint16_t)(q[i] >> (16 * k)));
      const float cc = h2f((uint16_t)(c[i] >> (16 * k))), ss = h2f((uint16_t)(s[i] >> (16 * k)));
      const float a = __half2float(__float2half_rn(x * cc));
      const float t = __half2float(__float2half_rn((upper ? y : -y) * ss));   // rotate_half: (-x2, x1)
      out[k] = __half_as_ushort(__float2half_rn(a + t));
    }
    r[i] = (uint32_t)out[0] | ((uint32_t)out[1] << 16);
  }
  return uint2{r[0], r[1]};
}

template <bool ROPE>
__global__ __launch_bounds__(256) void append_token_kernel(kitty_kv_layer L, const uint8_t* __restrict__ k_new,
                                                           const uint8_t* __restrict__ v_new, int64_t stride_b,
                                                           int64_t stride_h, const uint8_t* __restrict__ rope_cos,
                                                           const uint8_t* __restrict__ rope_sin, int64_t rope_stride_b) {
  const int b = blockIdx.x;
  int32_t* cnt = const_cast<int32_t*>(L.seq_counts) + b * KITTY_SEQ_COUNT_FIELDS;
  if (cnt[KITTY_CNT_FLAGS] & KITTY_SEQ_INACTIVE) return;   // the whole block: nobody reaches the barrier
  const int sink = cnt[KITTY_CNT_SINK], rk = cnt[KITTY_CNT_QBUF_K], rv = cnt[KITTY_CNT_QBUF_V];
  const int lv = cnt[KITTY_CNT_LOCAL_V], off = cnt[KITTY_CNT_LOCAL_OFF] & (kPage - 1);
  const bool to_sink = sink < L.S;
  // a full Q-buffer means the caller skipped a flush: drop the token rather than write out of bounds
  const bool ok = to_sink || (rk < kPage && (lv < kPage || rv < kPage));
  __syncthreads();   // every thread has read the counters before thread 0 rewrites them
  if (!ok) {
    if (threadIdx.x == 0) bump_status(L, b, KITTY_STATUS_TOKENS_DROPPED, 1);
    return;
  }
  for (int i = threadIdx.x; i < L.H_KV * 32; i += blockDim.x) {
    const int h = i >> 5, part = (i & 31) * 8;   // 8 bytes = 4 channels
    const uint8_t* krow = k_new + (int64_t)b * stride_b + (int64_t)h * stride_h;
    uint2 kk = *(const uint2*)(krow + part);
    if (ROPE) {
      const uint2 partner = *(const uint2*)(krow + (part ^ (kD)));   // the channel 64 away: 128 bytes
      const uint2 cs = *(const uint2*)(rope_cos + (int64_t)b * rope_stride_b + part);
      const uint2 sn = *(const uint2*)(rope_sin + (int64_t)b * rope_stride_b + part);
      kk = rope4(kk, partner, cs, sn, part >= kD);
    }
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

// blockIdx.z = 0: the K Q-buffer of (b, h) if it is full; 1: the V Q-buffer.
__global__ __launch_bounds__(256) void flush_full_kernel(kitty_kv_layer L) {
  const int h = blockIdx.x, b = blockIdx.y;
  const int32_t* cnt = L.seq_counts + b * KITTY_SEQ_COUNT_FIELDS;
  const int64_t w = (int64_t)b * L.win_stride_b + (int64_t)h * L.win_stride_h;
  if (cnt[KITTY_CNT_FLAGS] & KITTY_SEQ_INACTIVE) return;
  if (blockIdx.z == 0) {
    const int pk = cnt[KITTY_CNT_PAGES_K];
    if (cnt[KITTY_CNT_QBUF_K] != kPage || pk < 0 || pk >= L.MAX_PAGE) return;
    const int64_t pg = L.page_table_k[(int64_t)b * L.page_table_k_stride_b + pk];
    if (pg < 0 || pg >= L.cache_pages_k) return;
    quant_k_page<1>(StridedRows{(const uint8_t*)L.qbuf_k + w, kD * 2}, L.D_BOOSTED, nullptr, nullptr,
                    const_cast<uint8_t*>(L.key_cache) + pg * L.key_cache_stride_page + (int64_t)h * k_head_bytes(L.D_BOOSTED),
                    (uint8_t*)L.key_meta + pg * L.key_meta_stride_page + (int64_t)h * kD * 4);
  } else {
    const int pv = cnt[KITTY_CNT_PAGES_V];
    if (cnt[KITTY_CNT_QBUF_V] != kPage || pv < 0 || pv >= L.MAX_PAGE) return;
    const int64_t pg = L.page_table_v[(int64_t)b * L.page_table_v_stride_b + pv];
    if (pg < 0 || pg >= L.cache_pages_v) return;
    quant_v_page(StridedRows{(const uint8_t*)L.qbuf_v + w, kD * 2},
                 const_cast<uint8_t*>(L.value_cache) + pg * L.value_cache_stride_page + (int64_t)h * kVBytes,
                 (uint8_t*)L.value_meta + pg * L.value_meta_stride_page + (int64_t)h * kPage * 4);
  }
}

// after flush_full_kernel: the flushed Q-buffers are empty, their pages count.  The conditions are
// those under which flush_full_kernel wrote the page; a full Q-buffer that stays is recorded.
__global__ void advance_counts_kernel(kitty_kv_layer L, int B) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  int32_t* cnt = const_cast<int32_t*>(L.seq_counts) + b * KITTY_SEQ_COUNT_FIELDS;
  if (cnt[KITTY_CNT_FLAGS] & KITTY_SEQ_INACTIVE) return;
  const int pk = cnt[KITTY_CNT_PAGES_K], pv = cnt[KITTY_CNT_PAGES_V];
  int skipped = 0;
  bool bad = false;
  if (cnt[KITTY_CNT_QBUF_K] == kPage) {
    int64_t pg = -1;
    if (pk >= 0 && pk < L.MAX_PAGE) pg = L.page_table_k[(int64_t)b * L.page_table_k_stride_b + pk];
    if (pg >= 0 && pg < L.cache_pages_k) {
      cnt[KITTY_CNT_PAGES_K] = pk + 1;
      cnt[KITTY_CNT_QBUF_K] = 0;
    } else {
      ++skipped;
      bad |= pg != -1;
    }
  }
  if (cnt[KITTY_CNT_QBUF_V] == kPage) {
    int64_t pg = -1;
    if (pv >= 0 && pv < L.MAX_PAGE) pg = L.page_table_v[(int64_t)b * L.page_table_v_stride_b + pv];
    if (pg >= 0 && pg < L.cache_pages_v) {
      cnt[KITTY_CNT_PAGES_V] = pv + 1;
      cnt[KITTY_CNT_QBUF_V] = 0;
    } else {
      ++skipped;
      bad |= pg != -1;
    }
  }
  if (skipped) bump_status(L, b, KITTY_STATUS_FLUSH_SKIPPED, skipped);
  if (bad && L.status) L.status[b * KITTY_STATUS_FIELDS + KITTY_STATUS_BAD_PAGE_WRITE] = 1;
}

// ---------------------------------------------------------------------------------------------
// A chunk of T tokens per sequence in one go, with the state T single steps would leave.
//
// Per sequence the new rows (after those that still go to the sink) extend two streams of rows
// waiting to be packed.  K: [ Q_Buffer_K rows | chunk rows ].  V: [ Q_Buffer_V rows | the rows the
// ring gives up, oldest first | the chunk rows that pass through the ring and out again ]; the ring
// keeps the newest 128 rows.  Every full group of 128 stream rows is a page, quantized straight from
// wherever its rows lie; what is left of a stream is the new Q-buffer content.
// ---------------------------------------------------------------------------------------------
struct ChunkPlan {
  bool active, ok;
  int sink, pk, rk, pv, rv, lv, off;   // the sequence before the chunk
  int a, n;          // chunk rows that go to the sink / past it
  int npk, npv;      // new pages
  int e, er;         // rows leaving the ring (e), of which rows that were in it before (er)
  int rk2, rv2, lv2, off2;
};

// the counters part; `ok` still lacks the page ids (chunk_pages_ok)
__device__ inline ChunkPlan chunk_plan(const kitty_kv_layer& L, int b, int T) {
  const int32_t* cnt = L.seq_counts + b * KITTY_SEQ_COUNT_FIELDS;
  ChunkPlan p;
  p.active = !(cnt[KITTY_CNT_FLAGS] & KITTY_SEQ_INACTIVE);
  p.sink = cnt[KITTY_CNT_SINK]; p.pk = cnt[KITTY_CNT_PAGES_K]; p.rk = cnt[KITTY_CNT_QBUF_K];
  p.pv = cnt[KITTY_CNT_PAGES_V]; p.rv = cnt[KITTY_CNT_QBUF_V]; p.lv = cnt[KITTY_CNT_LOCAL_V];
  p.off = cnt[KITTY_CNT_LOCAL_OFF] & (kPage - 1);
  const bool sane = p.sink >= 0 && p.sink <= L.S && p.pk >= 0 && p.pv >= 0 && p.rk >= 0 && p.rv >= 0 && p.lv >= 0 &&
                    p.lv <= kPage && p.rk <= kPage && p.rv <= kPage;
  p.a = sane ? min(L.S - p.sink, T) : 0;
  p.n = T - p.a;
  p.npk = (p.rk + p.n) / kPage;
  p.rk2 = (p.rk + p.n) % kPage;
  p.lv2 = min(kPage, p.lv + p.n);
  p.e = p.lv + p.n - p.lv2;
  p.er = min(p.e, p.lv);
  p.npv = (p.rv + p.e) / kPage;
  p.rv2 = (p.rv + p.e) % kPage;
  p.off2 = (p.off + p.e) & (kPage - 1);
  // a Q-buffer that is still full (a flush found no page) takes nothing more, as in single steps
  p.ok = sane && (p.n == 0 || (p.rk < kPage && p.rv < kPage)) && p.pk + p.npk <= L.MAX_PAGE &&
         p.pv + p.npv <= L.MAX_PAGE;
  return p;
}
// every page the plan wants to write has a valid id; called by all threads of a block
__device__ inline bool chunk_pages_ok(const kitty_kv_layer& L, int b, const ChunkPlan& p) {
  int bad = 0;
  if (p.ok) {
    for (int i = threadIdx.x; i < p.npk + p.npv; i += blockDim.x) {
      const bool k = i < p.npk;
      const int64_t pg = k ? L.page_table_k[(int64_t)b * L.page_table_k_stride_b + p.pk + i]
                           : L.page_table_v[(int64_t)b * L.page_table_v_stride_b + p.pv + (i - p.npk)];
      bad |= pg < 0 || pg >= (k ? L.cache_pages_k : L.cache_pages_v);
    }
  }
  return p.ok && !__syncthreads_or(bad);
}

struct ChunkSrc {
  const uint8_t* k;   // chunk rows of this (b, h): row t at k + t * stride_t
  const uint8_t* v;
  int64_t stride_t;
};
// row s of the K stream / of the V stream of one (b, h)
struct KStreamRows {
  const uint8_t* qbuf; const uint8_t* chunk; int64_t stride_t; int rk, first;
  __device__ __forceinline__ const uint8_t* operator()(int t) const {
    const int s = first + t;
    return s < rk ? qbuf + (int64_t)s * (kD * 2) : chunk + (int64_t)(s - rk) * stride_t;
  }
  __device__ __forceinline__ const uint8_t* operator()(int t0, int r) const { return (*this)(t0 + r); }
};
struct VStreamRows {
  const uint8_t* qbuf; const uint8_t* ring; const uint8_t* chunk; int64_t stride_t; int rv, er, off, first;
  __device__ __forceinline__ const uint8_t* operator()(int t) const {
    const int s = first + t;
    if (s < rv) return qbuf + (int64_t)s * (kD * 2);
    if (s < rv + er) return ring + (int64_t)((off + s - rv) & (kPage - 1)) * (kD * 2);
    return chunk + (int64_t)(s - rv - er) * stride_t;
  }
};

// grid (2 * max_pages, H_KV, B): blockIdx.x < max_pages: new K page blockIdx.x, else new V page
__global__ __launch_bounds__(256) void chunk_quant_kernel(kitty_kv_layer L, const uint8_t* __restrict__ k_new,
                                                          const uint8_t* __restrict__ v_new, int64_t stride_b,
                                                          int64_t stride_h, int64_t stride_t, int T, int max_pages) {
  const int h = blockIdx.y, b = blockIdx.z;
  const bool vside = (int)blockIdx.x >= max_pages;
  const int p = vside ? blockIdx.x - max_pages : blockIdx.x;
  const ChunkPlan c = chunk_plan(L, b, T);
  if (!c.active || p >= (vside ? c.npv : c.npk)) return;        // uniform over the block
  if (!chunk_pages_ok(L, b, c)) return;
  const int64_t w = (int64_t)b * L.win_stride_b + (int64_t)h * L.win_stride_h;
  const int64_t src = (int64_t)b * stride_b + (int64_t)h * stride_h + (int64_t)c.a * stride_t;
  if (!vside) {
    const int64_t pg = L.page_table_k[(int64_t)b * L.page_table_k_stride_b + c.pk + p];
    quant_k_page<1>(KStreamRows{(const uint8_t*)L.qbuf_k + w, k_new + src, stride_t, c.rk, p * kPage}, L.D_BOOSTED,
                    nullptr, nullptr,
                    const_cast<uint8_t*>(L.key_cache) + pg * L.key_cache_stride_page + (int64_t)h * k_head_bytes(L.D_BOOSTED),
                    (uint8_t*)L.key_meta + pg * L.key_meta_stride_page + (int64_t)h * kD * 4);
  } else {
    const int64_t pg = L.page_table_v[(int64_t)b * L.page_table_v_stride_b + c.pv + p];
    quant_v_page(VStreamRows{(const uint8_t*)L.qbuf_v + w, (const uint8_t*)L.local_v + w, v_new + src, stride_t, c.rv,
                             c.er, c.off, p * kPage},
                 const_cast<uint8_t*>(L.value_cache) + pg * L.value_cache_stride_page + (int64_t)h * kVBytes,
                 (uint8_t*)L.value_meta + pg * L.value_meta_stride_page + (int64_t)h * kPage * 4);
  }
}

// grid (H_KV, B): the fp16 rows of one (b, h) after the chunk - sink rows, what is left of the two
// streams (the new Q-buffer contents) and the ring.  Runs after chunk_quant_kernel, which reads the
// old Q-buffers and ring.  Rows are moved by 16 lanes x 16 bytes.
__global__ __launch_bounds__(256) void chunk_rows_kernel(kitty_kv_layer L, const uint8_t* __restrict__ k_new,
                                                         const uint8_t* __restrict__ v_new, int64_t stride_b,
                                                         int64_t stride_h, int64_t stride_t, int T) {
  __shared__ uint4 s_stage[kPage][16];   // ring rows on their way to the V Q-buffer
  const int h = blockIdx.x, b = blockIdx.y;
  const ChunkPlan c = chunk_plan(L, b, T);
  if (!c.active) return;
  if (!chunk_pages_ok(L, b, c)) return;
  const int piece = threadIdx.x & 15, r0 = threadIdx.x >> 4;
  const int64_t w = (int64_t)b * L.win_stride_b + (int64_t)h * L.win_stride_h;
  const uint8_t* ksrc = k_new + (int64_t)b * stride_b + (int64_t)h * stride_h;
  const uint8_t* vsrc = v_new + (int64_t)b * stride_b + (int64_t)h * stride_h;
  auto row16 = [&](const uint8_t* p) { return ((const uint4*)p)[piece]; };
  // sink
  {
    const int64_t so = (int64_t)b * L.sink_stride_b + (int64_t)h * L.sink_stride_h;
    for (int i = r0; i < c.a; i += 16) {
      ((uint4*)((uint8_t*)L.sink_k + so + (int64_t)(c.sink + i) * (kD * 2)))[piece] = row16(ksrc + (int64_t)i * stride_t);
      ((uint4*)((uint8_t*)L.sink_v + so + (int64_t)(c.sink + i) * (kD * 2)))[piece] = row16(vsrc + (int64_t)i * stride_t);
    }
  }
  if (c.n == 0) return;
  ksrc += (int64_t)c.a * stride_t;
  vsrc += (int64_t)c.a * stride_t;
  // K: stream rows 128 npk + i -> Q_Buffer_K[i]; rows that already sit there stay (no page was cut)
  for (int i = (c.npk ? 0 : c.rk) + r0; i < c.rk2; i += 16)
    ((uint4*)((uint8_t*)L.qbuf_k + w + (int64_t)i * (kD * 2)))[piece] =
        row16(ksrc + (int64_t)(c.npk * kPage + i - c.rk) * stride_t);
  // V: the same, but a stream row may lie in the ring, whose slots are about to be overwritten:
  // those rows go through LDS
  const int v_first = c.npv * kPage;
  const int lo = c.npv ? 0 : c.rv;
  for (int i = lo + r0; i < c.rv2; i += 16) {
    const int s = v_first + i;
    if (s >= c.rv && s < c.rv + c.er)
      s_stage[i][piece] = row16((const uint8_t*)L.local_v + w + (int64_t)((c.off + s - c.rv) & (kPage - 1)) * (kD * 2));
  }
  __syncthreads();
  for (int i = lo + r0; i < c.rv2; i += 16) {
    const int s = v_first + i;
    const uint4 v = (s < c.rv + c.er) ? s_stage[i][piece] : row16(vsrc + (int64_t)(s - c.rv - c.er) * stride_t);
    ((uint4*)((uint8_t*)L.qbuf_v + w + (int64_t)i * (kD * 2)))[piece] = v;
  }
  // ring: the chunk rows that stay take the slots single steps would have given them
  const int base = c.lv < kPage ? c.lv : c.off;
  for (int j = c.e - c.er + r0; j < c.n; j += 16)
    ((uint4*)((uint8_t*)L.local_v + w + (int64_t)((base + j) & (kPage - 1)) * (kD * 2)))[piece] =
        row16(vsrc + (int64_t)j * stride_t);
}

// one block per sequence, after the two kernels above have read the old counters
__global__ __launch_bounds__(64) void chunk_advance_kernel(kitty_kv_layer L, int T) {
  const int b = blockIdx.x;
  const ChunkPlan c = chunk_plan(L, b, T);
  if (!c.active) return;
  const bool ok = chunk_pages_ok(L, b, c);
  if (threadIdx.x != 0) return;
  int32_t* cnt = const_cast<int32_t*>(L.seq_counts) + b * KITTY_SEQ_COUNT_FIELDS;
  if (!ok) {
    bump_status(L, b, KITTY_STATUS_TOKENS_DROPPED, T);
    return;
  }
  cnt[KITTY_CNT_SINK] = c.sink + c.a;
  cnt[KITTY_CNT_PAGES_K] = c.pk + c.npk;
  cnt[KITTY_CNT_QBUF_K] = c.rk2;
  cnt[KITTY_CNT_PAGES_V] = c.pv + c.npv;
  cnt[KITTY_CNT_QBUF_V] = c.rv2;
  cnt[KITTY_CNT_LOCAL_V] = c.lv2;
  cnt[KITTY_CNT_LOCAL_OFF] = c.off2;
}

int check_src(const void* p, int64_t sb, int64_t sh, int64_t st, int B, int H, int T, int D, int t_offset,
              int pages, int page_size) {
  KITTY_REQUIRE(p != nullptr, KITTY_E_NULL, "source tensor is NULL");
  KITTY_REQUIRE(head_dim_supported(D) && page_size == kPage, KITTY_E_SHAPE,
                "kernels are built for head_dim 64, 128 or 256 and page_size 128, got D=%d page_size=%d", D, page_size);
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
  KITTY_REQUIRE(d_boost >= 0 && d_boost <= D && d_boost <= 255, KITTY_E_SHAPE,
                "d_boost must be in [0, %d] and fit the uint8 slot map, got %d", D, d_boost);
  if (B == 0 || pages == 0) return 0;
  if (D != kD) {
    launch_quant_k_any(D, 2, key, stride_b, stride_h, stride_t, B, H, t_offset, pages, d_boost, nullptr, slot_map,
                       nullptr, 0, 0, nullptr, 0, nullptr, 0, 0, nullptr, (hipStream_t)stream);
    return check_launch("kitty_select_boost_k");
  }
  hipLaunchKernelGGL(quant_pack_k_kernel<2>, dim3(pages, H, B), dim3(256), 0, (hipStream_t)stream,
                     (const uint8_t*)key, stride_b, stride_h, stride_t, t_offset, d_boost, nullptr, slot_map,
                     pages, nullptr, 0, 0, nullptr, 0, nullptr, 0, 0, nullptr);
  return check_launch("kitty_select_boost_k");
}

extern "C" int kitty_quant_pack_k(const void* key, int64_t stride_b, int64_t stride_h, int64_t stride_t,
                                  int B, int H, int T, int D, int t_offset, int pages, int page_size, int d_boost,
                                  const uint8_t* slot_map,
                                  const int64_t* page_table, int64_t page_table_stride_b, int page_offset,
                                  uint8_t* cache, int64_t cache_stride_page,
                                  void* meta, int64_t meta_stride_page, int64_t cache_pages, int32_t* status,
                                  void* stream) {
  if (int rc = check_src(key, stride_b, stride_h, stride_t, B, H, T, D, t_offset, pages, page_size)) return rc;
  KITTY_REQUIRE(((uintptr_t)status % 4) == 0, KITTY_E_ALIGN, "status needs 4-byte alignment");
  // the slot map is a uint8 with d_boost as the "not boosted" marker, and the high plane has
  // d_boost rows: keep rows 4-byte friendly
  KITTY_REQUIRE(d_boost >= 0 && d_boost <= D && d_boost <= 255, KITTY_E_SHAPE,
                "d_boost must be in [0, %d] and fit the uint8 slot map, got %d", D, d_boost);
  KITTY_REQUIRE((k_head_bytes_d(D, d_boost) % 16) == 0, KITTY_E_ALIGN,
                "d_boost=%d gives a per-head page size that is not a multiple of 16 bytes", d_boost);
  if (int rc = check_dst(page_table, page_offset, cache, cache_stride_page, meta, meta_stride_page, cache_pages,
                         (int64_t)H * k_head_bytes_d(D, d_boost), (int64_t)H * D * 4))
    return rc;
  if (B == 0 || pages == 0) return 0;
  if (D != kD) {
    launch_quant_k_any(D, slot_map ? 0 : 1, key, stride_b, stride_h, stride_t, B, H, t_offset, pages, d_boost, slot_map,
                       nullptr, page_table, page_table_stride_b, page_offset, cache, cache_stride_page, meta,
                       meta_stride_page, cache_pages, status, (hipStream_t)stream);
    return check_launch("kitty_quant_pack_k");
  }
  dim3 grid(pages, H, B), block(256);
  if (slot_map)
    hipLaunchKernelGGL(quant_pack_k_kernel<0>, grid, block, 0, (hipStream_t)stream, (const uint8_t*)key, stride_b,
                       stride_h, stride_t, t_offset, d_boost, slot_map, nullptr, pages, page_table,
                       page_table_stride_b, page_offset, cache, cache_stride_page, (uint8_t*)meta,
                       meta_stride_page, cache_pages, status);
  else
    hipLaunchKernelGGL(quant_pack_k_kernel<1>, grid, block, 0, (hipStream_t)stream, (const uint8_t*)key, stride_b,
                       stride_h, stride_t, t_offset, d_boost, nullptr, nullptr, pages, page_table,
                       page_table_stride_b, page_offset, cache, cache_stride_page, (uint8_t*)meta,
                       meta_stride_page, cache_pages, status);
  return check_launch("kitty_quant_pack_k");
}

extern "C" int kitty_quant_pack_v(const void* value, int64_t stride_b, int64_t stride_h, int64_t stride_t,
                                  int B, int H, int T, int D, int t_offset, int pages, int page_size,
                                  const int64_t* page_table, int64_t page_table_stride_b, int page_offset,
                                  uint8_t* cache, int64_t cache_stride_page,
                                  void* meta, int64_t meta_stride_page, int64_t cache_pages, int32_t* status,
                                  void* stream) {
  if (int rc = check_src(value, stride_b, stride_h, stride_t, B, H, T, D, t_offset, pages, page_size)) return rc;
  KITTY_REQUIRE(((uintptr_t)status % 4) == 0, KITTY_E_ALIGN, "status needs 4-byte alignment");
  if (int rc = check_dst(page_table, page_offset, cache, cache_stride_page, meta, meta_stride_page, cache_pages,
                         (int64_t)H * v_head_bytes_d(D), (int64_t)H * kPage * 4))
    return rc;
  if (B == 0 || pages == 0) return 0;
  if (D != kD) {
    launch_quant_v_any(D, value, stride_b, stride_h, stride_t, B, H, t_offset, pages, page_table, page_table_stride_b,
                       page_offset, cache, cache_stride_page, meta, meta_stride_page, cache_pages, status,
                       (hipStream_t)stream);
    return check_launch("kitty_quant_pack_v");
  }
  hipLaunchKernelGGL(quant_pack_v_kernel, dim3(pages, H, B), dim3(256), 0, (hipStream_t)stream,
                     (const uint8_t*)value, stride_b, stride_h, stride_t, t_offset, page_table,
                     page_table_stride_b, page_offset, cache, cache_stride_page, (uint8_t*)meta, meta_stride_page,
                     cache_pages, status);
  return check_launch("kitty_quant_pack_v");
}

namespace {
int check_append_layer(const kitty_kv_layer* layer, int B) {
  KITTY_REQUIRE(layer != nullptr, KITTY_E_NULL, "layer is NULL");
  const kitty_kv_layer& L = *layer;
  KITTY_REQUIRE(L.seq_counts != nullptr, KITTY_E_NULL, "this entry point needs per-sequence counters (seq_counts)");
  KITTY_REQUIRE(L.D == kD && L.PAGE_SIZE == kPage, KITTY_E_SHAPE,
                "the device-counter entry points are built for head_dim 128 and page_size 128 (other head dimensions "
                "keep the counters on the host), got D=%d page_size=%d", L.D, L.PAGE_SIZE);
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
                    L.win_stride_b % 16 == 0 && L.win_stride_h % 16 == 0 && ((uintptr_t)L.seq_counts % 4) == 0 &&
                    ((uintptr_t)L.status % 4) == 0,
                KITTY_E_ALIGN, "cache tensors need 16-byte alignment");
  KITTY_REQUIRE(L.cache_pages_k >= 0 && L.cache_pages_v >= 0, KITTY_E_RANGE, "negative cache_pages_k / cache_pages_v");
  KITTY_REQUIRE(L.key_cache_stride_page >= (int64_t)L.H_KV * k_head_bytes(L.D_BOOSTED) &&
                    L.value_cache_stride_page >= (int64_t)L.H_KV * kVBytes &&
                    L.key_meta_stride_page >= (int64_t)L.H_KV * kD * 4 &&
                    L.value_meta_stride_page >= (int64_t)L.H_KV * kPage * 4,
                KITTY_E_RANGE, "a page stride is smaller than one page");
  return 0;
}
}  // namespace

extern "C" int kitty_append_token(const kitty_kv_layer* layer, const void* k_new, const void* v_new,
                                  int64_t stride_b, int64_t stride_h, const void* rope_cos, const void* rope_sin,
                                  int64_t rope_stride_b, int B, void* stream) {
  if (int rc = check_append_layer(layer, B)) return rc;
  KITTY_REQUIRE(k_new && v_new, KITTY_E_NULL, "k_new / v_new is NULL");
  KITTY_REQUIRE(((uintptr_t)k_new % 8) == 0 && ((uintptr_t)v_new % 8) == 0 && stride_b % 8 == 0 && stride_h % 8 == 0,
                KITTY_E_ALIGN, "k_new / v_new need 8-byte aligned bases and strides");
  KITTY_REQUIRE((rope_cos == nullptr) == (rope_sin == nullptr), KITTY_E_NULL, "rope_cos and rope_sin go together");
  if (rope_cos) {
    KITTY_REQUIRE(((uintptr_t)rope_cos % 8) == 0 && ((uintptr_t)rope_sin % 8) == 0 && rope_stride_b % 8 == 0 &&
                      (rope_stride_b == 0 || rope_stride_b >= kD * 2),
                  KITTY_E_ALIGN, "rope_cos / rope_sin need 8-byte aligned rows of D fp16 values");
    hipLaunchKernelGGL(append_token_kernel<true>, dim3(B), dim3(256), 0, (hipStream_t)stream, *layer,
                       (const uint8_t*)k_new, (const uint8_t*)v_new, stride_b, stride_h, (const uint8_t*)rope_cos,
                       (const uint8_t*)rope_sin, rope_stride_b);
  } else {
    hipLaunchKernelGGL(append_token_kernel<false>, dim3(B), dim3(256), 0, (hipStream_t)stream, *layer,
                       (const uint8_t*)k_new, (const uint8_t*)v_new, stride_b, stride_h, nullptr, nullptr, 0);
  }
  return check_launch("kitty_append_token");
}

extern "C" int kitty_flush_full(const kitty_kv_layer* layer, int B, void* stream) {
  if (int rc = check_append_layer(layer, B)) return rc;
  hipLaunchKernelGGL(flush_full_kernel, dim3(layer->H_KV, B, 2), dim3(256), 0, (hipStream_t)stream, *layer);
  hipLaunchKernelGGL(advance_counts_kernel, dim3((B + 63) / 64), dim3(64), 0, (hipStream_t)stream, *layer, B);
  return check_launch("kitty_flush_full");
}

extern "C" int kitty_append_chunk(const kitty_kv_layer* layer, const void* k_new, const void* v_new,
                                  int64_t stride_b, int64_t stride_h, int64_t stride_t, int B, int T, void* stream) {
  if (int rc = check_append_layer(layer, B)) return rc;
  KITTY_REQUIRE(k_new && v_new, KITTY_E_NULL, "k_new / v_new is NULL");
  KITTY_REQUIRE(T >= 1 && T <= (1 << 24), KITTY_E_RANGE, "T=%d out of range", T);
  KITTY_REQUIRE(((uintptr_t)k_new % 16) == 0 && ((uintptr_t)v_new % 16) == 0 && stride_b % 16 == 0 &&
                    stride_h % 16 == 0 && stride_t % 16 == 0 && stride_t >= kD * 2,
                KITTY_E_ALIGN, "k_new / v_new need 16-byte aligned bases and strides with D contiguous");
  const int max_pages = (T + kPage - 1) / kPage;   // a stream holds at most 127 rows before the chunk
  const hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(chunk_quant_kernel, dim3(2 * max_pages, layer->H_KV, B), dim3(256), 0, st, *layer,
                     (const uint8_t*)k_new, (const uint8_t*)v_new, stride_b, stride_h, stride_t, T, max_pages);
  hipLaunchKernelGGL(chunk_rows_kernel, dim3(layer->H_KV, B), dim3(256), 0, st, *layer, (const uint8_t*)k_new,
                     (const uint8_t*)v_new, stride_b, stride_h, stride_t, T);
  hipLaunchKernelGGL(chunk_advance_kernel, dim3(B), dim3(64), 0, st, *layer, T);
  return check_launch("kitty_append_chunk");
}
