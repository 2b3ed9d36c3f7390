// Decode attention, plain variant: the reference's order of operations (dequantize a tile to fp16
// with fp16 arithmetic, fp32 dot products) in one fused split-K pass on the vector ALUs.  Logits
// and probabilities stay fp32 (the reference rounds both to fp16, kitty_attention.py:169,473,
// which costs it accuracy and nothing else).  It is the readable baseline the matrix-core kernel is checked against on the
// GPU and it accepts every boost count; it is not the fast path.
#include "decode_common.h"

using namespace kitty;

namespace kitty {

constexpr int kMaxHeadBytes = kRowBytes * (kD + kD) + kD;   // d_boost up to D

// fp16(code) * scale + zero with BOTH operations rounded to fp16, as eager torch and the Triton
// interpreter evaluate kitty_attention.py:162-165 and :317-320.  Written on _Float16 with
// contraction switched off for this function: a fused multiply-add would round once and move
// large-magnitude channels by up to an fp16 ulp.
__device__ inline float dequant_ref(uint32_t code, __half scale, __half zero) {
#pragma clang fp contract(off)
  const _Float16 s = static_cast<__half_raw>(scale).data;
  const _Float16 z = static_cast<__half_raw>(zero).data;
  const _Float16 c = (_Float16)(float)code;
  const _Float16 prod = c * s;
  const _Float16 r = prod + z;
  return (float)r;
}

// ROWS: 4, 8 or 16 query heads per kv head at most (a group of 4 does not pay for 16).
template <int ROWS>
__global__ __launch_bounds__(256) void decode_plain_kernel(kitty_kv_layer L, const __half* __restrict__ q, int H_Q,
                                                           float scaling, float* __restrict__ ws_ml,
                                                           float* __restrict__ ws_acc, int num_splits) {
  const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int G = H_Q / L.H_KV;
  const int DB = L.D_BOOSTED;
  const SeqCounts c = load_counts(L, b);
  const int per = (c.ntiles + num_splits - 1) / num_splits;
  const int tile_begin = split * per, tile_end = min(c.ntiles, tile_begin + per);
  int bad_page = 0;

  __shared__ __attribute__((aligned(16))) float s_q[kD][ROWS];      // [channel][head]: a thread reads the heads of a channel at once
  __shared__ __attribute__((aligned(16))) uint8_t s_codes[kMaxHeadBytes];
  __shared__ __half2 s_meta[kD];
  __shared__ __attribute__((aligned(16))) float s_p[kPage][ROWS];   // [token][head]
  __shared__ float s_part[2][ROWS][kPage];
  __shared__ float s_m[ROWS], s_l[ROWS], s_alpha[ROWS];

  for (int i = tid; i < G * kD; i += 256)
    s_q[i % kD][i / kD] = __half2float(q[((int64_t)b * H_Q + (int64_t)h * G) * kD + i]);
  if (tid < ROWS) { s_m[tid] = -INFINITY; s_l[tid] = 0.f; }
  float acc_o[ROWS];
#pragma unroll
  for (int g = 0; g < ROWS; ++g) acc_o[g] = 0.f;
  __syncthreads();

  const int t = tid & 127, half = tid >> 7;
  const int64_t sink_base = (int64_t)b * L.sink_stride_b + (int64_t)h * L.sink_stride_h;
  const int64_t win_base = (int64_t)b * L.win_stride_b + (int64_t)h * L.win_stride_h;

  for (int tile = tile_begin; tile < tile_end; ++tile) {
    const int body = tile - 1;                                  // -1 = sink
    const int ntok = tile == 0 ? c.sink : min(kPage, c.nbody - body * kPage);
    const bool k_packed = tile > 0 && body < c.pk;
    const bool v_packed = tile > 0 && body < c.pv;

    // ---- logits -----------------------------------------------------------------------------
    float acc[ROWS];
#pragma unroll
    for (int g = 0; g < ROWS; ++g) acc[g] = 0.f;
    if (k_packed) {
      const int64_t pg = checked_page(page_id(L.page_table_k, (int64_t)b * L.page_table_k_stride_b + body), L.cache_pages_k, bad_page);
      const uint8_t* src = L.key_cache + pg * L.key_cache_stride_page + (int64_t)h * k_head_bytes(DB);
      for (int i = tid; i < k_head_bytes(DB) / 16; i += 256) ((uint4*)s_codes)[i] = ((const uint4*)src)[i];
      if (tid < kD)
        s_meta[tid] = *(const __half2*)((const uint8_t*)L.key_meta + pg * L.key_meta_stride_page +
                                        ((int64_t)h * kD + tid) * 4);
      __syncthreads();
      const int sh = 2 * (t & 3);
      const uint8_t* idx = s_codes + kRowBytes * (kD + DB);
      for (int d = half * 64; d < half * 64 + 64; ++d) {
        uint32_t code = (s_codes[d * kRowBytes + (t >> 2)] >> sh) & 3u;
        const uint32_t slot = idx[d];
        if (slot < (uint32_t)DB) code |= ((s_codes[kLoBytes + slot * kRowBytes + (t >> 2)] >> sh) & 3u) << 2;
        const __half2 m = s_meta[d];
        const float x = dequant_ref(code, __low2half(m), __high2half(m));
#pragma unroll
        for (int g = 0; g < ROWS; ++g)
          if (g < G) acc[g] += s_q[d][g] * x;
      }
    } else if (t < ntok) {
      const __half* row = tile == 0 ? (const __half*)((const uint8_t*)L.sink_k + sink_base) + (int64_t)t * kD
                                    : (const __half*)((const uint8_t*)L.qbuf_k + win_base) + (int64_t)t * kD;
      for (int d = half * 64; d < half * 64 + 64; ++d) {
        const float x = __half2float(row[d]);
#pragma unroll
        for (int g = 0; g < ROWS; ++g)
          if (g < G) acc[g] += s_q[d][g] * x;
      }
    }
#pragma unroll
    for (int g = 0; g < ROWS; ++g)
      if (g < G) s_part[half][g][t] = acc[g];
    __syncthreads();

    // ---- online softmax: one wave per query head ---------------------------------------------
    for (int g = wave; g < G; g += 4) {
      float v0 = -INFINITY, v1 = -INFINITY;
      if (lane < ntok) v0 = (s_part[0][g][lane] + s_part[1][g][lane]) * scaling;
      if (lane + 64 < ntok) v1 = (s_part[0][g][lane + 64] + s_part[1][g][lane + 64]) * scaling;
      float mx = fmaxf(v0, v1);
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
      const float m_old = s_m[g];
      const float m_new = fmaxf(m_old, mx);
      const float p0 = (v0 == -INFINITY) ? 0.f : __expf(v0 - m_new);
      const float p1 = (v1 == -INFINITY) ? 0.f : __expf(v1 - m_new);
      float sum = p0 + p1;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
      const float alpha = (m_old == -INFINITY) ? 0.f : __expf(m_old - m_new);
      s_p[lane][g] = p0;
      s_p[lane + 64][g] = p1;
      if (lane == 0) { s_m[g] = m_new; s_l[g] = s_l[g] * alpha + sum; s_alpha[g] = alpha; }
    }
    // ---- stage V ---------------------------------------------------------------------------
    if (v_packed) {
      const int64_t pg = checked_page(page_id(L.page_table_v, (int64_t)b * L.page_table_v_stride_b + body), L.cache_pages_v, bad_page);
      const uint8_t* src = L.value_cache + pg * L.value_cache_stride_page + (int64_t)h * kVBytes;
      ((uint4*)s_codes)[tid] = ((const uint4*)src)[tid];
      if (tid < kPage)
        s_meta[tid] = *(const __half2*)((const uint8_t*)L.value_meta + pg * L.value_meta_stride_page +
                                        ((int64_t)h * kPage + tid) * 4);
    }
    __syncthreads();

    // ---- out += P V : thread = (channel, half of the tile's tokens) ---------------------------
    {
      const int d = t;
#pragma unroll
      for (int g = 0; g < ROWS; ++g)
        if (g < G) acc_o[g] *= s_alpha[g];
      const int t0 = half * 64, t1 = min(ntok, half * 64 + 64);
      for (int tt = t0; tt < t1; ++tt) {
        float x;
        if (v_packed) {
          const uint32_t code = (s_codes[tt * kRowBytes + (d >> 2)] >> (2 * (d & 3))) & 3u;
          const __half2 m = s_meta[tt];
          x = dequant_ref(code, __low2half(m), __high2half(m));
        } else if (tile == 0) {
          x = __half2float(((const __half*)((const uint8_t*)L.sink_v + sink_base))[(int64_t)tt * kD + d]);
        } else {
          x = __half2float(v_tail_row(L, c, b, h, (body - c.pv) * kPage + tt)[d]);
        }
#pragma unroll
        for (int g = 0; g < ROWS; ++g)
          if (g < G) acc_o[g] += s_p[tt][g] * x;
      }
    }
    __syncthreads();
  }

  if (tid == 0) report_bad_page(L, b, bad_page);
  // ---- write this split's partial --------------------------------------------------------------
#pragma unroll
  for (int g = 0; g < ROWS; ++g)
    if (g < G) s_part[half][g][t] = acc_o[g];
  __syncthreads();
  for (int i = tid; i < G * kD; i += 256) {
    const int g = i / kD, d = i % kD;
    const int64_t row = ((int64_t)b * H_Q + (int64_t)h * G + g) * num_splits + split;
    ws_acc[row * kD + d] = s_part[0][g][d] + s_part[1][g][d];
    if (d == 0) { ws_ml[row * 2] = s_m[g] * 1.44269504088896f; ws_ml[row * 2 + 1] = s_l[g]; }
  }
}

// out[b, 0, hq, :] = sum_s acc_s * 2^(m_s - m) / sum_s l_s * 2^(m_s - m); the running maxima of
// the partials are in log2 units.  One block per (CH channels, query head, batch row).  GROUPS
// groups of CH lanes stride over the splits; a thread asks for everything it will read - the
// (max, sum) pairs and its channel of the accumulator rows of up to eight splits at a time, the
// indices clamped instead of tested so that no load waits for a branch - and folds the splits into
// one partial of its own as they arrive (the partials were written by other XCDs a moment ago and
// come from memory: one round trip instead of the two that "first the maximum, then the sums"
// costs).  The groups' partials are combined through LDS in a fixed order.  GROUPS = 8 up to 32
// splits (2 for a large batch), 32 beyond (a long sequence at batch 1 has hundreds of splits).
// CH: a launch of thousands of one-wave blocks is bound by the rate at which blocks are handed out,
// not by its loads - all 128 channels of a head in one block where there are many heads.
// kBatch: splits a thread asks for at a time (the launcher picks the smallest of 2, 4, 8 that covers a
// group's share).
template <int GROUPS, int kMergeChannels, int kBatch>
__global__ __launch_bounds__(GROUPS * kMergeChannels) void decode_merge_kernel(
    const float* __restrict__ ws_ml, const float* __restrict__ ws_acc, __half* __restrict__ out, int num_splits) {
  static_assert(kD % kMergeChannels == 0 && (GROUPS * kMergeChannels) % 64 == 0, "whole waves, whole heads");
  __shared__ float s_m[GROUPS], s_l[GROUPS], s_o[GROUPS][kMergeChannels];
  const int64_t head = (int64_t)blockIdx.z * gridDim.y + blockIdx.y;
  const int64_t row0 = head * num_splits;
  const int lane = threadIdx.x % kMergeChannels, grp = threadIdx.x / kMergeChannels;
  const int d = blockIdx.x * kMergeChannels + lane;
  float m = -INFINITY, l = 0.f, o = 0.f;
  for (int s0 = grp; s0 < num_splits; s0 += GROUPS * kBatch) {
    float ms[kBatch], ls[kBatch], as[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      const int s = s0 + i * GROUPS;
      const int64_t row = row0 + (s < num_splits ? s : s0);
      ms[i] = ws_ml[row * 2];
      ls[i] = ws_ml[row * 2 + 1];
      as[i] = ws_acc[row * kD + d];
      if (s >= num_splits) ms[i] = -INFINITY;
    }
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      // an empty split (max = -inf; its accumulator row may never have been written) changes nothing
      const bool live = ms[i] != -INFINITY;
      const float mn = live ? fmaxf(m, ms[i]) : m;
      const float wa = live ? exp2f(m - mn) : 1.f;   // (m = -inf at first: 2^-inf = 0)
      const float wb = live ? exp2f(ms[i] - mn) : 0.f;
      l = l * wa + (live ? ls[i] : 0.f) * wb;
      o = o * wa + (live ? as[i] : 0.f) * wb;
      m = mn;
    }
  }
  if (lane == 0) s_m[grp] = m, s_l[grp] = l;
  s_o[grp][lane] = o;
  __syncthreads();
  if (grp == 0) {
    float mm = -INFINITY;
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) mm = fmaxf(mm, s_m[g]);
    l = 0.f, o = 0.f;
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
      const float w = s_m[g] != -INFINITY ? exp2f(s_m[g] - mm) : 0.f;
      l += s_l[g] * w;
      o += s_o[g][lane] * w;
    }
    out[head * kD + d] = __float2half_rn(l > 0.f ? o / l : 0.f);
  }
}

void launch_decode_plain(const kitty_kv_layer& L, const void* q, int B, int H_Q, float scaling, float* ws_ml,
                         float* ws_acc, int num_splits, hipStream_t stream) {
  const int G = H_Q / L.H_KV;
  const dim3 grid(num_splits, L.H_KV, B), block(256);
  if (G <= 4)
    hipLaunchKernelGGL(decode_plain_kernel<4>, grid, block, 0, stream, L, (const __half*)q, H_Q, scaling, ws_ml, ws_acc, num_splits);
  else if (G <= 8)
    hipLaunchKernelGGL(decode_plain_kernel<8>, grid, block, 0, stream, L, (const __half*)q, H_Q, scaling, ws_ml, ws_acc, num_splits);
  else
    hipLaunchKernelGGL(decode_plain_kernel<16>, grid, block, 0, stream, L, (const __half*)q, H_Q, scaling, ws_ml, ws_acc, num_splits);
}

namespace {
template <int GROUPS, int CH>
void launch_merge(const float* ws_ml, const float* ws_acc, void* out, int B, int H_Q, int num_splits, hipStream_t stream) {
  const dim3 grid(kD / CH, H_Q, B), block(GROUPS * CH);
  const int share = (num_splits + GROUPS - 1) / GROUPS;
  if (share <= 2)
    hipLaunchKernelGGL((decode_merge_kernel<GROUPS, CH, 2>), grid, block, 0, stream, ws_ml, ws_acc, (__half*)out, num_splits);
  else if (share <= 4)
    hipLaunchKernelGGL((decode_merge_kernel<GROUPS, CH, 4>), grid, block, 0, stream, ws_ml, ws_acc, (__half*)out, num_splits);
  else
    hipLaunchKernelGGL((decode_merge_kernel<GROUPS, CH, 8>), grid, block, 0, stream, ws_ml, ws_acc, (__half*)out, num_splits);
}
}  // namespace

void launch_decode_merge(const float* ws_ml, const float* ws_acc, void* out, int B, int H_Q, int num_splits,
                         hipStream_t stream) {
  const int64_t heads = (int64_t)B * H_Q;
  if (num_splits <= 32 && heads >= 1024) launch_merge<2, kD>(ws_ml, ws_acc, out, B, H_Q, num_splits, stream);   // large batch
  else if (num_splits <= 32 && heads >= 256) launch_merge<8, 64>(ws_ml, ws_acc, out, B, H_Q, num_splits, stream);
  else if (num_splits <= 32) launch_merge<8, 32>(ws_ml, ws_acc, out, B, H_Q, num_splits, stream);
  else launch_merge<32, 32>(ws_ml, ws_acc, out, B, H_Q, num_splits, stream);
}

}  // namespace kitty
