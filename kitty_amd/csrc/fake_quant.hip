// Fake quantization of dense fp16 K / V in place: the arithmetic of the reference's accuracy
// simulator, fake_quant_groupwise_lastdim (src/kitty_sim/utils_quant.py:64-114), as it evaluates on a
// GPU for fp16 tensors: every torch operator of its chain computes in fp32 and rounds its result to
// fp16, and a division by a Python scalar multiplies by the scalar's fp32 reciprocal.
//
//   mn, mx   = min / max of the group                               (:90-91)
//   rng      = fp16(max(fp16(mx - mn), 1e-4f))                      (:92, :96-97 or :106)
//   scale    = fp16(rng * (1.f / qmax)),  qmax = 2^bit - 1, or 2^promote_bit - 1 where the mask is set
//   q        = rint(clamp(fp16(fp16(x - mn) / scale), 0, qmax))     (:112: clamp first, then round half to even)
//   result   = fp16(fp16(q * scale) + mn)                           (:113)
//
// A tile is 128 tokens x 128 channels of one (batch row, head), 256 threads.
// AXIS 0: groups run along the tokens (keys: one channel over group_size tokens; the reference
// transposes K to [B, nh, D, T] for this, kitty_simulate.py:204-207), optional promote mask per
// channel.  A thread owns two channels (4 bytes) of 32 consecutive tokens, a wave one quarter of the
// tile's tokens: a wave's load is one whole token row, the minimum and maximum of a 32-token group
// never leave the thread, and larger groups combine two or four waves through 4 KB of LDS.
// AXIS 1: groups run along the channels (values: one token over group_size channels).  A thread owns
// 8 channels (16 bytes) of the 8 tokens r*16 + tg, a token row is 16 lanes, groups combine by shuffles.
#include "kitty_common.h"

namespace kitty {
namespace {

__device__ __forceinline__ float hr(float v) { return __half2float(__float2half_rn(v)); }

struct GroupParams { float mn, scale, rscale, qmax; };

__device__ __forceinline__ GroupParams group_params(float mn, float mx, float qmax, float inv_qmax) {
  float rng = hr(mx - mn);
  rng = hr(fmaxf(rng, 1e-4f));
  const float scale = hr(rng * inv_qmax);
  return GroupParams{mn, scale, __frcp_rn(scale), qmax};
}

// The quotient (x - mn) / scale is needed rounded to fp32 and then to fp16.  d * (1 / scale) is
// within 3 ulp of the fp32 quotient, so both round to the same fp16 number unless the product
// lies within 4 ulp of the midpoint of two fp16 numbers (the 13 bits fp16 drops read 0x1000 +- 4),
// or in fp16's subnormal range, where more bits are dropped: a wave with such a lane (one in
// twenty) divides.
__device__ __forceinline__ float fake_quant_one(float x, const GroupParams& g) {
  const float d = hr(x - g.mn);
  float q = d * g.rscale;
  const uint32_t low = __float_as_uint(q) & 0x1fffu;
  const bool unsure = (low - 0x0ffcu <= 8u) || (q != 0.f && q < 6.2e-5f) || !(q < 65000.f);
  if (__builtin_expect(__any(unsure), 0)) q = __fdiv_rn(d, g.scale);
  q = rintf(fminf(fmaxf(hr(q), 0.f), g.qmax));
  return hr(hr(q * g.scale) + g.mn);
}

__device__ __forceinline__ void unpack8(const uint4& raw, float (&x)[8]) {
  const __half2* p = (const __half2*)&raw;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float2 f = __half22float2(p[j]);
    x[2 * j] = f.x;
    x[2 * j + 1] = f.y;
  }
}

__device__ __forceinline__ uint4 pack8(const float (&x)[8]) {
  uint4 raw;
  __half2* p = (__half2*)&raw;
#pragma unroll
  for (int j = 0; j < 4; ++j) p[j] = __floats2half2_rn(x[2 * j], x[2 * j + 1]);
  return raw;
}

template <int AXIS, int GS>
__global__ __launch_bounds__(256) void fake_quant_kernel(uint8_t* __restrict__ data, int64_t stride_b, int64_t stride_h,
                                                         int64_t stride_t, int t_offset, int n_tokens, float qmax,
                                                         float inv_qmax, float qmax_promote, float inv_qmax_promote,
                                                         const uint8_t* __restrict__ mask, int64_t mask_stride_b,
                                                         int64_t mask_stride_h, int64_t mask_stride_tile) {
  const int tile = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int n_here = min(kPage, n_tokens - tile * kPage);
  uint8_t* tile_base = data + (int64_t)b * stride_b + (int64_t)h * stride_h + (int64_t)(t_offset + tile * kPage) * stride_t;

  if constexpr (AXIS == 1) {
    const int cg = threadIdx.x & 15, tg = threadIdx.x >> 4;
    uint8_t* base = tile_base + cg * 16;
    uint4 raw[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int tok = r * 16 + tg;
      raw[r] = tok < n_here ? *(const uint4*)(base + (int64_t)tok * stride_t) : uint4{0, 0, 0, 0};
    }
    // one token row = 16 lanes; a group = GS / 8 neighbouring lanes
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      float x[8];
      unpack8(raw[r], x);
      float mn = x[0], mx = x[0];
#pragma unroll
      for (int j = 1; j < 8; ++j) { mn = fminf(mn, x[j]); mx = fmaxf(mx, x[j]); }
#pragma unroll
      for (int o = 1; o * 8 < GS; o <<= 1) {
        mn = fminf(mn, __shfl_xor(mn, o));
        mx = fmaxf(mx, __shfl_xor(mx, o));
      }
      const GroupParams g = group_params(mn, mx, qmax, inv_qmax);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] = fake_quant_one(x[j], g);
      const int tok = r * 16 + tg;
      if (tok < n_here) *(uint4*)(base + (int64_t)tok * stride_t) = pack8(x);
    }
  } else {
    // channels 2cp, 2cp+1; tokens 32wq .. 32wq+31 (wq = the wave's number, uniform)
    const int cp = threadIdx.x & 63, wq = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool live = wq * 32 < n_here;                            // n_tokens is a multiple of GS >= 32
    uint8_t* base = tile_base + (int64_t)(wq * 32) * stride_t;
    const uint32_t lane_off = cp * 4;
    uint32_t raw[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) raw[i] = live ? *(const uint32_t*)(base + (int64_t)i * stride_t + lane_off) : 0u;
    float mn0 = INFINITY, mx0 = -INFINITY, mn1 = INFINITY, mx1 = -INFINITY;
    if (live) {
#pragma unroll
      for (int i = 0; i < 32; ++i) {
        const float2 f = __half22float2(*(const __half2*)&raw[i]);
        mn0 = fminf(mn0, f.x); mx0 = fmaxf(mx0, f.x);
        mn1 = fminf(mn1, f.y); mx1 = fmaxf(mx1, f.y);
      }
    }
    if constexpr (GS > 32) {
      __shared__ float4 s_mm[4][64];
      s_mm[wq][cp] = float4{mn0, mx0, mn1, mx1};
      __syncthreads();
      constexpr int wpg = GS / 32;                                 // waves per group
      const int w0 = wq / wpg * wpg;
#pragma unroll
      for (int w = 0; w < wpg; ++w) {
        const float4 o = s_mm[w0 + w][cp];
        mn0 = fminf(mn0, o.x); mx0 = fmaxf(mx0, o.y);
        mn1 = fminf(mn1, o.z); mx1 = fmaxf(mx1, o.w);
      }
    }
    if (!live) return;
    uint32_t promoted = 0;
    if (mask)
      promoted = *(const uint16_t*)(mask + (int64_t)b * mask_stride_b + (int64_t)h * mask_stride_h +
                                    (int64_t)tile * mask_stride_tile + cp * 2);
    const GroupParams g0 = (promoted & 0xffu) ? group_params(mn0, mx0, qmax_promote, inv_qmax_promote)
                                              : group_params(mn0, mx0, qmax, inv_qmax);
    const GroupParams g1 = (promoted >> 8) ? group_params(mn1, mx1, qmax_promote, inv_qmax_promote)
                                           : group_params(mn1, mx1, qmax, inv_qmax);
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      const float2 f = __half22float2(*(const __half2*)&raw[i]);
      const __half2 o = __floats2half2_rn(fake_quant_one(f.x, g0), fake_quant_one(f.y, g1));
      *(uint32_t*)(base + (int64_t)i * stride_t + lane_off) = *(const uint32_t*)&o;
    }
  }
}

}  // namespace
}  // namespace kitty

using namespace kitty;

extern "C" int kitty_fake_quant(void* data, int64_t stride_b, int64_t stride_h, int64_t stride_t, int B, int H, int T,
                                int D, int t_offset, int n_tokens, int axis, int group_size, int bit,
                                const uint8_t* promote_mask, int64_t mask_stride_b, int64_t mask_stride_h,
                                int64_t mask_stride_tile, int promote_bit, void* stream) {
  KITTY_REQUIRE(data != nullptr, KITTY_E_NULL, "data is NULL");
  KITTY_REQUIRE(D == kD, KITTY_E_SHAPE, "kernels are built for head_dim 128, got D=%d", D);
  KITTY_REQUIRE(axis == 0 || axis == 1, KITTY_E_SHAPE, "axis must be 0 (groups along tokens) or 1 (along channels)");
  KITTY_REQUIRE(group_size == 32 || group_size == 64 || group_size == 128, KITTY_E_SHAPE,
                "group_size must be 32, 64 or 128, got %d", group_size);
  KITTY_REQUIRE(bit >= 1 && bit <= 8 && (!promote_mask || (promote_bit >= 1 && promote_bit <= 8)), KITTY_E_SHAPE,
                "bit widths must be in [1, 8], got %d / %d", bit, promote_bit);
  KITTY_REQUIRE(B >= 0 && H >= 1 && B <= 65535 && H <= 65535 && t_offset >= 0 && n_tokens >= 0 &&
                    (int64_t)t_offset + n_tokens <= (int64_t)T,
                KITTY_E_RANGE, "bad B=%d H=%d or tokens [%d, %d) outside the %d of the tensor", B, H, t_offset,
                t_offset + n_tokens, T);
  KITTY_REQUIRE(axis == 1 || n_tokens % group_size == 0, KITTY_E_RANGE,
                "%d tokens are not a whole number of groups of %d", n_tokens, group_size);
  KITTY_REQUIRE(axis == 0 || promote_mask == nullptr, KITTY_E_SHAPE, "the promote mask goes with groups along tokens");
  KITTY_REQUIRE(((uintptr_t)data % 16) == 0 && stride_b % 16 == 0 && stride_h % 16 == 0 && stride_t % 16 == 0 &&
                    stride_t >= D * 2,
                KITTY_E_ALIGN, "data needs a 16-byte aligned base and strides with D contiguous");
  KITTY_REQUIRE(!promote_mask || (((uintptr_t)promote_mask % 8) == 0 && mask_stride_b % 8 == 0 &&
                                  mask_stride_h % 8 == 0 && mask_stride_tile % 8 == 0),
                KITTY_E_ALIGN, "the promote mask needs 8-byte aligned rows");
  if (B == 0 || n_tokens == 0) return 0;
  const float qmax = (float)((1 << bit) - 1), qmax_p = (float)((1 << (promote_mask ? promote_bit : bit)) - 1);
  const dim3 grid((n_tokens + kPage - 1) / kPage, H, B), block(256);
  const uint8_t* m = axis == 0 ? promote_mask : nullptr;
#define KITTY_FQ_LAUNCH(AXIS, GS)                                                                                      \
  hipLaunchKernelGGL((fake_quant_kernel<AXIS, GS>), grid, block, 0, (hipStream_t)stream, (uint8_t*)data, stride_b,     \
                     stride_h, stride_t, t_offset, n_tokens, qmax, 1.0f / qmax, qmax_p, 1.0f / qmax_p, m,              \
                     mask_stride_b, mask_stride_h, mask_stride_tile)
  if (axis == 0) {
    if (group_size == 32) KITTY_FQ_LAUNCH(0, 32);
    else if (group_size == 64) KITTY_FQ_LAUNCH(0, 64);
    else KITTY_FQ_LAUNCH(0, 128);
  } else {
    if (group_size == 32) KITTY_FQ_LAUNCH(1, 32);
    else if (group_size == 64) KITTY_FQ_LAUNCH(1, 64);
    else KITTY_FQ_LAUNCH(1, 128);
  }
#undef KITTY_FQ_LAUNCH
  return check_launch("kitty_fake_quant");
}
