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
// A tile is 128 tokens x 128 channels of one (batch row, head): 256 threads, each owning 8 channels
// (16 bytes) of the 8 tokens r*16 + tg, so that a wave's load covers four consecutive token rows.
// AXIS 0: groups run along the tokens (keys: one channel over group_size tokens; the reference
// transposes K to [B, nh, D, T] for this, kitty_simulate.py:204-207), optional promote mask per
// channel.  AXIS 1: groups run along the channels (values: one token over group_size channels).
#include "kitty_common.h"

namespace kitty {
namespace {

__device__ __forceinline__ float hr(float v) { return __half2float(__float2half_rn(v)); }

struct GroupParams { float mn, scale, qmax; };

__device__ __forceinline__ GroupParams group_params(float mn, float mx, float qmax, float inv_qmax) {
  float rng = hr(mx - mn);
  rng = hr(fmaxf(rng, 1e-4f));
  return GroupParams{mn, hr(rng * inv_qmax), qmax};
}

__device__ __forceinline__ float fake_quant_one(float x, const GroupParams& g) {
  float q = hr(__fdiv_rn(hr(x - g.mn), g.scale));
  q = rintf(fminf(fmaxf(q, 0.f), g.qmax));
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

template <int AXIS>
__global__ __launch_bounds__(256) void fake_quant_kernel(uint8_t* __restrict__ data, int64_t stride_b, int64_t stride_h,
                                                         int64_t stride_t, int t_offset, int n_tokens, int group_size,
                                                         float qmax, float inv_qmax, float qmax_promote,
                                                         float inv_qmax_promote, const uint8_t* __restrict__ mask,
                                                         int64_t mask_stride_b, int64_t mask_stride_h,
                                                         int64_t mask_stride_tile) {
  const int tile = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int cg = threadIdx.x & 15, tg = threadIdx.x >> 4;
  const int n_here = min(kPage, n_tokens - tile * kPage);
  uint8_t* base = data + (int64_t)b * stride_b + (int64_t)h * stride_h +
                  (int64_t)(t_offset + tile * kPage) * stride_t + cg * 16;
  uint4 raw[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int tok = r * 16 + tg;
    raw[r] = tok < n_here ? *(const uint4*)(base + (int64_t)tok * stride_t) : uint4{0, 0, 0, 0};
  }

  if constexpr (AXIS == 1) {
    // one token row = 16 lanes; a group = group_size / 8 neighbouring lanes
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      float x[8];
      unpack8(raw[r], x);
      float mn = x[0], mx = x[0];
#pragma unroll
      for (int j = 1; j < 8; ++j) { mn = fminf(mn, x[j]); mx = fmaxf(mx, x[j]); }
      for (int o = 1; o * 8 < group_size; o <<= 1) {
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
    // a group = group_size consecutive tokens of one channel = rows r in [g * rpg, (g + 1) * rpg) of all 16 tg
    __shared__ float s_mn[4][4][kD], s_mx[4][4][kD];     // [group][wave][channel]
    const int rpg = group_size / 16, n_groups = kPage / group_size;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int g = 0; g < n_groups; ++g) {
      float mn[8], mx[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) { mn[j] = INFINITY; mx[j] = -INFINITY; }
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        if (r / rpg != g || r * 16 + tg >= n_here) continue;
        float x[8];
        unpack8(raw[r], x);
#pragma unroll
        for (int j = 0; j < 8; ++j) { mn[j] = fminf(mn[j], x[j]); mx[j] = fmaxf(mx[j], x[j]); }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        mn[j] = fminf(mn[j], __shfl_xor(mn[j], 16));
        mx[j] = fmaxf(mx[j], __shfl_xor(mx[j], 16));
        mn[j] = fminf(mn[j], __shfl_xor(mn[j], 32));
        mx[j] = fmaxf(mx[j], __shfl_xor(mx[j], 32));
      }
      if (lane < 16) {
#pragma unroll
        for (int j = 0; j < 8; ++j) { s_mn[g][wave][cg * 8 + j] = mn[j]; s_mx[g][wave][cg * 8 + j] = mx[j]; }
      }
    }
    __syncthreads();
    uint8_t promoted[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) promoted[j] = 0;
    if (mask) {
      const uint2 m = *(const uint2*)(mask + (int64_t)b * mask_stride_b + (int64_t)h * mask_stride_h +
                                      (int64_t)tile * mask_stride_tile + cg * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) promoted[j] = ((j < 4 ? m.x >> (8 * j) : m.y >> (8 * (j - 4))) & 0xff) != 0;
    }
    for (int g = 0; g < n_groups; ++g) {
      if (g * group_size >= n_here) break;      // n_tokens is a multiple of group_size: a group is whole or absent
      GroupParams gp[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int c = cg * 8 + j;
        const float mn = fminf(fminf(s_mn[g][0][c], s_mn[g][1][c]), fminf(s_mn[g][2][c], s_mn[g][3][c]));
        const float mx = fmaxf(fmaxf(s_mx[g][0][c], s_mx[g][1][c]), fmaxf(s_mx[g][2][c], s_mx[g][3][c]));
        gp[j] = promoted[j] ? group_params(mn, mx, qmax_promote, inv_qmax_promote) : group_params(mn, mx, qmax, inv_qmax);
      }
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        if (r / rpg != g) continue;
        float x[8];
        unpack8(raw[r], x);
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = fake_quant_one(x[j], gp[j]);
        *(uint4*)(base + (int64_t)(r * 16 + tg) * stride_t) = pack8(x);
      }
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
  if (axis == 0)
    hipLaunchKernelGGL(fake_quant_kernel<0>, grid, block, 0, (hipStream_t)stream, (uint8_t*)data, stride_b, stride_h,
                       stride_t, t_offset, n_tokens, group_size, qmax, 1.0f / qmax, qmax_p, 1.0f / qmax_p, promote_mask,
                       mask_stride_b, mask_stride_h, mask_stride_tile);
  else
    hipLaunchKernelGGL(fake_quant_kernel<1>, grid, block, 0, (hipStream_t)stream, (uint8_t*)data, stride_b, stride_h,
                       stride_t, t_offset, n_tokens, group_size, qmax, 1.0f / qmax, qmax_p, 1.0f / qmax_p, nullptr, 0, 0,
                       0);
  return check_launch("kitty_fake_quant");
}
