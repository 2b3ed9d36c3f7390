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
#include "half_ops.h"

// a * b + c below is a product rounded to fp16 and then a sum rounded to fp16, as the reference's two
// operators are: no fused multiply-add.
#pragma clang fp contract(off)

namespace kitty {
namespace {

// fp16 results computed "in fp32, then rounded" equal the native fp16 operation for +, - and *: the
// exact result of two 11-bit operands rounded first to 24 bits and then to 11 bits is the exact result
// rounded to 11 bits (24 >= 2 * 11 + 2), and sums and products that are subnormal in fp16 are exact in
// fp32.  So x - mn, q * scale and . + mn are packed fp16 instructions on two elements at once, clamp
// and rint work on fp16 directly (rint as + 1024 - 1024: the codes are at most 255 and fp16 numbers
// from 1024 up are whole), and only the quotient takes fp32 arithmetic.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// the tensor is read once and written once: non-temporal both ways
__device__ __forceinline__ uint4 nt_load16(const uint8_t* p) {
  const u32x4 v = __builtin_nontemporal_load((const u32x4*)p);
  return uint4{v.x, v.y, v.z, v.w};
}
__device__ __forceinline__ half2_t as_h2(uint32_t w) { return __builtin_bit_cast(half2_t, w); }
__device__ __forceinline__ uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ uint32_t pack_h2(float lo, float hi) {       // both representable in fp16
  return as_u32(half2_t{(_Float16)lo, (_Float16)hi});
}

__device__ __forceinline__ float hr(float v) { return (float)(_Float16)v; }

struct GroupParams { float mn, scale, rscale, qmax; };

__device__ __forceinline__ GroupParams group_params(float mn, float mx, float qmax, float inv_qmax) {
  float rng = hr(mx - mn);
  rng = hr(fmaxf(rng, 1e-4f));
  const float scale = hr(rng * inv_qmax);
  return GroupParams{mn, scale, __frcp_rn(scale), qmax};
}

// The parameters of the two groups that the halves of a data word belong to
struct PairParams {
  uint32_t mn2, scale2, qmax2;          // packed fp16
  float r0, r1, scale0, scale1;         // 1 / scale and scale of the low and the high half
};
__device__ __forceinline__ PairParams pair_params(const GroupParams& g0, const GroupParams& g1) {
  return PairParams{pack_h2(g0.mn, g1.mn), pack_h2(g0.scale, g1.scale), pack_h2(g0.qmax, g1.qmax),
                    g0.rscale, g1.rscale, g0.scale, g1.scale};
}

// The quotient (x - mn) / scale is needed rounded to fp32 and then to fp16.  d * (1 / scale) is
// within 3 ulp of the fp32 quotient, so both round to the same fp16 number unless the product
// lies within 4 ulp of the midpoint of two fp16 numbers (the 13 bits fp16 drops read 0x1000 +- 4):
// a wave with such a lane (one in twenty) divides.  Outside fp16's normal range more bits are dropped
// or the rounding overflows, but there both quotients give the same code: below 6.1e-5 both round
// far below one half, from 65504 up both clamp to qmax.
__device__ __forceinline__ bool near_tie(float q) { return (__float_as_uint(q) & 0x1fffu) - 0x0ffcu <= 8u; }

__device__ __forceinline__ uint32_t fake_quant_pair(uint32_t w, const PairParams& p) {
  const half2_t d = as_h2(w) - as_h2(p.mn2);
  const uint32_t dw = as_u32(d);
  float q0 = mul_f16_f32(dw, 0, p.r0), q1 = mul_f16_f32(dw, 1, p.r1);
  if (__builtin_expect(__any(near_tie(q0) || near_tie(q1)), 0)) {
    q0 = __fdiv_rn((float)d.x, p.scale0);
    q1 = __fdiv_rn((float)d.y, p.scale1);
  }
  typedef float float2_t __attribute__((ext_vector_type(2)));
  half2_t h = __builtin_convertvector(float2_t{q0, q1}, half2_t);
  // the quotient of two non-negative numbers needs no lower clamp
  h = as_h2(pk_min_f16(as_u32(h), p.qmax2));
  const half2_t whole = {(_Float16)1024.f, (_Float16)1024.f};
  h = (h + whole) - whole;
  return as_u32(h * as_h2(p.scale2) + as_h2(p.mn2));
}

// Minimum in the low half and negated maximum in the high half of one word, from packed minima and
// maxima of pairs: one packed minimum then folds both across lanes.
__device__ __forceinline__ uint32_t fold_min_negmax(uint32_t mnw, uint32_t mxw) {
  const uint32_t nmx = mxw ^ 0x80008000u;
  return pk_min_f16(__builtin_amdgcn_perm(nmx, mnw, 0x05040100u),    // (mnw.lo, nmx.lo)
                    __builtin_amdgcn_perm(nmx, mnw, 0x07060302u));   // (mnw.hi, nmx.hi)
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
      raw[r] = tok < n_here ? nt_load16(base + (int64_t)tok * stride_t) : uint4{0, 0, 0, 0};
    }
    // one token row = 16 lanes; a group = GS / 8 neighbouring lanes
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const uint32_t w[4] = {raw[r].x, raw[r].y, raw[r].z, raw[r].w};
      uint32_t m = fold_min_negmax(pk_min_f16(pk_min_f16(w[0], w[1]), pk_min_f16(w[2], w[3])),
                                   pk_max_f16(pk_max_f16(w[0], w[1]), pk_max_f16(w[2], w[3])));
      // lanes l ^ 1, l ^ 2, then 7 - l of 8 and 15 - l of 16 (whose smaller blocks agree by then)
      m = pk_min_f16(m, (uint32_t)__builtin_amdgcn_mov_dpp((int)m, 0xB1 /* quad_perm [1,0,3,2] */, 0xf, 0xf, true));
      m = pk_min_f16(m, (uint32_t)__builtin_amdgcn_mov_dpp((int)m, 0x4E /* quad_perm [2,3,0,1] */, 0xf, 0xf, true));
      if constexpr (GS >= 64)
        m = pk_min_f16(m, (uint32_t)__builtin_amdgcn_mov_dpp((int)m, 0x141 /* row_half_mirror */, 0xf, 0xf, true));
      if constexpr (GS >= 128)
        m = pk_min_f16(m, (uint32_t)__builtin_amdgcn_mov_dpp((int)m, 0x140 /* row_mirror */, 0xf, 0xf, true));
      const GroupParams g = group_params(widen_f16(m, 0), -widen_f16(m, 1), qmax, inv_qmax);
      const PairParams p = pair_params(g, g);
      const int tok = r * 16 + tg;
      if (tok < n_here)
        __builtin_nontemporal_store(
            u32x4{fake_quant_pair(w[0], p), fake_quant_pair(w[1], p), fake_quant_pair(w[2], p), fake_quant_pair(w[3], p)},
            (u32x4*)(base + (int64_t)tok * stride_t));
    }
  } else {
    // channels 2cp, 2cp+1; tokens 32wq .. 32wq+31 (wq = the wave's number, uniform)
    const int cp = threadIdx.x & 63, wq = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool live = wq * 32 < n_here;                            // n_tokens is a multiple of GS >= 32
    uint8_t* base = tile_base + (int64_t)(wq * 32) * stride_t;
    const uint32_t lane_off = cp * 4;
    uint32_t raw[32];
    // minima and maxima of the two channels, packed; a wave without tokens takes no part in a group
    // (its +inf / -inf leave the others' as they are)
    uint32_t mn2 = 0x7c007c00u, mx2 = 0xfc00fc00u;
    if (live) {
#pragma unroll
      for (int i = 0; i < 32; ++i) raw[i] = __builtin_nontemporal_load((const uint32_t*)(base + (int64_t)i * stride_t + lane_off));
#pragma unroll
      for (int i = 0; i < 32; ++i) {
        mn2 = pk_min_f16(mn2, raw[i]);
        mx2 = pk_max_f16(mx2, raw[i]);
      }
    }
    if constexpr (GS > 32) {
      __shared__ uint2 s_mm[4][64];
      s_mm[wq][cp] = uint2{mn2, mx2};
      __syncthreads();
      constexpr int wpg = GS / 32;                                 // waves per group
      const int w0 = wq / wpg * wpg;
#pragma unroll
      for (int w = 0; w < wpg; ++w) {
        const uint2 o = s_mm[w0 + w][cp];
        mn2 = pk_min_f16(mn2, o.x);
        mx2 = pk_max_f16(mx2, o.y);
      }
    }
    if (!live) return;
    uint32_t promoted = 0;
    if (mask)
      promoted = *(const uint16_t*)(mask + (int64_t)b * mask_stride_b + (int64_t)h * mask_stride_h +
                                    (int64_t)tile * mask_stride_tile + cp * 2);
    const float mn0 = widen_f16(mn2, 0), mx0 = widen_f16(mx2, 0), mn1 = widen_f16(mn2, 1), mx1 = widen_f16(mx2, 1);
    const GroupParams g0 = (promoted & 0xffu) ? group_params(mn0, mx0, qmax_promote, inv_qmax_promote)
                                              : group_params(mn0, mx0, qmax, inv_qmax);
    const GroupParams g1 = (promoted >> 8) ? group_params(mn1, mx1, qmax_promote, inv_qmax_promote)
                                           : group_params(mn1, mx1, qmax, inv_qmax);
    const PairParams p = pair_params(g0, g1);
#pragma unroll
    for (int i = 0; i < 32; ++i)
      __builtin_nontemporal_store(fake_quant_pair(raw[i], p), (uint32_t*)(base + (int64_t)i * stride_t + lane_off));
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
