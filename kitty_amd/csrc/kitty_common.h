// Shared host/device helpers for the gfx950 kernels of the quantized-KV path.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/kitty_hip.h"

namespace kitty {

// Geometry the kernels are specialised for (the only one the reference uses: kitty.py:43-47).
constexpr int kD = 128;        // head_dim
constexpr int kPage = 128;     // tokens per page == quantization group
constexpr int kRowBytes = 32;  // one 2-bit plane row: 128 codes
constexpr int kLoBytes = kD * kRowBytes;                 // 4096: low plane of a K page-head
constexpr int kVBytes = kPage * kRowBytes;               // 4096: a V page-head

__host__ __device__ inline int k_head_bytes(int d_boost) { return kRowBytes * (kD + d_boost) + kD; }
// Other head dimensions (the reference derives everything from config.head_dim, kitty.py:39-44, and its
// kernels take D as a parameter, kitty_quant_pack.py:42-45, kitty_attention.py:59-62): 64 and 256 run
// on plain kernels of their own (any_dim.hip); the tuned kernels are those for 128.
__host__ __device__ inline bool head_dim_supported(int d) { return d == 64 || d == kD || d == 256; }
__host__ __device__ inline int k_head_bytes_d(int head_dim, int d_boost) {
  return kRowBytes * (head_dim + d_boost) + head_dim;
}
__host__ __device__ inline int v_head_bytes_d(int head_dim) { return kPage * head_dim / 4; }

// v_max_f32 / v_max3_f32 as single instructions.  In front of fmaxf the compiler puts a NaN-quieting
// `v_max_f32 x, x, x` for every operand it cannot prove canonical (anything that crosses a basic
// block), which doubles the cost of a reduction.  The hardware instruction already returns the
// other operand when one is a NaN, like fmaxf.
__device__ __forceinline__ float vmax(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float vmax3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

int set_error(int code, const char* fmt, ...);
int check_launch(const char* what);

}  // namespace kitty

#define KITTY_REQUIRE(cond, code, ...) \
  do { if (!(cond)) return kitty::set_error((code), __VA_ARGS__); } while (0)
