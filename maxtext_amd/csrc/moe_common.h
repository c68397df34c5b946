// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "moe_mi355x.h"

namespace moe {

constexpr int kWave = 64;

// Records the message returned by moe_last_error() and yields `code`.
int fail(int code, const char* fmt, ...);
// Returns MOE_OK or records hipGetLastError() and yields MOE_ERR_LAUNCH.
int check_launch(const char* what);

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// Round-to-nearest-even f32 -> bf16 bits (NaN kept quiet).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

__device__ __forceinline__ float round_bf16_fn(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// Two f32 -> packed bf16 (round to nearest even) in one v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// 1 / (1 + 2^(-x log2 e)) on the hardware exp2 / rcp units (about 1 ulp each): five instructions.
__device__ __forceinline__ float sigmoidf_(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

// gate/up -> activation, computed in f32 (moe.py:841-870).  ACT is a compile-time moe_act so that the
// epilogues stay straight-line code.
template <int ACT>
__device__ __forceinline__ float glu_act(float g, float u, float limit) {
  if (ACT == MOE_ACT_SILU) return g * sigmoidf_(g) * u;
  if (ACT == MOE_ACT_SWIGLUOAI) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * sigmoidf_(1.702f * g) * (u + 1.0f);
  }
  if (ACT == MOE_ACT_SILU_CLIP) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * sigmoidf_(g) * u;
  }
  return g;
}

// Calls f(std::integral_constant<int, act>) with the runtime activation turned into a constant.
template <typename F>
__device__ __forceinline__ void dispatch_act(int act, F&& f) {
  if (act == MOE_ACT_SILU) f(std::integral_constant<int, MOE_ACT_SILU>{});
  else if (act == MOE_ACT_SWIGLUOAI) f(std::integral_constant<int, MOE_ACT_SWIGLUOAI>{});
  else if (act == MOE_ACT_SILU_CLIP) f(std::integral_constant<int, MOE_ACT_SILU_CLIP>{});
  else f(std::integral_constant<int, MOE_ACT_NONE>{});
}

inline int cdiv(int a, int b) { return (a + b - 1) / b; }

// Operands of global_load_lds (global -> LDS copy without staging registers).
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

// ds_read_b64_tr_b16, gfx950's transposing LDS load: within 16 lanes, lane L receives the L-th 16-bit column of a
// 4 x 16 block whose rows are addressed by lanes 0-3, 4-7, ... (8 bytes each).  Two such reads, 4 rows apart, give a
// lane the 8 contraction values of its channel that a 16 x 16 x 32 (or 32 x 32 x 16) bf16 MFMA fragment holds when the
// tile is stored with the contraction index as the ROW index.  p: the lane's 8 bytes of the first block.
typedef short v4s __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s* lds_v4s_t;
__device__ __forceinline__ v8bf tr_read_frag(const uint8_t* p, int row_stride) {
  const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t)p);
  const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t)(p + 4 * row_stride));
  typedef short v8s __attribute__((ext_vector_type(8)));
  const v8s v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(v8bf, v);
}

// Swizzle of unpadded 512-byte rows (256 bf16 channels) that are read that way: the 16-byte chunk q of row r is stored
// at slot q ^ tr_swz(r), so that the 4 rows x 32 bytes which 16 lanes address, and those of the next 16 lanes (8 rows
// further down), fall into 8 different 32-byte bank groups.  The permutation stays inside aligned 256 bytes of a row.
__device__ __forceinline__ int tr_swz(int row) { return ((row & 3) << 2) ^ (((row >> 3) & 1) << 1); }

// global -> LDS copy of 16 bytes per lane (1 KB per wave at lds_addr, a wave-uniform LDS byte address) written as asm.
// For kernels that use the transposing read: the compiler puts s_waitcnt vmcnt(0) before every such read that follows a
// copy it knows of, a full memory latency several times per stage.  Which buffer a copy writes and a read reads must
// then be settled by explicit vmcnt waits and barriers.
__device__ __forceinline__ void dma16_untracked(const void* src, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(lds_addr) : "memory", "m0");
}

// s_waitcnt with only vmcnt constrained (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[15:14]).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

}  // namespace moe
