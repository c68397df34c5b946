// Benchmark-only library (libbench_calib.so), not part of the product ABI: nothing in the MoE path calls it.
// Calibration kernels: what the machine delivers with no memory system in the way (a register-only MFMA loop,
// with operands that stay constant or change every instruction) and with nothing but the memory system (a plain
// streaming read).  The benchmark reports them beside the roofline fractions of the real kernels, whose peaks are
// the published ones.

#include "moe_common.h"

namespace moe {

constexpr int kCalibAcc = 16;   // independent accumulators per wave: back-to-back MFMAs without dependency stalls
constexpr int kCalibFrag = 8;   // operand fragments per wave that the loop rotates through

// The 16 x 16 instructions of the GEMM kernels (16x16x64 i8, 16x16x32 bf16).  CHANGING: every MFMA takes another pair
// of the 8 + 8 fragments a lane holds (random bits, drawn before the loop: no VALU work inside it), so the operand
// buses toggle as they do on real data; otherwise all fragments are equal.  BF16: the random bits are confined to sign
// and mantissa of values in +-[0.5, 1).
template <bool BF16, bool CHANGING>
__global__ __launch_bounds__(256) void calib_mfma_kernel(int iters, int seed, int* __restrict__ sink) {
  unsigned s = seed * 7919u + threadIdx.x * 104729u + blockIdx.x * 1299709u;
  v4i fa[kCalibFrag], fb[kCalibFrag];
#pragma unroll
  for (int i = 0; i < kCalibFrag; i++)
#pragma unroll
    for (int c = 0; c < 4; c++) {
      unsigned x = 0x01010101u, y = 0x01010101u;
      if (CHANGING) {
        s = s * 1664525u + 1013904223u; x = s ^ (s >> 15);
        s = s * 1664525u + 1013904223u; y = s ^ (s >> 15);
      }
      if (BF16) { x = (x & 0x807f807fu) | 0x3f003f00u; y = (y & 0x807f807fu) | 0x3f003f00u; }
      fa[i][c] = x; fb[i][c] = y;
    }
  typedef typename std::conditional<BF16, v4f, v4i>::type acc_t;
  acc_t acc[kCalibAcc];
#pragma unroll
  for (int i = 0; i < kCalibAcc; i++)
#pragma unroll
    for (int r = 0; r < 4; r++) acc[i][r] = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < kCalibAcc; i++) {
      const int ia = i % kCalibFrag, ib = (i / 2 + 3 * (i & 1)) % kCalibFrag;
      if constexpr (BF16) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, fa[ia]), __builtin_bit_cast(v8bf, fb[ib]), acc[i], 0, 0, 0);
      else acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[ia], fb[ib], acc[i], 0, 0, 0);
    }
  }
  int sum = 0;
#pragma unroll
  for (int i = 0; i < kCalibAcc; i++)
#pragma unroll
    for (int r = 0; r < 4; r++) sum += (int)acc[i][r];
  sink[blockIdx.x * 256 + threadIdx.x] = sum;
}

// every wave reads 8 KB per step with non-temporal requests of 1 KB (whole 128-byte lines: the request shape that
// streams fastest on this part), the grid strides over the buffer once
__global__ __launch_bounds__(256) void calib_read_kernel(const v4i* __restrict__ src, size_t nvec, int* __restrict__ sink) {
  constexpr int U = 8;
  const size_t stride = (size_t)gridDim.x * 256 * U;
  v4i s = {0, 0, 0, 0};
  for (size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x / kWave * kWave) * U + threadIdx.x % kWave; i + (U - 1) * kWave < nvec; i += stride) {
    v4i v[U];
#pragma unroll
    for (int j = 0; j < U; j++) v[j] = __builtin_nontemporal_load(src + i + j * kWave);
#pragma unroll
    for (int j = 0; j < U; j++) s ^= v[j];
  }
  if ((s[0] ^ s[1] ^ s[2] ^ s[3]) == 0x12345678) sink[0] = 1;
}

constexpr int kCalibBlocks = 256 * 8;  // 2 waves per SIMD on 256 CUs

}  // namespace moe

using namespace moe;

extern "C" {

// Every function returns 0 or a hipError_t value; the caller times the launches.
#define CALIB_API __attribute__((visibility("default")))

CALIB_API size_t calib_scratch_bytes(void) { return (size_t)kCalibBlocks * 256 * sizeof(int); }

CALIB_API double calib_mfma_ops(int dtype, int iters) {
  const double per_mfma = dtype == MOE_INT8 ? 2.0 * 16 * 16 * 64 : 2.0 * 16 * 16 * 32;
  return (double)kCalibBlocks * 4 * (double)iters * kCalibAcc * per_mfma;
}

CALIB_API int calib_mfma(int dtype, int random_operands, int iters, void* scratch, void* stream) {
  if (!scratch || iters <= 0) return (int)hipErrorInvalidValue;
  hipStream_t s = (hipStream_t)stream;
  int* sink = (int*)scratch;
  if (dtype == MOE_INT8) {
    if (random_operands) calib_mfma_kernel<false, true><<<kCalibBlocks, 256, 0, s>>>(iters, 12345, sink);
    else calib_mfma_kernel<false, false><<<kCalibBlocks, 256, 0, s>>>(iters, 12345, sink);
  } else if (dtype == MOE_BF16) {
    if (random_operands) calib_mfma_kernel<true, true><<<kCalibBlocks, 256, 0, s>>>(iters, 12345, sink);
    else calib_mfma_kernel<true, false><<<kCalibBlocks, 256, 0, s>>>(iters, 12345, sink);
  } else {
    return (int)hipErrorInvalidValue;
  }
  return (int)hipGetLastError();
}

CALIB_API int calib_read(const void* src, size_t bytes, void* scratch, void* stream) {
  if (!src || !scratch || bytes < 65536 || ((uintptr_t)src & 15)) return (int)hipErrorInvalidValue;
  calib_read_kernel<<<kCalibBlocks, 256, 0, (hipStream_t)stream>>>((const v4i*)src, bytes / 16, (int*)scratch);
  return (int)hipGetLastError();
}

}  // extern "C"
