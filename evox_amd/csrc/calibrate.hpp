// Issue-rate calibration kernels for the roofline of the dominance kernel: long runs of independent
// instructions of one kind, so that the measured rate is what the vector unit sustains for that kind
// on the device and at the clock of the moment.  Used by the benchmark only.
//   kind 0: v_add_f32 (result in a VGPR)
//   kind 1: v_cmp_le_f32 with the lane mask written to an SGPR pair (what every compare of the dominance
//           kernel is); v_addc_co_u32 with SGPR carries runs at the same rate
//   kind 2: the dominance kernel's unit for three objectives -- three v_cmp_le_f32, one v_cmp_ne_u32,
//           three s_and_b64, one v_addc_co_u32 -- twice, on two sets of SGPRs
//   kind 3: the unit of the arithmetic form for three objectives -- three v_sub_f32 with a scalar operand,
//           v_or3_b32, v_med3_i32, v_lshl_or_b32 -- twice
// Every iteration issues 16 VALU instructions for kinds 0 and 1, 10 for kind 2 and 12 for kind 3.
#pragma once

#include "common.hpp"

namespace evx {

template <int KIND>
__global__ __launch_bounds__(256) void calibrate_kernel(float* out, int iters, float a, float b) {
  float x = threadIdx.x * 0.001f + a, y = b, z0 = 0, z1 = 0, z2 = 0, z3 = 0;
  unsigned acc0 = 0, acc1 = 0;
#pragma unroll 1
  for (int it = 0; it < iters; ++it) {
    if (KIND == 0) {
      asm volatile(
          "v_add_f32 %0, %0, %4\n v_add_f32 %1, %1, %4\n v_add_f32 %2, %2, %4\n v_add_f32 %3, %3, %4\n"
          "v_add_f32 %0, %0, %4\n v_add_f32 %1, %1, %4\n v_add_f32 %2, %2, %4\n v_add_f32 %3, %3, %4\n"
          "v_add_f32 %0, %0, %4\n v_add_f32 %1, %1, %4\n v_add_f32 %2, %2, %4\n v_add_f32 %3, %3, %4\n"
          "v_add_f32 %0, %0, %4\n v_add_f32 %1, %1, %4\n v_add_f32 %2, %2, %4\n v_add_f32 %3, %3, %4\n"
          : "+v"(z0), "+v"(z1), "+v"(z2), "+v"(z3)
          : "v"(y));
    } else if (KIND == 1) {
      asm volatile(
          "v_cmp_le_f32_e64 s[20:21], %0, %1\n v_cmp_le_f32_e64 s[22:23], %1, %0\n v_cmp_le_f32_e64 s[24:25], %0, %1\n"
          "v_cmp_le_f32_e64 s[26:27], %1, %0\n v_cmp_le_f32_e64 s[28:29], %0, %1\n v_cmp_le_f32_e64 s[30:31], %1, %0\n"
          "v_cmp_le_f32_e64 s[32:33], %0, %1\n v_cmp_le_f32_e64 s[34:35], %1, %0\n v_cmp_le_f32_e64 s[20:21], %0, %1\n"
          "v_cmp_le_f32_e64 s[22:23], %1, %0\n v_cmp_le_f32_e64 s[24:25], %0, %1\n v_cmp_le_f32_e64 s[26:27], %1, %0\n"
          "v_cmp_le_f32_e64 s[28:29], %0, %1\n v_cmp_le_f32_e64 s[30:31], %1, %0\n v_cmp_le_f32_e64 s[32:33], %0, %1\n"
          "v_cmp_le_f32_e64 s[34:35], %1, %0\n"
          :
          : "v"(x), "v"(y)
          : "s20", "s21", "s22", "s23", "s24", "s25", "s26", "s27", "s28", "s29", "s30", "s31", "s32", "s33", "s34", "s35");
    } else if (KIND == 3) {
      asm volatile(
          "v_sub_f32 %2, %6, s20\n v_sub_f32 %3, %7, s21\n v_sub_f32 %4, %6, s22\n v_or3_b32 %2, %2, %3, %4\n"
          "v_med3_i32 %2, %2, 0, 1\n v_lshl_or_b32 %0, %0, 1, %2\n"
          "v_sub_f32 %5, %6, s23\n v_sub_f32 %3, %7, s24\n v_sub_f32 %4, %6, s25\n v_or3_b32 %5, %5, %3, %4\n"
          "v_med3_i32 %5, %5, 0, 1\n v_lshl_or_b32 %1, %1, 1, %5\n"
          : "+v"(acc0), "+v"(acc1), "=&v"(z0), "=&v"(z1), "=&v"(z2), "=&v"(z3)
          : "v"(x), "v"(y)
          : "s20", "s21", "s22", "s23", "s24", "s25");
    } else {
      // s_and_b64 writes SCC: declared, or the loop's own compare would be carried across this block
      asm volatile(
          "v_cmp_le_f32_e64 s[20:21], %2, %3\n v_cmp_le_f32_e64 s[22:23], %3, %2\n v_cmp_le_f32_e64 s[24:25], %2, %3\n"
          "v_cmp_ne_u32_e64 s[26:27], %0, %1\n"
          "s_and_b64 s[20:21], s[20:21], s[22:23]\n s_and_b64 s[24:25], s[24:25], s[26:27]\n"
          "s_and_b64 s[20:21], s[20:21], s[24:25]\n"
          "v_addc_co_u32_e64 %0, s[20:21], %0, %0, s[20:21]\n"
          "v_cmp_le_f32_e64 s[28:29], %2, %3\n v_cmp_le_f32_e64 s[30:31], %3, %2\n v_cmp_le_f32_e64 s[32:33], %2, %3\n"
          "v_cmp_ne_u32_e64 s[34:35], %0, %1\n"
          "s_and_b64 s[28:29], s[28:29], s[30:31]\n s_and_b64 s[32:33], s[32:33], s[34:35]\n"
          "s_and_b64 s[28:29], s[28:29], s[32:33]\n"
          "v_addc_co_u32_e64 %1, s[28:29], %1, %1, s[28:29]\n"
          : "+v"(acc0), "+v"(acc1)
          : "v"(x), "v"(y)
          : "scc", "s20", "s21", "s22", "s23", "s24", "s25", "s26", "s27", "s28", "s29", "s30", "s31", "s32", "s33", "s34",
            "s35");
    }
  }
  if (x + z0 + z1 + z2 + z3 + (float)acc0 + (float)acc1 == 12345.678f) out[0] = 1.0f;  // keeps the results alive
}

}  // namespace evx
