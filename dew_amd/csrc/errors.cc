// Error string plumbing and introspection strings.
#include <stdarg.h>
#include <string.h>

#include "common.h"

namespace dew {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, args);
  va_end(args);
}

int fail(int code, const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, args);
  va_end(args);
  return code;
}

int launched(const char* kernel) {
  hipError_t status = hipGetLastError();
  if (status == hipSuccess) return DEW_MOE_OK;
  return fail(DEW_MOE_ELAUNCH, "%s: %s", kernel, hipGetErrorString(status));
}

}  // namespace dew

extern "C" {

const char* dew_moe_last_error(void) { return dew::g_error; }

const char* dew_moe_architecture(void) { return "gfx950"; }

const char* dew_moe_kernel_fields(void) { return "name,tile_m,tile_n,tile_k,waves,mfma,operands"; }

const char* dew_moe_kernels(void) {
  return "route,1 token/wave,-,-,4,-,f32 logits\n"
         "permute_small|permute_count+scan+scatter,2048 slots/block,-,-,4,-,i32 ballot+LDS histogram\n"
         "grouped_gemm<large>,256,256 (paired 2x128),64,4 (1x4),v_mfma_f32_32x32x16_bf16,bf16 rows via global_load_lds x nvfp4|mxfp4 fragments from global; 1 block/CU\n"
         "grouped_gemm<medium>,128,256 (paired 2x128) | 128,64,4 (1x4),v_mfma_f32_32x32x16_bf16,bf16 x {fp8 block|fp8 channel|nvfp4|mxfp4}; 2 blocks/CU\n"
         "grouped_gemm<decode>,32,128 (paired 2x128),64,4 (1x4),v_mfma_f32_32x32x16_bf16,weight streaming for groups under 24 rows\n"
         "grouped_gemm epilogues,-,-,-,-,-,plain (+bias) | swiglu of two banks | interleaved gate/up clamped 1.702 gating (+bias); tile staged in LDS and stored as whole rows\n"
         "grouped_gemm<split rows>,128 (paired; 2 blocks/CU) | 256,256 (paired 2x128),64,4 (2x2),v_mfma_scale_f32_32x32x64_f8f6f4,two e4m3 terms per bf16 activation x mxfp4 codes as stored; SwiGLU rows written already split\n"
         "grouped_gemm<split rows; fp6 second term>,128,256 (paired 2x128),64,4 (2x2),v_mfma_scale_f32_32x32x64_f8f6f4,an e4m3 term and an e2m3 term under one e8m0 scale per 32 depths x mxfp4 codes: opt-in; three quarters of the issue time\n"
         "grouped_gemm<fp8 rows>,256,256 | 128,128,4 (2x2),v_mfma_scale_f32_32x32x64_f8f6f4,e4m3 rows (1x128 power-of-two scales) x fp8 128x128 blocks (power-of-two scales)\n"
         "grouped_gemm<mxfp8 rows>,256,256,128,4 (2x2),v_mfma_scale_f32_32x32x64_f8f6f4,OCP MXFP8 rows x MXFP8 bank: e4m3 codes and E8M0 scales per 32 depths of both operands as stored\n"
         "split_rows | split_rows_fp6 | quantize_rows_fp8 | quantize_rows_mxfp8,1 row/wave,-,-,4,-,bf16 rows -> e4m3 terms (or e4m3 + e2m3) | e4m3 codes in operand order + e8m0 scales\n"
         "grouped_gemm<bf16>,32|64|128|256,128|256,64,3,v_mfma_f32_32x32x16_bf16,unquantized bf16 matrices as fragment atoms: no dequantization\n"
         "grouped_gemm<mxfp8 window>,256,256 | 128,128,4 (2x2),v_mfma_scale_f32_32x32x64_f8f6f4,a kernel gradient: each group's window of 128-token steps of lhs_t rows x the rhs_t bank; bf16 or fp32 out\n"
         "grouped_gemm<bf16 window>,256,256 | 128,64,3,v_mfma_f32_32x32x16_bf16,gemm_t: each group's window of 64-token steps of bf16 lhs_t rows x the bf16 rhs_t bank; tensor scales on the sums\n"
         "transpose_columns,128 tokens x 64 columns/block,-,-,4,-,bf16 [tokens x dim] transposed (or its NVFP4 values along the tokens): rows or bf16 bank atoms\n"
         "quantize_columns,128 tokens x 64 columns/block,-,-,4,-,bf16 [tokens x dim] -> e4m3 along the tokens and transposed: operand rows or bank atoms + e8m0 scales\n"
         "absmax + quantize_rows_nvfp4,1 row/wave,-,-,4,-,bf16 rows -> bf16 (e2m1 code x e4m3 scale) + the tensor scale\n"
         "combine,8 columns/lane,-,-,4,-,bf16 slots x f32 weights\n";
}

int dew_moe_device_check(void) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return dew::fail(DEW_MOE_EDEVICE, "no HIP device is current");
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) != hipSuccess)
    return dew::fail(DEW_MOE_EDEVICE, "hipGetDeviceProperties failed for device %d", device);
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return dew::fail(DEW_MOE_EDEVICE, "device %d is %s; these kernels are built for gfx950 only", device,
                     prop.gcnArchName);
  return DEW_MOE_OK;
}

}  // extern "C"
