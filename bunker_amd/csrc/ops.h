// Internal launcher declarations: one per kernel family.  All pointers are
// device pointers; every launcher validates its shapes on the host before it
// launches and enqueues on bk::stream().
#pragma once
#include "common.h"

namespace bk {

enum : int { DT_F32 = 0, DT_BF16 = 1 };

// runtime.hip
bool inited();
bool prof_on();
int prof_begin(int kernel);
int prof_end();

// quant.hip
int launch_quantize_q8_1(const void* x, int x_dtype, void* out, int K, int batch);
int launch_dequant_legacy_i8(const void* blocks, void* out, int64_t nblocks);
int launch_q4k_nibbles(const void* blocks, void* out, int64_t nblocks);
int launch_q4k_dequant_f32(const void* blocks, void* out, int64_t nblocks);

// gemv.hip
int launch_gemv_q4k_f32(const void* W, const float* x, float* y, int N, int K);
int launch_gemv_q4k_q8_1(const void* W, const void* xq, void* y, int N, int K, int batch,
                         int out_dtype, const void* residual);
int launch_q4k_q8_1_subdots(const void* W, const void* xq, int32_t* I, int N, int K);

}  // namespace bk
