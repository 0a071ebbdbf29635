// Shared device/host helpers for the gfx950 Hyena kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/hyena_mi355x.h"

typedef unsigned short bf16_t;                                   // raw bfloat16 bits
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

// bf16 <-> fp32.  Widening is a shift; narrowing is round-to-nearest-even,
// the rounding torch applies when it casts float32 to bfloat16.
__device__ __forceinline__ float bf_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ float bf_to_f(bf16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;

// fp32 -> bf16 goes through the gfx950 conversion instruction (v_cvt_pk_bf16_f32, RNE).
__device__ __forceinline__ uint32_t pack_bf2(float lo, float hi) {
    const f32x2_t f = {lo, hi};
    union { bf16x2_t h; uint32_t u; } c;
    c.h = __builtin_convertvector(f, bf16x2_t);
    return c.u;
}
__device__ __forceinline__ uint32_t f_to_bf_bits(float f) { return pack_bf2(f, 0.f) & 0xffffu; }
__device__ __forceinline__ float round_bf(float f) { return __uint_as_float(pack_bf2(f, 0.f) << 16); }

struct RowMap {            // device copy of hyena_rows; channel arithmetic in 32 bits (64-bit division is emulated)
    const bf16_t* ptr;
    int64_t batch_stride, row_stride;
    uint32_t ch_inner, ch_outer;
    __device__ __forceinline__ const bf16_t* row(int64_t b, int64_t d) const {
        const uint32_t du = (uint32_t)d;
        const uint32_t r = (du < ch_inner) ? du : (du / ch_inner) * ch_outer + (du % ch_inner);
        return ptr + b * batch_stride + (int64_t)r * row_stride;
    }
};

static inline RowMap make_rowmap(const hyena_rows* r) {
    RowMap m;
    if (r) { m.ptr = (const bf16_t*)r->ptr; m.batch_stride = r->batch_stride; m.row_stride = r->row_stride;
             m.ch_inner = (uint32_t)r->ch_inner; m.ch_outer = (uint32_t)r->ch_outer; }
    else   { m.ptr = nullptr; m.batch_stride = m.row_stride = 0; m.ch_inner = m.ch_outer = 1; }
    return m;
}

// error reporting shared by all entry points (api.hip owns the buffer)
int hyena_fail(int code, const char* fmt, ...);
int hyena_check_launch(const char* what);

// launch-shape overrides set through hyena_set_launch_override (api.hip); -1 = the launcher's own choice
enum { HYENA_OV_MR_NSEG, HYENA_OV_CL_NSEG, HYENA_OV_SE_NT, HYENA_OV_MR_NT, HYENA_OV_LI_NT, HYENA_OV_CL_NT,
       HYENA_OV_LI_CPW, HYENA_OV_LI_COOP, HYENA_OV_LI_XCD, HYENA_OV_CL_NS, HYENA_OV_CL_F32_MFMA, HYENA_OV_COUNT };
int64_t hyena_override(int id);

// direct-form channel-last FIR for float16 / float32 tensors (fir_cl_direct.hip); arguments as hyena_fir_cl_fwd_dtype
int hyena_fir_cl_direct(const hyena_cl* x1, const hyena_cl* x2, const hyena_cl* v, const float* h, int taps_reversed,
                        const float* bias, int bias_mode, void* out, void* y2_out, void* bx_out, int64_t bx_from,
                        int64_t B, int64_t L, int64_t D, int64_t G, int K, int dtype, void* stream, const char* who);

// short-filter form of hyena_fir_layer_fwd_rows (se_fir.hip): 2 <= K <= 8, no inner bias, taps[g][K-1] on the current sample
int hyena_se_layer_rows(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const float* feat_taps,
                        const float* taps, void* out, int64_t B, int64_t D, int64_t L, int64_t G, int K, void* stream,
                        const char* who);

static inline bool rows_aligned8(const hyena_rows* r) {
    return r == nullptr || ((((uintptr_t)r->ptr) & 15) == 0 && r->batch_stride % 8 == 0 && r->row_stride % 8 == 0);
}
static inline bool rows_valid(const hyena_rows* r) {
    return r == nullptr || r->ptr == nullptr || (r->ch_inner > 0 && r->ch_inner < (1LL << 31) && r->ch_outer >= 0 &&
                            r->ch_outer < (1LL << 31));
}
