// Shared device/host helpers for the gfx950 kernels: bf16 bit handling, MFMA operand types,
// error plumbing of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdexcept>
#include <string>

typedef uint16_t bf16_t; // raw bf16 bits in memory
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
// native vectors for 16/8-byte memory accesses (HIP's uint4/uint2 structs copy through memcpy,
// which keeps register arrays of them in scratch memory)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define TG_DEVICE __device__ __forceinline__

TG_DEVICE float bf16_to_float(bf16_t b) {
    return __uint_as_float(uint32_t(b) << 16);
}
// round to nearest even (v_cvt_pk_bf16_f32 on gfx950)
TG_DEVICE bf16_t float_to_bf16(float f) {
    return __builtin_bit_cast(uint16_t, (__bf16)f);
}
// both halves in one v_cvt_pk_bf16_f32
TG_DEVICE uint32_t pack_bf16(float lo, float hi) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const f32x2 pair = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
}
TG_DEVICE float bf16_lo(uint32_t pair) {
    return __uint_as_float(pair << 16);
}
TG_DEVICE float bf16_hi(uint32_t pair) {
    return __uint_as_float(pair & 0xffff0000u);
}
TG_DEVICE float round_bf16(float f) {
    return bf16_to_float(float_to_bf16(f));
}
// GELU with the exact-erf definition and its derivative.  erf is evaluated with Abramowitz-Stegun
// 7.1.26 (|error| <= 1.5e-7, far below bf16 resolution): one reciprocal, one exp2 and a degree-5
// Horner chain, branch free.  gelu'(x) = Phi(x) + x phi(x) shares the exponential, because
// erf(x/sqrt2) needs exp(-x^2/2) and so does phi.  Constants are folded so that one element costs 13
// instructions forward: the epilogues that call this are bound by their instruction count.
struct GeluParts {
    float tail; // 0.5 erfc(|x| / sqrt 2) = Phi(-|x|)
    float e;    // exp(-x^2 / 2)
};
TG_DEVICE GeluParts gelu_parts(float x) {
    const float t = __builtin_amdgcn_rcpf(fmaf(fabsf(x), 0.3275911f * 0.70710678118654752f, 1.0f));
    const float s = x * 0.84932180028801905f; // s^2 = x^2 / (2 ln 2)
    const float e = __builtin_amdgcn_exp2f(-(s * s));
    float poly = fmaf(0.5f * 1.061405429f, t, 0.5f * -1.453152027f);
    poly = fmaf(poly, t, 0.5f * 1.421413741f);
    poly = fmaf(poly, t, 0.5f * -0.284496736f);
    poly = fmaf(poly, t, 0.5f * 0.254829592f);
    return {poly * t * e, e};
}
TG_DEVICE float gelu_f(float x) {
    // x Phi(x) = max(x, 0) - |x| Phi(-|x|)
    float positive; // fmaxf would add a canonicalising v_max x, x in front
    asm("v_max_f32 %0, 0, %1" : "=v"(positive) : "v"(x));
    return fmaf(-fabsf(x), gelu_parts(x).tail, positive);
}
TG_DEVICE float gelu_grad_f(float x) {
    const GeluParts g = gelu_parts(x);
    const float cdf = x < 0.f ? g.tail : 1.0f - g.tail;
    return fmaf(x * g.e, 0.39894228040143268f, cdf);
}
TG_DEVICE float wave_sum(float x) {
#pragma unroll
    for (int k = 32; k; k >>= 1)
        x += __shfl_xor(x, k, 64);
    return x;
}
TG_DEVICE float wave_max(float x) {
#pragma unroll
    for (int k = 32; k; k >>= 1)
        x = fmaxf(x, __shfl_xor(x, k, 64));
    return x;
}

// One wave-wide global -> LDS copy of 16 bytes per lane (global_load_lds_dwordx4): lane l lands at
// LDS byte address lds_base + 16*l, lds_base wave-uniform.  The compiler does not track these copies;
// completion is awaited explicitly with wait_vmcnt<N>() ("at most N of this wave's vector-memory
// operations still outstanding") before the barrier that publishes the data to the other waves.
TG_DEVICE void async_copy16(uint32_t lds_base, const void *global) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(global) : "memory");
}
// the same copy from a wave-uniform base plus a 32-bit byte offset per lane: one address register instead of two
TG_DEVICE void async_copy16(uint32_t lds_base, const void *uniform_base, uint32_t lane_offset) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(lane_offset), "s"(uniform_base)
                 : "memory");
}
// the 4-byte form: lane l lands at lds_base + 4*l
TG_DEVICE void async_copy4(uint32_t lds_base, const void *global) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_base), "v"(global) : "memory");
}
template <int N> TG_DEVICE void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
TG_DEVICE uint32_t lds_address(const void *shared_pointer) {
    return uint32_t(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void *)shared_pointer));
}

// ---- host side ---------------------------------------------------------------------------
extern thread_local std::string tg_last_error;

inline void check_hip(hipError_t error, const char *what = "") {
    if (error != hipSuccess)
        throw std::runtime_error(std::string(what) + hipGetErrorString(error));
}
inline void require(bool ok, const char *message) {
    if (!ok)
        throw std::invalid_argument(message);
}
// Every C entry point is `return guarded([&]{ ... });` : 0 on success, -1 with the message
// kept for tg_error()/tgk_error(); no exception crosses the ABI.
template <class F> inline int guarded(F &&body) {
    try {
        body();
        return 0;
    } catch (const std::exception &error) {
        tg_last_error = error.what();
        return -1;
    }
}
