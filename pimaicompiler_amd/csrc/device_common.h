// Device-side helpers shared by the gfx950 kernels: fp16 vector types, fp32-accumulating
// dot products on v_dot2_f32_f16, and 64-lane wavefront reductions built on DPP.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pimhip
{
typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

static constexpr int kWave = 64;

// The bit pattern of a partial-sum record of the sliced I_X_W GEMV that has not arrived yet (gemv_kernels.h); host code
// fills the record buffers with it.
static constexpr unsigned int kVmEmpty = 0xffffffffu;

// acc += sum_{i<8} w[i] * x[i], products and sum in fp32.
__device__ __forceinline__ float dot8(const half8_t w, const half8_t x, float acc)
{
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(w, w, 0, 1), __builtin_shufflevector(x, x, 0, 1), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(w, w, 2, 3), __builtin_shufflevector(x, x, 2, 3), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(w, w, 4, 5), __builtin_shufflevector(x, x, 4, 5), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(w, w, 6, 7), __builtin_shufflevector(x, x, 6, 7), acc, false);
    return acc;
}

__device__ __forceinline__ float dot4(const half4_t w, const half4_t x, float acc)
{
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(w, w, 0, 1), __builtin_shufflevector(x, x, 0, 1), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(w, w, 2, 3), __builtin_shufflevector(x, x, 2, 3), acc, false);
    return acc;
}

// 16-byte streaming load of weight data that is read exactly once per launch.
__device__ __forceinline__ half8_t load_stream(const half8_t* p) { return __builtin_nontemporal_load(p); }

// The same with the choice of the cache policy.  Lines read with non-temporal loads are the first the caches drop, which
// is what a matrix far larger than the caches wants (the GEMV sweep's 134 MB shapes lose 7 % with plain loads: the lines
// they leave push out what other wavefronts still need).  The weights of a decoding loop are small and come round again
// every token, with other weights read in between: read with plain loads they stay in the caches (the XCDs' L2s and the
// 256 MB Infinity Cache behind them) until then.  Measured on MI355X, graph replays: one 1024 x 1024 matrix multiplied
// over and over 2.0 us either way; 64 such matrices in turn (134 MB) 2.43 us non-temporal, 2.19 us plain; 512 in turn
// (1 GB, more than the caches hold) 2.45 us either way; the three products of the mixture-of-experts step 7.3 -> 6.3 us.
static constexpr unsigned long long kKeepCachedBytes = 16ull << 20;  // the weights of a launch up to this size are read with plain loads
template <bool KEEP>
__device__ __forceinline__ half8_t load_weight(const half8_t* p)
{
    if constexpr (KEEP)
        return *p;
    else
        return __builtin_nontemporal_load(p);
}

// DPP controls (gfx9 encoding).
static constexpr int kDppQuadXor1 = 0xB1;     // quad_perm:[1,0,3,2]
static constexpr int kDppQuadXor2 = 0x4E;     // quad_perm:[2,3,0,1]
static constexpr int kDppRowHalfMirror = 0x141;
static constexpr int kDppRowMirror = 0x140;

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// Sum over the 64 lanes of a wavefront; every lane returns the total.
__device__ __forceinline__ float wave_sum(float v)
{
    v += dpp_f32<kDppQuadXor1>(v);
    v += dpp_f32<kDppQuadXor2>(v);
    v += dpp_f32<kDppRowHalfMirror>(v);
    v += dpp_f32<kDppRowMirror>(v);
    // The two steps across rows of 16 lanes: v_permlane16_swap a, b exchanges rows 1 and 3 of a with rows 0 and 2 of b,
    // v_permlane32_swap a, b the upper 32 lanes of a with the lower 32 of b; with a == b == v on entry, a + b is the
    // pairwise sum in every lane.  (No trip through the LDS crossbar, which the generic shuffle takes.)
    {
        float a = v, b = v;
        asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
        v = a + b;
    }
    {
        float a = v, b = v;
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
        v = a + b;
    }
    return v;
}

// The XCD a wavefront runs on: HW_REG_XCC_ID (hardware register 20), bits 3:0.  The probe that reports the placement of a
// launch and the kernel that relies on it read it through this one function.
static constexpr unsigned int kXccIdMask = 15u;
__device__ __forceinline__ unsigned int hw_xcc_id() { return __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & kXccIdMask; }

// Every bounded wait of the kernels here also ends after kWaitTicks of the constant 100 MHz clock, whatever its poll
// count: where a poll takes far longer than usual (counter collection serialising the memory system, a tool stepping the
// device), the poll limit alone bounds nothing useful.  Called every 256 unsuccessful polls; `t_first` keeps the time of
// the first such call.
static constexpr unsigned long long kWaitTicks = 100000000ull;  // one second
__device__ __forceinline__ bool wait_clock_expired(unsigned int spins, unsigned long long& t_first)
{
    const unsigned long long now = __builtin_amdgcn_s_memrealtime();
    if (spins <= 256u) {
        t_first = now;
        return false;
    }
    return now - t_first > kWaitTicks;
}

// One 16-byte device-scope load.  Each 8-byte half is validated on its own by the caller, so nothing depends on the
// 16 bytes being read as a unit.
__device__ __forceinline__ void load16_device_scope(const void* p, unsigned long long& lo, unsigned long long& hi)
{
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    lo = (unsigned long long)v[0] | ((unsigned long long)v[1] << 32);
    hi = (unsigned long long)v[2] | ((unsigned long long)v[3] << 32);
}

// One 16-byte device-scope store of two 8-byte words (each validated on its own by the readers).
__device__ __forceinline__ void store16_device_scope(void* p, unsigned long long lo, unsigned long long hi)
{
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 v = {(unsigned int)lo, (unsigned int)(lo >> 32), (unsigned int)hi, (unsigned int)(hi >> 32)};
    asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}

// relu as at::relu computes it (the reference applies it to its GEMV's result, aten_ops.cpp:466, 704-705): below zero
// becomes zero and a NaN stays a NaN; fmaxf would return its other operand for one.
__device__ __forceinline__ float relu_f32(float v) { return v < 0.0f ? 0.0f : v; }

// fp32 -> fp16 with the fp32 value made first.  Without the empty statement in between, hipcc folds a product or an fma
// whose only use is the conversion into v_fma_mixlo_f16, which rounds once from the exact result; the same expression with a
// second use rounds twice (fp32, then fp16).  Code paths that must agree bit for bit convert through this.
__device__ __forceinline__ half_t round_f16(float v)
{
    asm volatile("" : "+v"(v));
    return (half_t)v;
}

__device__ __forceinline__ float sigmoid_f32(float v) { return 1.0f / (1.0f + __expf(-v)); }

// Sigmoid on the hardware exp2 and reciprocal (about 1 ulp each): exact limits 0 and 1 at -+inf, absolute error
// below 1e-6, far inside the fp16 rounding of h.  Used where the activation sits on a latency-critical path.
__device__ __forceinline__ float fast_sigmoid_f32(float v)
{
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
}

__device__ __forceinline__ float tanh_f32(float v)
{
    // tanh(v) = 1 - 2 / (exp(2v) + 1); exact limits at +-inf, no cancellation near 0 beyond 1 ulp of 1.
    const float e = __expf(2.0f * v);
    return 1.0f - 2.0f / (e + 1.0f);
}

}  // namespace pimhip
