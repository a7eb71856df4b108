// Shared host/device helpers for the gfx950 kernels: error reporting, dtype traits,
// 16-byte vector access, wavefront (64-lane) group reductions on DPP / ds_swizzle, fast division.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/rgd_hip.h"

// ------------------------------------------------------------------------------------------
// host: errors
// ------------------------------------------------------------------------------------------
void rgd_set_error(const char* fmt, ...);  // defined in api.hip

#define RGD_REQUIRE(cond, code, ...)        \
    do {                                    \
        if (!(cond)) {                      \
            rgd_set_error(__VA_ARGS__);     \
            return (code);                  \
        }                                   \
    } while (0)

// One-time set-up of the library (api.hip): compute-unit count, LDS size attributes of the attention kernels, address
// of the fixed scratch array.  Every entry point calls it first; once it has run on a process with a device it is one
// atomic load, so in the steady state an entry point makes no runtime call other than its kernel launches.  A process
// without a usable device latches nothing: the next call tries again.
void rgd_ensure_init();
int rgd_attn_ready();  // rgd_ensure_init, then the status of the attention kernels' set-up (error text set on failure)
int rgd_num_cus();     // compute units of the device seen by the set-up (256 while none has been seen)

// Kernel launch that returns its own error code.  Kernels take their parameter struct by value; a second scalar
// argument is allowed.
template <typename P>
inline hipError_t rgd_launch(void (*kern)(P), dim3 grid, dim3 block, size_t lds, hipStream_t s, const P& p) {
    void* args[] = {const_cast<P*>(&p)};
    return hipLaunchKernel(reinterpret_cast<const void*>(kern), grid, block, args, lds, s);
}
template <typename P, typename A>
inline hipError_t rgd_launch(void (*kern)(P, A), dim3 grid, dim3 block, size_t lds, hipStream_t s, const P& p, A a) {
    void* args[] = {const_cast<P*>(&p), &a};
    return hipLaunchKernel(reinterpret_cast<const void*>(kern), grid, block, args, lds, s);
}
// hipError_t of a launch -> rgd_status, with the error text set; a failure is also cleared from the runtime's
// per-thread last error
int rgd_launch_status(const char* what, hipError_t e);

static inline bool rgd_dtype_ok(int d) { return d == RGD_F32 || d == RGD_F16 || d == RGD_BF16; }
static inline int rgd_dtype_size(int d) { return d == RGD_F32 ? 4 : 2; }
static inline bool rgd_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ------------------------------------------------------------------------------------------
// element types
// ------------------------------------------------------------------------------------------
typedef _Float16 f16_t;
typedef __bf16 bf16_t;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef f16_t f16x8 __attribute__((ext_vector_type(8)));
typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
typedef f16_t f16x4 __attribute__((ext_vector_type(4)));

template <typename T> struct DType;
template <> struct DType<float> { static constexpr int code = RGD_F32; };
template <> struct DType<f16_t> { static constexpr int code = RGD_F16; };
template <> struct DType<bf16_t> { static constexpr int code = RGD_BF16; };

template <typename T> __device__ __forceinline__ float to_f32(T v) { return static_cast<float>(v); }
template <typename T> __device__ __forceinline__ T from_f32(float v) { return static_cast<T>(v); }

// ------------------------------------------------------------------------------------------
// chunk access: N contiguous elements of type T <-> N floats.
// VECTOR = true uses 16-byte accesses (address and N*sizeof(T) must be multiples of 16).
// ------------------------------------------------------------------------------------------
template <typename T, int N, bool VECTOR>
__device__ __forceinline__ void load_chunk(const T* __restrict__ p, int first, int limit, float (&out)[N]) {
    // loads elements [first, first+N) of the row at p; elements at or beyond `limit` read as 0
    // a chunk that is not a whole number of 16-byte vectors (fp32 rows with 16-bit weights) is read
    // element by element
    if constexpr (VECTOR && (N * sizeof(T)) % 16 == 0) {
        constexpr int BYTES = N * sizeof(T);
        constexpr int NV = BYTES / 16;
        constexpr int EPV = 16 / sizeof(T);
        if (first < limit) {  // limit is a multiple of N on this path
            const u32x4* vp = reinterpret_cast<const u32x4*>(p + first);
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                u32x4 raw = vp[v];
                T tmp[EPV];
                __builtin_memcpy(tmp, &raw, 16);
#pragma unroll
                for (int e = 0; e < EPV; ++e) out[v * EPV + e] = to_f32<T>(tmp[e]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < N; ++e) out[e] = 0.f;
        }
    } else {
#pragma unroll
        for (int e = 0; e < N; ++e) out[e] = (first + e < limit) ? to_f32<T>(p[first + e]) : 0.f;
    }
}

template <typename T, int N, bool VECTOR, bool NT = false>
__device__ __forceinline__ void store_chunk(T* __restrict__ p, int first, int limit, const float (&in)[N]) {
    if constexpr (VECTOR && (N * sizeof(T)) % 16 == 0) {
        constexpr int BYTES = N * sizeof(T);
        constexpr int NV = BYTES / 16;
        constexpr int EPV = 16 / sizeof(T);
        if (first < limit) {
            u32x4* vp = reinterpret_cast<u32x4*>(p + first);
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                T tmp[EPV];
#pragma unroll
                for (int e = 0; e < EPV; ++e) tmp[e] = from_f32<T>(in[v * EPV + e]);
                u32x4 raw;
                __builtin_memcpy(&raw, tmp, 16);
                if constexpr (NT)
                    __builtin_nontemporal_store(raw, vp + v);
                else
                    vp[v] = raw;
            }
        }
    } else {
#pragma unroll
        for (int e = 0; e < N; ++e)
            if (first + e < limit) p[first + e] = from_f32<T>(in[e]);
    }
}

// 16-byte path: N floats -> `base + byte_off` (uniform base, 32-bit offset per lane), if `ok`
template <typename T, int N, bool NT = false>
__device__ __forceinline__ void store_chunk_at(void* __restrict__ base, uint32_t byte_off, bool ok, const float (&in)[N]) {
    static_assert((N * sizeof(T)) % 16 == 0, "store_chunk_at: 16-byte chunks");
    constexpr int NV = N * sizeof(T) / 16;
    constexpr int EPV = 16 / sizeof(T);
    if (ok) {
        u32x4* vp = reinterpret_cast<u32x4*>(static_cast<char*>(base) + byte_off);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            T tmp[EPV];
#pragma unroll
            for (int e = 0; e < EPV; ++e) tmp[e] = from_f32<T>(in[v * EPV + e]);
            u32x4 raw;
            __builtin_memcpy(&raw, tmp, 16);
            if constexpr (NT)
                __builtin_nontemporal_store(raw, vp + v);
            else
                vp[v] = raw;
        }
    }
}

// Branch-free variant used in the streaming loops: the load is unconditional (a chunk that is out of
// range reads the start of the row instead, which is always valid memory) and out-of-range elements are
// zeroed by a select when the raw bits are decoded.  Issue every load() of an iteration first, then
// decode(): the loads overlap and the wavefront waits once.
// NT: non-temporal loads (data that is read once and not shared between workgroups).  Measured: on x they
// shorten forward kernels by 7-12 % but take the rows out of the Infinity Cache, which a backward that
// re-reads them soon pays for; on the upstream gradient of the backward kernels they gain 3-5 %.
template <typename T, int N, bool VECTOR, bool NT = false> struct Chunk {
    static constexpr bool VEC = VECTOR && (N * sizeof(T)) % 16 == 0;
    static constexpr int NVEC = VEC ? (N * sizeof(T)) / 16 : 1;
    static constexpr int EPV = 16 / sizeof(T);
    u32x4 v[NVEC];
    T s[VEC ? 1 : N];

    __device__ __forceinline__ void load(const T* __restrict__ row, int first, int limit) {
        if constexpr (VEC) {
            const u32x4* p = reinterpret_cast<const u32x4*>(row + (first < limit ? first : 0));
#pragma unroll
            for (int i = 0; i < NVEC; ++i) {
                if constexpr (NT)
                    v[i] = __builtin_nontemporal_load(p + i);
                else
                    v[i] = p[i];
            }
        } else {
#pragma unroll
            for (int e = 0; e < N; ++e) s[e] = row[first + e < limit ? first + e : 0];
        }
    }
    // 16-byte path only: the chunk at `base + byte_off`, a uniform base and a 32-bit offset per lane (the address
    // arithmetic stays in 32 bits and the load takes the base from scalar registers)
    __device__ __forceinline__ void load_at(const void* __restrict__ base, uint32_t byte_off) {
        static_assert(VEC, "load_at: 16-byte chunks");
        const u32x4* p = reinterpret_cast<const u32x4*>(static_cast<const char*>(base) + byte_off);
#pragma unroll
        for (int i = 0; i < NVEC; ++i) {
            if constexpr (NT)
                v[i] = __builtin_nontemporal_load(p + i);
            else
                v[i] = p[i];
        }
    }
    // MASK = false skips the zeroing selects (the caller knows every element is in range)
    template <bool MASK = true> __device__ __forceinline__ void decode(int first, int limit, float (&out)[N]) const {
        if constexpr (VEC) {
            const bool ok = !MASK || first < limit;
#pragma unroll
            for (int i = 0; i < NVEC; ++i) {
                T tmp[EPV];
                __builtin_memcpy(tmp, &v[i], 16);
#pragma unroll
                for (int e = 0; e < EPV; ++e) out[i * EPV + e] = ok ? to_f32<T>(tmp[e]) : 0.f;
            }
        } else {
#pragma unroll
            for (int e = 0; e < N; ++e) out[e] = (!MASK || first + e < limit) ? to_f32<T>(s[e]) : 0.f;
        }
    }
};

// chunk load whose element type is only known at run time (weights, rotary tables)
template <int N, bool VECTOR>
__device__ __forceinline__ void load_chunk_dyn(const void* p, int dtype, int first, int limit, float (&out)[N]) {
    if (dtype == RGD_BF16)
        load_chunk<bf16_t, N, VECTOR>(static_cast<const bf16_t*>(p), first, limit, out);
    else if (dtype == RGD_F16)
        load_chunk<f16_t, N, VECTOR>(static_cast<const f16_t*>(p), first, limit, out);
    else
        load_chunk<float, N, VECTOR>(static_cast<const float*>(p), first, limit, out);
}

__device__ __forceinline__ void store_dyn(void* p, int dtype, int64_t idx, float v) {
    if (dtype == RGD_BF16)
        static_cast<bf16_t*>(p)[idx] = from_f32<bf16_t>(v);
    else if (dtype == RGD_F16)
        static_cast<f16_t*>(p)[idx] = from_f32<f16_t>(v);
    else
        static_cast<float*>(p)[idx] = v;
}

// ------------------------------------------------------------------------------------------
// wavefront group reductions.  A "group" is G consecutive lanes (G a power of two <= 64);
// every lane of the group ends up with the group's result.
// ------------------------------------------------------------------------------------------
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float lane_xor16(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // SWAP,16
}
__device__ __forceinline__ float lane_xor32(float v) {
    int lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, v)));
}

struct OpSum { static __device__ __forceinline__ float apply(float a, float b) { return a + b; } };
struct OpMax { static __device__ __forceinline__ float apply(float a, float b) { return fmaxf(a, b); } };

template <int G, typename Op = OpSum> __device__ __forceinline__ float group_reduce(float v) {
    // quad_perm [1,0,3,2] / [2,3,0,1], then row_half_mirror and row_mirror: after the quad steps all
    // four lanes of a quad agree, so the mirrors are equivalent to xor 4 and xor 8
    if constexpr (G >= 2) v = Op::apply(v, dpp_move<0xB1>(v));
    if constexpr (G >= 4) v = Op::apply(v, dpp_move<0x4E>(v));
    if constexpr (G >= 8) v = Op::apply(v, dpp_move<0x141>(v));
    if constexpr (G >= 16) v = Op::apply(v, dpp_move<0x140>(v));
    if constexpr (G >= 32) v = Op::apply(v, lane_xor16(v));
    if constexpr (G >= 64) v = Op::apply(v, lane_xor32(v));
    return v;
}

// sum over the lanes of a wave that share (lane % G): used once per block for the dw partials
template <int G> __device__ __forceinline__ float cross_group_sum(float v) {
#pragma unroll
    for (int off = G; off < 64; off <<= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// ------------------------------------------------------------------------------------------
// division of a 31-bit value by a run-time constant: q = (mulhi(n, m) + n) >> s
// ------------------------------------------------------------------------------------------
struct FastDiv {
    uint32_t d, m, s;
};
static inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d ? d : 1;
    uint32_t s = 0;
    while ((1ull << s) < f.d) ++s;
    f.s = s;
    f.m = static_cast<uint32_t>(((1ull << 32) * ((1ull << s) - f.d)) / f.d + 1);
    return f;
}
__device__ __forceinline__ uint32_t fast_div(uint32_t n, const FastDiv& f) {
    return (__umulhi(n, f.m) + n) >> f.s;
}

__device__ __forceinline__ int lane_id() { return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }
