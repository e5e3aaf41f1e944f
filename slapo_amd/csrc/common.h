// Shared device/host helpers for the gfx950 kernels: element-type traits, 128-bit vector
// access, launch checking, and the host-side conversion of a dropout plan into kernel state.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/slapo_amd.h"
#include "philox.h"

namespace slapo {

typedef _Float16 f16_t;
typedef __bf16 bf16_t;

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

template <typename T>
struct Elem;

template <>
struct Elem<float> {
    static constexpr int kPerVec = 4;  // elements per 16-byte access
    static __device__ __forceinline__ float to_f32(float v) { return v; }
    static __device__ __forceinline__ float from_f32(float v) { return v; }
};
template <>
struct Elem<f16_t> {
    static constexpr int kPerVec = 8;
    static __device__ __forceinline__ float to_f32(f16_t v) { return (float)v; }
    static __device__ __forceinline__ f16_t from_f32(float v) { return (f16_t)v; }
};
template <>
struct Elem<bf16_t> {
    static constexpr int kPerVec = 8;
    static __device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }
    static __device__ __forceinline__ bf16_t from_f32(float v) { return (bf16_t)v; }
};

// A 16-byte packet of elements of type T, loadable/storable with one 128-bit access.
template <typename T>
struct alignas(16) Packet {
    T v[Elem<T>::kPerVec];
};

template <typename T>
__device__ __forceinline__ Packet<T> load_packet(const T* p) {
    Packet<T> r;
    *reinterpret_cast<u32x4_t*>(&r) = *reinterpret_cast<const u32x4_t*>(p);
    return r;
}
template <typename T>
__device__ __forceinline__ void store_packet(T* p, const Packet<T>& r) {
    *reinterpret_cast<u32x4_t*>(p) = *reinterpret_cast<const u32x4_t*>(&r);
}
// Streaming variants: data touched once, keep it from displacing reusable lines.
template <typename T>
__device__ __forceinline__ Packet<T> load_packet_nt(const T* p) {
    Packet<T> r;
    *reinterpret_cast<u32x4_t*>(&r) =
        __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return r;
}
template <typename T>
__device__ __forceinline__ void store_packet_nt(T* p, const Packet<T>& r) {
    __builtin_nontemporal_store(*reinterpret_cast<const u32x4_t*>(&r),
                                reinterpret_cast<u32x4_t*>(p));
}

inline int check_launch() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SLAPO_OK : SLAPO_ERR_LAUNCH;
}

// Kernels that need more than 48 KB of dynamic LDS must be told so once per device.  `done` is
// the caller's flag word (one per kernel instantiation), bit i = device i has been set up.
inline int allow_dynamic_lds(const void* kern, size_t bytes, std::atomic<uint64_t>& done) {
    if (bytes <= 48 * 1024) return SLAPO_OK;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return SLAPO_ERR_LAUNCH;
    const uint64_t bit = 1ull << (dev & 63);
    if (dev < 64 && (done.load(std::memory_order_acquire) & bit)) return SLAPO_OK;
    if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) !=
        hipSuccess)
        return SLAPO_ERR_LAUNCH;
    if (dev < 64) done.fetch_or(bit, std::memory_order_release);
    return SLAPO_OK;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Host: turn (plan, p, seed, offset) into the state the kernels read.
inline DropoutState make_dropout_state(const slapo_dropout_plan& plan, double p, uint64_t seed,
                                       uint64_t offset) {
    DropoutState s;
    s.key0 = (uint32_t)seed;
    s.key1 = (uint32_t)(seed >> 32);
    s.base_counter = offset / 4;
    s.total_threads = (uint64_t)plan.total_threads;
    s.vec = (uint32_t)plan.vec;
    s.calls_per_iter = (uint32_t)plan.calls_per_iter;
    int all = 0, none = 0;
    s.keep_max = slapo_amd_dropout_threshold(p, &all, &none);
    s.keep_none = (uint32_t)none;
    s.t_shift = -1;
    if (s.total_threads && (s.total_threads & (s.total_threads - 1)) == 0) {
        int sh = 0;
        while ((1ull << sh) != s.total_threads) ++sh;
        s.t_shift = sh;
    }
    s.g_shift = s.vec >= 4 ? (s.vec == 4 ? 0 : s.vec == 8 ? 1 : 2) : -1;
    s.inv_keep = p < 1.0 ? (float)(1.0 / (double)(float)(1.0 - p)) : 0.f;
    s.device_state = static_cast<const uint64_t*>(plan.rng_state);
    return s;
}

inline bool plan_ok(const slapo_dropout_plan* plan, int64_t numel) {
    if (!plan) return false;
    if (plan->numel != numel || plan->total_threads <= 0) return false;
    const int v = plan->vec;
    if (!(v == 1 || v == 2 || v == 4 || v == 8 || v == 16)) return false;
    if (numel % v != 0) return false;
    const int calls = v == 1 ? 1 : (v + 3) / 4;
    return plan->calls_per_iter == calls;
}

}  // namespace slapo
