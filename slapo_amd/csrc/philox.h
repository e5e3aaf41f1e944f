// Philox4x32-10 counter-based RNG and the element -> (subsequence, counter, lane) mapping that
// ATen's fused dropout kernels use, written once for host and device so the two agree bit for
// bit.  The mapping (reference call sites: torch.nn.functional.dropout at
// slapo/op/fused_bias.py:74 and slapo/op/attention.py:179-180):
//
//   launch:  block = 256 threads, grid = min(num_cus * (max_threads_per_cu / 256),
//            ceil(numel / 256)), T = 256 * grid subsequences, one per thread;
//   vector kernel (vec in {2,4,8,16}): thread t, loop trip m handles the `vec` consecutive
//            elements starting at (m * T + t) * vec and draws ceil(vec/4) Philox blocks per
//            trip; element e of the group uses word e % 4 of block e / 4;
//   scalar kernel (vec == 1): thread t, loop trip m draws one block; word w belongs to
//            element t + T * (4 * m + w);
//   Philox block number c of subsequence t under generator state (seed, offset) has
//            key = seed, counter = { lo(offset/4 + c), hi(offset/4 + c), lo(t), hi(t) };
//   keep iff  2^-32 + float(word) * 2^-32 < float(1 - p)   (rocRAND's uniform conversion).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define SLAPO_HD __host__ __device__ __forceinline__
#else
#define SLAPO_HD inline
#endif

namespace slapo {

struct u32x4 {
    uint32_t x, y, z, w;
};

// a ^ b ^ c.  On the device one instruction (v_bitop3_b32 with the truth table of a three-way XOR)
// where two v_xor_b32 would be needed: a Philox round is then two multiplications and two of
// these instead of two and four.
SLAPO_HD uint32_t xor3(uint32_t a, uint32_t b, uint32_t c) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
#else
    return a ^ b ^ c;
#endif
}

SLAPO_HD u32x4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                             uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = xor3((uint32_t)(p1 >> 32), c1, k0);
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = xor3((uint32_t)(p0 >> 32), c3, k1);
        const uint32_t n3 = (uint32_t)p0;
        c0 = n0;
        c1 = n1;
        c2 = n2;
        c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return u32x4{c0, c1, c2, c3};
}

// Everything a kernel needs to regenerate mask bits; filled on the host.
struct DropoutState {
    uint32_t key0, key1;      // seed lo / hi
    uint64_t base_counter;    // offset / 4
    uint64_t total_threads;   // T
    uint32_t vec;             // 1,2,4,8,16
    uint32_t calls_per_iter;  // ceil(vec/4), 1 for vec==1
    uint32_t keep_max;        // keep iff word <= keep_max (unless keep_none)
    uint32_t keep_none;       // 1: nothing is kept (p == 1)
    int32_t t_shift;          // log2(T) when T is a power of two, else -1
    int32_t g_shift;          // log2(vec / 4) when vec >= 4, else -1
    float inv_keep;           // 1 / (1 - p)
    // NULL, or device memory holding {seed, offset}: a kernel then takes key and base counter
    // from there (resolve_device_state) instead of the three fields above
    const uint64_t* device_state;
};

#if defined(__HIPCC__)
// First statement of every kernel that draws: a uniform branch and one 16-byte uniform read.
__device__ __forceinline__ void resolve_device_state(DropoutState& s) {
    if (s.device_state != nullptr) {
        const uint64_t seed = s.device_state[0];
        const uint64_t offset = s.device_state[1];
        s.key0 = (uint32_t)seed;
        s.key1 = (uint32_t)(seed >> 32);
        s.base_counter = offset >> 2;
    }
}
#endif

SLAPO_HD void split_by_threads(const DropoutState& s, uint64_t v, uint64_t& thread,
                               uint64_t& trip) {
    if (s.t_shift >= 0) {
        trip = v >> s.t_shift;
        thread = v & (s.total_threads - 1);
    } else {
        trip = v / s.total_threads;
        thread = v - trip * s.total_threads;
    }
}

SLAPO_HD u32x4 philox_block(const DropoutState& s, uint64_t thread, uint64_t call) {
    const uint64_t c = s.base_counter + call;
    return philox4x32_10((uint32_t)c, (uint32_t)(c >> 32), (uint32_t)thread,
                         (uint32_t)(thread >> 32), s.key0, s.key1);
}

SLAPO_HD bool keep_word(const DropoutState& s, uint32_t w) {
    return (w <= s.keep_max) && !s.keep_none;
}

// Keep-bit of one element (any vec).  Costs a full Philox block per element.
SLAPO_HD bool dropout_keep1(const DropoutState& s, uint64_t elem) {
    uint64_t thread, trip, call;
    uint32_t lane;
    if (s.vec == 1) {
        uint64_t q;
        split_by_threads(s, elem, thread, q);
        call = q >> 2;
        lane = (uint32_t)(q & 3);
    } else {
        const uint64_t v = elem / s.vec;
        const uint32_t e = (uint32_t)(elem - v * s.vec);
        split_by_threads(s, v, thread, trip);
        call = trip * s.calls_per_iter + (e >> 2);
        lane = e & 3;
    }
    const u32x4 r = philox_block(s, thread, call);
    const uint32_t w = lane == 0 ? r.x : lane == 1 ? r.y : lane == 2 ? r.z : r.w;
    return keep_word(s, w);
}

// Keep-bits (bit i <-> element 4*group + i) of an aligned group of four consecutive elements.
// Valid only when vec is 4, 8 or 16 (one Philox block covers the group).
SLAPO_HD uint32_t dropout_keep4(const DropoutState& s, uint64_t group) {
    const uint32_t groups_per_vec = s.vec >> 2;  // 1, 2 or 4
    uint64_t v, sub;
    if (groups_per_vec == 1) {
        v = group;
        sub = 0;
    } else if (groups_per_vec == 2) {
        v = group >> 1;
        sub = group & 1;
    } else {
        v = group >> 2;
        sub = group & 3;
    }
    uint64_t thread, trip;
    split_by_threads(s, v, thread, trip);
    const u32x4 r = philox_block(s, thread, trip * s.calls_per_iter + sub);
    return (keep_word(s, r.x) ? 1u : 0u) | (keep_word(s, r.y) ? 2u : 0u) |
           (keep_word(s, r.z) ? 4u : 0u) | (keep_word(s, r.w) ? 8u : 0u);
}

// dropout_keep4 for the common launch geometry: vec >= 4 and a power-of-two thread count, so the
// element -> (subsequence, counter) split is shifts and masks only.
SLAPO_HD uint32_t dropout_keep4_pow2(const DropoutState& s, uint64_t group) {
    const uint64_t v = group >> s.g_shift;
    const uint32_t sub = (uint32_t)group & ((1u << s.g_shift) - 1u);
    const uint64_t thread = v & (s.total_threads - 1);
    const uint64_t trip = v >> s.t_shift;
    const u32x4 r = philox_block(s, thread, trip * s.calls_per_iter + sub);
    return (keep_word(s, r.x) ? 1u : 0u) | (keep_word(s, r.y) ? 2u : 0u) |
           (keep_word(s, r.z) ? 4u : 0u) | (keep_word(s, r.w) ? 8u : 0u);
}

// Keep-bits of the n (1..4) consecutive elements starting at elem, for any launch geometry and
// alignment.  Deliberately a rolled loop: this path is rare and must stay small.
SLAPO_HD uint32_t dropout_keep_any(const DropoutState& s, uint64_t elem, int n) {
    uint32_t bits = 0;
#if defined(__HIPCC__)
#pragma unroll 1
#endif
    for (int e = 0; e < n; ++e) bits |= (dropout_keep1(s, elem + (uint64_t)e) ? 1u : 0u) << e;
    return bits;
}

}  // namespace slapo
