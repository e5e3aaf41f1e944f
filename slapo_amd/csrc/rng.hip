// Dropout RNG: host-side Philox mirror, ATen launch-plan arithmetic, keep threshold, and the
// host / device mask generators behind slapo_amd_dropout_mask*.  The mapping itself lives in
// philox.h (shared by every kernel that regenerates mask bits).
#include "common.h"

using namespace slapo;

extern "C" void slapo_amd_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2],
                                        uint32_t out[4]) {
    const u32x4 r = philox4x32_10(ctr[0], ctr[1], ctr[2], ctr[3], key[0], key[1]);
    out[0] = r.x;
    out[1] = r.y;
    out[2] = r.z;
    out[3] = r.w;
}

extern "C" int slapo_amd_dropout_plan_for(int64_t numel, int elem_bytes, int64_t ptr_align,
                                          int num_cus, int max_threads_per_cu,
                                          slapo_dropout_plan* plan) {
    if (!plan || numel <= 0 || num_cus <= 0 || max_threads_per_cu < 256) return SLAPO_ERR_ARG;
    if (!(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8))
        return SLAPO_ERR_DTYPE;
    const int64_t block = 256;
    const int64_t cap = (int64_t)num_cus * (max_threads_per_cu / block);
    int64_t grid = (numel + block - 1) / block;
    if (grid > cap) grid = cap;
    // Widest vector the ROCm build of ATen allows for this element size and alignment:
    // 16 elements for 1-byte types, 8 for 2-byte types, 4 otherwise, limited by the pointer
    // alignment, then halved until it divides numel.
    int vec;
    if (elem_bytes == 1 && ptr_align % 16 == 0)
        vec = 16;
    else if (elem_bytes <= 2 && ptr_align % (8 * elem_bytes) == 0)
        vec = 8;
    else if (ptr_align % (4 * elem_bytes) == 0)
        vec = 4;
    else if (ptr_align % (2 * elem_bytes) == 0)
        vec = 2;
    else
        vec = 1;
    while (vec > 1 && numel % vec != 0) vec /= 2;
    plan->numel = numel;
    plan->total_threads = grid * block;
    plan->vec = vec;
    plan->calls_per_iter = vec == 1 ? 1 : (vec + 3) / 4;
    const int64_t unroll = 4;
    plan->offset_increment = ((numel - 1) / (block * grid * unroll) + 1) * unroll;
    plan->rng_state = nullptr;
    return SLAPO_OK;
}

extern "C" int slapo_amd_dropout_plan(int64_t numel, int elem_bytes, int64_t ptr_align,
                                      int device, slapo_dropout_plan* plan) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) return SLAPO_ERR_DEVICE;
    return slapo_amd_dropout_plan_for(numel, elem_bytes, ptr_align, prop.multiProcessorCount,
                                      prop.maxThreadsPerMultiProcessor, plan);
}

static inline float uniform_of(uint32_t v) {
    const float inv = 2.3283064365386963e-10f;  // 2^-32
    volatile float prod = (float)v * inv;       // exact: power-of-two scaling
    return inv + prod;
}

extern "C" uint32_t slapo_amd_dropout_threshold(double p, int* keep_all, int* keep_none) {
    const float pkeep = (float)(1.0 - p);
    int all = 0, none = 0;
    uint32_t thr = 0;
    if (!(uniform_of(0u) < pkeep)) {
        none = 1;
    } else if (uniform_of(0xFFFFFFFFu) < pkeep) {
        all = 1;
        thr = 0xFFFFFFFFu;
    } else {
        uint32_t lo = 0, hi = 0xFFFFFFFFu;  // keep(lo) true, keep(hi) false
        while (hi - lo > 1) {
            const uint32_t mid = lo + (hi - lo) / 2;
            if (uniform_of(mid) < pkeep)
                lo = mid;
            else
                hi = mid;
        }
        thr = lo;
    }
    if (keep_all) *keep_all = all;
    if (keep_none) *keep_none = none;
    return thr;
}

extern "C" int slapo_amd_dropout_mask_host(uint8_t* mask, const slapo_dropout_plan* plan,
                                           double p, uint64_t seed, uint64_t offset) {
    if (!mask || !plan || !plan_ok(plan, plan->numel)) return SLAPO_ERR_ARG;
    if (!(p >= 0.0 && p <= 1.0)) return SLAPO_ERR_ARG;
    if (plan->rng_state != nullptr) return SLAPO_ERR_ARG;  // device memory: not readable here
    const DropoutState s = make_dropout_state(*plan, p, seed, offset);
    const int64_t n = plan->numel;
    if (s.vec >= 4 && n % 4 == 0) {
        for (int64_t g = 0; g < n / 4; ++g) {
            const uint32_t bits = dropout_keep4(s, (uint64_t)g);
            for (int i = 0; i < 4; ++i) mask[4 * g + i] = (bits >> i) & 1u;
        }
    } else {
        for (int64_t i = 0; i < n; ++i) mask[i] = dropout_keep1(s, (uint64_t)i) ? 1 : 0;
    }
    return SLAPO_OK;
}

__global__ __launch_bounds__(256) void dropout_mask_kernel(uint8_t* __restrict__ mask,
                                                           int64_t numel, DropoutState s) {
    resolve_device_state(s);
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (s.vec >= 4) {
        const int64_t g = tid;
        if (4 * g >= numel) return;
        const uint32_t bits = dropout_keep4(s, (uint64_t)g);
        uint32_t packed = (bits & 1u) | ((bits & 2u) << 7) | ((bits & 4u) << 14) |
                          ((bits & 8u) << 21);
        *reinterpret_cast<uint32_t*>(mask + 4 * g) = packed;
    } else {
        for (int i = 0; i < 4; ++i) {
            const int64_t e = 4 * tid + i;
            if (e < numel) mask[e] = dropout_keep1(s, (uint64_t)e) ? 1 : 0;
        }
    }
}

extern "C" int slapo_amd_dropout_mask(uint8_t* mask, const slapo_dropout_plan* plan, double p,
                                      uint64_t seed, uint64_t offset, void* stream) {
    if (!mask || !plan || !plan_ok(plan, plan->numel)) return SLAPO_ERR_ARG;
    if (!(p >= 0.0 && p <= 1.0)) return SLAPO_ERR_ARG;
    if (plan->vec >= 4 && (reinterpret_cast<uintptr_t>(mask) & 3u)) return SLAPO_ERR_ALIGN;
    const DropoutState s = make_dropout_state(*plan, p, seed, offset);
    const int64_t groups = (plan->numel + 3) / 4;
    const int64_t blocks = (groups + 255) / 256;
    if (blocks > 0x7FFFFFFF) return SLAPO_ERR_SHAPE;
    hipLaunchKernelGGL(dropout_mask_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, mask, plan->numel, s);
    return check_launch();
}

extern "C" int slapo_amd_abi_version(void) { return SLAPO_AMD_ABI_VERSION; }

extern "C" const char* slapo_amd_status_string(int status) {
    switch (status) {
        case SLAPO_OK: return "ok";
        case SLAPO_ERR_DTYPE: return "unsupported element type";
        case SLAPO_ERR_SHAPE: return "unsupported or inconsistent shape";
        case SLAPO_ERR_ALIGN: return "pointer or stride not sufficiently aligned";
        case SLAPO_ERR_ARG: return "invalid argument";
        case SLAPO_ERR_LAUNCH: return "kernel launch failed";
        case SLAPO_ERR_DEVICE: return "no usable gfx950 device";
        case SLAPO_ERR_WORKSPACE: return "workspace missing or too small";
        default: return "unknown status";
    }
}
