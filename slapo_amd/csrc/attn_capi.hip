// C-ABI entry points of the attention path: argument validation, kernel selection (MFMA kernels
// for fp16 / bf16, FMA kernels for fp32) and the small helper kernels around the backward
// (delta = rowsum(dO * O)).
#include <mutex>

#include "attn_common.h"

namespace slapo {
int attn_fwd_mfma_f16(const AttnArgs& a, hipStream_t st);
int attn_fwd_mfma_bf16(const AttnArgs& a, hipStream_t st);
int attn_bwd_mfma_f16(const AttnArgs& a, hipStream_t st);
int attn_bwd_mfma_bf16(const AttnArgs& a, hipStream_t st);
int attn_bwd_dq_mfma_f16(const AttnArgs& a, hipStream_t st);
int attn_bwd_dq_mfma_bf16(const AttnArgs& a, hipStream_t st);
int attn_fwd_f32(const AttnArgs& a, hipStream_t st);
int attn_bwd_f32(const AttnArgs& a, hipStream_t st);
}  // namespace slapo

using namespace slapo;

namespace {

// delta[bh, i] = sum_d dO[b,i,h,d] * O[b,i,h,d]; eight lanes share a row, 16 bytes per lane.
template <typename T>
__global__ __launch_bounds__(256) void attn_delta_kernel(const AttnArgs a) {
    constexpr int V = Elem<T>::kPerVec;
    const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 3;
    const int sub = threadIdx.x & 7;
    const int64_t n_rows = (int64_t)a.batch * a.heads * a.sq;
    float acc = 0.f;
    if (row < n_rows) {
        const int i = (int)(row % a.sq);
        const int bh = (int)(row / a.sq);
        const int b = bh / a.heads, h = bh % a.heads;
        const int64_t off = b * a.os[0] + (int64_t)i * a.os[1] + h * a.os[2];
        const T* o = reinterpret_cast<const T*>(a.o) + off;
        const T* g = reinterpret_cast<const T*>(a.dout) + off;
        // head_dim is a multiple of V on this path (checked by the dispatcher)
        for (int c = sub * V; c < a.d; c += 8 * V) {
            const Packet<T> po = load_packet<T>(o + c);
            const Packet<T> pg = load_packet<T>(g + c);
#pragma unroll
            for (int e = 0; e < V; ++e)
                acc = __builtin_fmaf(Elem<T>::to_f32(po.v[e]), Elem<T>::to_f32(pg.v[e]), acc);
        }
    }
    acc += __shfl_xor(acc, 1, 64);
    acc += __shfl_xor(acc, 2, 64);
    acc += __shfl_xor(acc, 4, 64);
    if (row < n_rows && sub == 0) a.delta[row] = acc;
}

// Scalar variant for fp32 tensors whose rows are not 16-byte aligned.
__global__ __launch_bounds__(256) void attn_delta_scalar_kernel(const AttnArgs a) {
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t n_rows = (int64_t)a.batch * a.heads * a.sq;
    if (row >= n_rows) return;
    const int i = (int)(row % a.sq);
    const int bh = (int)(row / a.sq);
    const int b = bh / a.heads, h = bh % a.heads;
    const int64_t off = b * a.os[0] + (int64_t)i * a.os[1] + h * a.os[2];
    const float* o = reinterpret_cast<const float*>(a.o) + off;
    const float* g = reinterpret_cast<const float*>(a.dout) + off;
    float acc = 0.f;
    for (int e = 0; e < a.d; ++e) acc = __builtin_fmaf(o[e], g[e], acc);
    a.delta[row] = acc;
}

// Dropout keep bits of a 16-bit attention call, drawn once for the forward and both backward
// kernels: thread (row i, word w) draws the eight Philox blocks of keys 32 w .. 32 w + 31 of
// query i and stores them as one word, keep_mask[(bh * mask_words + w) * mask_pitch + i], bit j =
// keep(i, 32 w + j).  The matrix kernels then only test bits; drawing inside the forward kernel
// costs about forty vector-ALU cycles per score beside thirty-two (head_dim 128) or sixteen (64)
// of matrix work.  Only words that hold a key the row itself can see are drawn: the kernels read
// whole words of every 64-key tile that some query of a 32-query group sees, but a bit that
// belongs to a pair outside the row's own mask meets a probability of zero, so what such words
// hold does not matter and they are left as they are.  With a local window the grid's second
// dimension counts words from the first one of the row's window (window / 32 + 1 of them, not
// seqlen_k / 32: every thread then has a word to draw); without one it is the word itself.
// kExact: any launch geometry of the dropout plan and any seqlen_k (one Philox block per bit).
template <bool kExact>
__global__ __launch_bounds__(256) void keep_mask_kernel(const AttnArgs a_in) {
    AttnArgs a = a_in;
    resolve_device_state(a.rng);
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int bh = blockIdx.z;
    if (i >= a.sq) return;
    int w = blockIdx.y;
    if (a.window > 0) w += max(i - a.window + 1, 0) >> 5;
    if (w >= a.mask_words) return;
    if (a.causal && 32 * w > i) return;
    if (a.window > 0 && i - (32 * w + 31) >= a.window) return;
    const uint64_t row_base = ((uint64_t)bh * a.sq + (uint64_t)i) * (uint64_t)a.sk;
    uint32_t word = 0;
#pragma unroll
    for (int blk = 0; blk < 8; ++blk) {
        const int key0 = 32 * w + 4 * blk;
        if (key0 < a.sk) {
            const uint64_t e0 = row_base + (uint64_t)key0;
            if constexpr (kExact)
                word |= dropout_keep_any(a.rng, e0, min(4, a.sk - key0)) << (4 * blk);
            else
                word |= dropout_keep4_pow2(a.rng, e0 >> 2) << (4 * blk);
        }
    }
    a.keep_mask[((int64_t)bh * a.mask_words + w) * a.mask_pitch + i] = word;
}

// (grid limits of keep_mask_kernel: one grid row per word of 32 keys, one grid plane per head)
bool keep_mask_kernel_fits(const AttnArgs& a) {
    return a.mask_words <= 65535 && (int64_t)a.batch * a.heads <= 65535;
}
int draw_keep_mask(const AttnArgs& a, hipStream_t st) {
    const int64_t bh = (int64_t)a.batch * a.heads;
    if (!keep_mask_kernel_fits(a)) return SLAPO_ERR_SHAPE;
    // with a window: the words of a row's own window (it spans window / 32 + 1 words at most)
    const int words = a.window > 0 ? min(a.mask_words, a.window / 32 + 2) : a.mask_words;
    const dim3 grid((unsigned)((a.sq + 255) / 256), (unsigned)words, (unsigned)bh);
    if (a.dropout == 1)
        hipLaunchKernelGGL(keep_mask_kernel<false>, grid, dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL(keep_mask_kernel<true>, grid, dim3(256), 0, st, a);
    return check_launch();
}

// Compute units of the current device (0 if the runtime will not say), asked once per device.
int cus_of_current_device() {
    static std::atomic<int> known[64];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    int n = known[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
            return 0;
        known[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

bool strides_ok(const int64_t s[3], int mult) {
    return s[0] % mult == 0 && s[1] % mult == 0 && s[2] % mult == 0;
}

int fill_args(const slapo_attn_params* p, AttnArgs* a, bool backward) {
    if (!p) return SLAPO_ERR_ARG;
    if (p->batch <= 0 || p->heads <= 0 || p->seqlen_q <= 0 || p->seqlen_k <= 0 ||
        p->head_dim <= 0)
        return SLAPO_ERR_SHAPE;
    if (p->head_dim > 128) return SLAPO_ERR_SHAPE;
    if ((int64_t)p->batch * p->heads > 0x7FFFFFFF / 2) return SLAPO_ERR_SHAPE;
    if (!(p->p_drop >= 0.f && p->p_drop <= 1.f)) return SLAPO_ERR_ARG;
    if (p->window < 0) return SLAPO_ERR_ARG;
    // the scale is folded into Q / K fragments: a NaN or infinite one would poison every score
    if (!(p->scale > -kFltMax && p->scale < kFltMax)) return SLAPO_ERR_ARG;
    const bool half = p->dtype == SLAPO_F16 || p->dtype == SLAPO_BF16;
    if (!half && p->dtype != SLAPO_F32) return SLAPO_ERR_DTYPE;
    if (half) {
        if (p->head_dim % 8 != 0) return SLAPO_ERR_SHAPE;
        if (!strides_ok(p->q_strides, 8) || !strides_ok(p->k_strides, 8) ||
            !strides_ok(p->v_strides, 8) || !strides_ok(p->o_strides, 8))
            return SLAPO_ERR_ALIGN;
        // the tile loads address rows with 32-bit byte offsets from a per-tile base
        for (const int64_t* st : {p->q_strides, p->k_strides, p->v_strides, p->o_strides})
            if (st[1] < 0 || st[1] >= (int64_t(1) << 24)) return SLAPO_ERR_SHAPE;
    }
    for (int i = 0; i < 3; ++i) {
        a->qs[i] = p->q_strides[i];
        a->ks[i] = p->k_strides[i];
        a->vs[i] = p->v_strides[i];
        a->os[i] = p->o_strides[i];
    }
    for (int i = 0; i < 4; ++i) a->bs[i] = p->bias_strides[i];
    a->batch = p->batch;
    a->heads = p->heads;
    a->sq = p->seqlen_q;
    a->sk = p->seqlen_k;
    a->d = p->head_dim;
    a->causal = p->causal ? 1 : 0;
    a->window = p->window;
    a->scale = p->scale;
    a->scale_log2 = p->scale * kLog2e;
    a->dropout = p->p_drop > 0.f ? 1 : 0;
    if (a->dropout) {
        const int64_t numel = (int64_t)p->batch * p->heads * p->seqlen_q * p->seqlen_k;
        if (!plan_ok(&p->plan, numel)) return SLAPO_ERR_ARG;
        a->rng = make_dropout_state(p->plan, (double)p->p_drop, p->seed, p->offset);
        if (!(a->rng.g_shift >= 0 && a->rng.t_shift >= 0 && p->seqlen_k % 4 == 0)) a->dropout = 2;
    } else {
        a->rng = DropoutState{};
    }
    a->snake_len = 0, a->snake_rows = 0;
    a->n_cus = half ? cus_of_current_device() : 0;
    a->keep_mask = nullptr;
    a->mask_words = (p->seqlen_k + 31) / 32;
    a->mask_pitch = (p->seqlen_q + 3) & ~3;
    if (a->dropout && half && p->keep_mask) {
        if (!aligned16(p->keep_mask)) return SLAPO_ERR_ALIGN;
        a->keep_mask = reinterpret_cast<uint32_t*>(p->keep_mask);
        if (backward) a->dropout = 3;
    }
    return SLAPO_OK;
}

void set_bias(AttnArgs* a, const float* bias) {
    a->bias = bias;
    a->has_bias = bias ? 1 : 0;
    a->bias_vec4 = 0;
    if (bias && a->bs[3] == 1 && aligned16(bias) && a->bs[0] % 4 == 0 && a->bs[1] % 4 == 0 &&
        a->bs[2] % 4 == 0)
        a->bias_vec4 = 1;
}

bool half_ptrs_ok(std::initializer_list<const void*> ptrs) {
    for (const void* p : ptrs)
        if (!p || !aligned16(p)) return false;
    return true;
}

}  // namespace


extern "C" size_t slapo_amd_attn_keep_mask_bytes(const slapo_attn_params* p) {
    if (!p || !(p->p_drop > 0.f) || (p->dtype != SLAPO_F16 && p->dtype != SLAPO_BF16)) return 0;
    if (p->batch <= 0 || p->heads <= 0 || p->seqlen_q <= 0 || p->seqlen_k <= 0) return 0;
    const size_t words = (size_t)((p->seqlen_k + 31) / 32) * (size_t)((p->seqlen_q + 3) & ~3);
    return (size_t)p->batch * p->heads * words * sizeof(uint32_t);
}

extern "C" int slapo_amd_attn_fwd(const slapo_attn_params* prm, const void* q, const void* k,
                                  const void* v, const float* bias, void* o, float* lse,
                                  void* stream) {
    AttnArgs a = {};
    int rc = fill_args(prm, &a, false);
    if (rc != SLAPO_OK) return rc;
    if (!q || !k || !v || !o || !lse) return SLAPO_ERR_ARG;
    a.q = q, a.k = k, a.v = v, a.o = o, a.lse = lse;
    set_bias(&a, bias);
    hipStream_t st = (hipStream_t)stream;
    if (prm->dtype == SLAPO_F32) return attn_fwd_f32(a, st);
    if (!half_ptrs_ok({q, k, v, o})) return SLAPO_ERR_ALIGN;
    if (a.dropout && a.keep_mask && a.window > 0 && keep_mask_kernel_fits(a)) {
        // Local window with a buffer for the keep bits: draw them first, the forward kernel
        // then reads them like the backward kernels do (bf16 B4 S2048 H16 D128, window 256,
        // p 0.1: 88 against 127 us).  Without a window the forward draws them itself and
        // stores them as it goes: there the Philox arithmetic overlaps the matrix instructions
        // and a separate pass measured slower (239 against 199 us at the same shape, 116
        // against 87 us at fp16 B8 S1024 H16 D64).
        rc = draw_keep_mask(a, st);
        if (rc != SLAPO_OK) return rc;
        a.dropout = 3;
    }
    return prm->dtype == SLAPO_F16 ? attn_fwd_mfma_f16(a, st) : attn_fwd_mfma_bf16(a, st);
}

extern "C" size_t slapo_amd_attn_bwd_workspace_bytes(const slapo_attn_params* prm) {
    if (!prm || prm->batch <= 0 || prm->heads <= 0 || prm->seqlen_q <= 0 || prm->head_dim <= 0)
        return 0;
    const size_t rows = (size_t)prm->batch * prm->heads * prm->seqlen_q;
    return rows * sizeof(float);  // delta
}

extern "C" int slapo_amd_attn_bwd_stages(const slapo_attn_params* prm, const void* q,
                                         const void* k, const void* v, const float* bias,
                                         const void* o, const void* dout, const float* lse,
                                         void* dq, void* dk, void* dv,
                                         const int64_t dq_strides[3], const int64_t dk_strides[3],
                                         const int64_t dv_strides[3], void* workspace,
                                         size_t workspace_bytes, int stages, void* stream) {
    AttnArgs a = {};
    int rc = fill_args(prm, &a, true);
    if (rc != SLAPO_OK) return rc;
    if (!q || !k || !v || !o || !dout || !lse || !dq || !dk || !dv || !dq_strides ||
        !dk_strides || !dv_strides)
        return SLAPO_ERR_ARG;
    if (stages <= 0 || stages > SLAPO_BWD_ALL) return SLAPO_ERR_ARG;
    if (!workspace || workspace_bytes < slapo_amd_attn_bwd_workspace_bytes(prm) ||
        !aligned16(workspace))
        return SLAPO_ERR_WORKSPACE;
    for (int i = 0; i < 3; ++i) {
        a.dqs[i] = dq_strides[i];
        a.dks[i] = dk_strides[i];
        a.dvs[i] = dv_strides[i];
    }
    a.q = q, a.k = k, a.v = v, a.o = const_cast<void*>(o), a.dout = dout;
    a.lse = const_cast<float*>(lse);
    a.dk = dk, a.dv = dv;
    set_bias(&a, bias);
    hipStream_t st = (hipStream_t)stream;

    const int64_t rows = (int64_t)a.batch * a.heads * a.sq;
    const bool is_f32 = prm->dtype == SLAPO_F32;
    a.delta = reinterpret_cast<float*>(workspace);
    a.dq = dq;

    if (is_f32) {
        if (stages & SLAPO_BWD_PREPARE) {
            const bool vec_ok = a.d % 4 == 0 && aligned16(o) && aligned16(dout) &&
                                strides_ok(prm->o_strides, 4);
            if (vec_ok) {
                const unsigned blocks = (unsigned)((rows * 8 + 255) / 256);
                hipLaunchKernelGGL((attn_delta_kernel<float>), dim3(blocks), dim3(256), 0, st, a);
            } else {
                const unsigned blocks = (unsigned)((rows + 255) / 256);
                hipLaunchKernelGGL(attn_delta_scalar_kernel, dim3(blocks), dim3(256), 0, st, a);
            }
            rc = check_launch();
            if (rc != SLAPO_OK) return rc;
        }
        if (stages & SLAPO_BWD_DKDV) rc = attn_bwd_f32(a, st);
        return rc;
    }

    if (!half_ptrs_ok({q, k, v, o, dout, dq, dk, dv})) return SLAPO_ERR_ALIGN;
    if (!strides_ok(dq_strides, 8) || !strides_ok(dk_strides, 8) || !strides_ok(dv_strides, 8))
        return SLAPO_ERR_ALIGN;

    // 16-bit types: PREPARE has nothing to do (the dQ kernel computes delta for its own rows and
    // stores it for the dK / dV kernel), so DQ runs before DKDV.
    if (stages & SLAPO_BWD_DQ) {
        rc = prm->dtype == SLAPO_F16 ? attn_bwd_dq_mfma_f16(a, st) : attn_bwd_dq_mfma_bf16(a, st);
        if (rc != SLAPO_OK) return rc;
    }
    if (stages & SLAPO_BWD_DKDV) {
        rc = prm->dtype == SLAPO_F16 ? attn_bwd_mfma_f16(a, st) : attn_bwd_mfma_bf16(a, st);
    }
    return rc;
}

extern "C" int slapo_amd_attn_bwd(const slapo_attn_params* prm, const void* q, const void* k,
                                  const void* v, const float* bias, const void* o,
                                  const void* dout, const float* lse, void* dq, void* dk,
                                  void* dv, const int64_t dq_strides[3],
                                  const int64_t dk_strides[3], const int64_t dv_strides[3],
                                  void* workspace, size_t workspace_bytes, void* stream) {
    return slapo_amd_attn_bwd_stages(prm, q, k, v, bias, o, dout, lse, dq, dk, dv, dq_strides,
                                     dk_strides, dv_strides, workspace, workspace_bytes,
                                     SLAPO_BWD_ALL, stream);
}

// ---- backward without a caller workspace -------------------------------------------------------
// delta = rowsum(dO * O) lives in an array of the library's own, so that callers that must not
// allocate (HIP graph capture, serving loops) need no workspace: every device that runs the
// library holds one copy of the array until the process ends.
namespace {

constexpr size_t kScratchFloats = size_t(1) << 20;  // 4 MiB: batch * heads * seqlen_q <= 1 048 576
__device__ __align__(256) float scratch[kScratchFloats];

std::mutex scratch_lock;
float* scratch_of_device[64] = {};  // device address of `scratch`, per device, once resolved

// The array's name is only a handle on the host; its address on the current device comes from
// the runtime, once per device.
int scratch_on_current_device(float** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return SLAPO_ERR_DEVICE;
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_of_device[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p)
            return SLAPO_ERR_DEVICE;
        scratch_of_device[dev] = static_cast<float*>(p);
    }
    *out = scratch_of_device[dev];
    return SLAPO_OK;
}

}  // namespace

extern "C" int slapo_amd_attn_bwd_static_scratch(
    const slapo_attn_params* prm, const void* q, const void* k, const void* v, const float* bias,
    const void* o, const void* dout, const float* lse, void* dq, void* dk, void* dv,
    const int64_t dq_strides[3], const int64_t dk_strides[3], const int64_t dv_strides[3],
    void* stream) {
    const size_t need = slapo_amd_attn_bwd_workspace_bytes(prm);
    if (need == 0) return SLAPO_ERR_SHAPE;
    if (need > kScratchFloats * sizeof(float)) return SLAPO_ERR_WORKSPACE;
    float* ws = nullptr;
    const int rc = scratch_on_current_device(&ws);
    if (rc != SLAPO_OK) return rc;
    return slapo_amd_attn_bwd_stages(prm, q, k, v, bias, o, dout, lse, dq, dk, dv, dq_strides,
                                     dk_strides, dv_strides, ws, kScratchFloats * sizeof(float),
                                     SLAPO_BWD_ALL, stream);
}
