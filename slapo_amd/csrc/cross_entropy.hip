// Vocab-parallel cross entropy, the part that one GPU computes on its shard of the vocabulary
// (slapo/op/cross_entropy.py:17-124, Megatron's _VocabParallelCrossEntropy).
//
// The reference reads the [tokens, vocab/p] logits for the maximum, again for exp / sum, keeps the
// softmax in their place and touches it three more times in the backward.  Here the forward is
// one read: every row leaves as four fp32 numbers -- its local maximum m, s = sum exp(x - m)
// relative to that maximum, the raw logit of the target if the target lies in this shard, and
// sum x (label smoothing) -- which is exactly what the tensor-parallel group has to combine:
//     M = max_r m_r,  S = sum_r s_r exp(m_r - M),  predicted = sum_r predicted_r,
//     loss = log S + M - predicted.
// The backward recomputes the softmax from the logits and (M, 1/S): one read, one write, and no
// softmax tensor kept between the passes.
//
// Both kernels are HBM-bound streams: one block per row, 128-bit accesses on the 16-byte aligned
// body of the row (rows of an unpadded vocabulary such as 50257 start at any 2- or 4-byte
// offset, so each row is peeled into head / aligned body / tail), fp32 math.
#include "common.h"

using namespace slapo;

namespace {

// Threads per block (= per row).  Long rows take larger blocks: at 8192 x 50257 fp16 the forward
// measured 130 / 123.5 / 147 us with 256 / 512 / 1024 threads (its block reduction grows with the
// block) and the backward, which only streams, 307 / 293 / 279 us.
constexpr int kCeMaxThreads = 1024;
constexpr int kCeAlign = 128;  // bytes: alignment of a row's vector body

// (m, s) pairs combine as  m = max(m1, m2),  s = s1 exp(m1 - m) + s2 exp(m2 - m); an empty
// partner is (-inf, 0).
__device__ __forceinline__ void ce_merge(float& m, float& s, float m2, float s2) {
    const float mn = fmaxf(m, m2);
    if (mn == -INFINITY) return;  // both empty
    s = s * __builtin_amdgcn_exp2f((m - mn) * 1.4426950408889634f) +
        s2 * __builtin_amdgcn_exp2f((m2 - mn) * 1.4426950408889634f);
    m = mn;
}

template <typename T>
struct RowSplit {
    int head;   // scalar elements before the first kCeAlign-byte boundary
    int nvec;   // 16-byte vectors in the aligned body
    int tail0;  // first element of the scalar tail
};

template <typename T, int V>
__device__ __forceinline__ RowSplit<T> split_row(const T* row, int n) {
    RowSplit<T> r;
    if constexpr (V == 1) {
        r.head = 0, r.nvec = n, r.tail0 = n;
    } else {
        // The vector body starts on a cache line, not just on a 16-byte boundary: a wavefront's
        // 1 KB access then covers whole lines (rows of an odd vocabulary start anywhere; with
        // 16-byte alignment only, the backward ran at 4.6 TB/s instead of 5.4 and the forward at
        // 6.2 instead of 6.5 at 8192 x 50257 fp16).  The head is at most 63 elements.
        constexpr int kPer = kCeAlign / (int)sizeof(T);
        static_assert(kPer <= 256, "one thread per head element (smallest block)");
        const int mis = (int)((reinterpret_cast<uintptr_t>(row) & (kCeAlign - 1)) / sizeof(T));
        r.head = min(n, mis ? kPer - mis : 0);
        r.nvec = (n - r.head) / V;
        r.tail0 = r.head + r.nvec * V;
    }
    return r;
}

template <typename T, int V>
struct CeVec {
    T v[V];
};

// Forward: m[row], s[row], predicted[row], sum_x[row] of one shard.  target may be any integer;
// it counts when vocab_start <= target < vocab_start + n.
template <typename T, int V, int kCeThreads>
__global__ __launch_bounds__(kCeThreads) void ce_fwd_kernel(
    const T* __restrict__ logits, const int64_t* __restrict__ target, float* __restrict__ m_out,
    float* __restrict__ s_out, float* __restrict__ pred_out, float* __restrict__ sumx_out, int n,
    int64_t vocab_start) {
    const int64_t row = blockIdx.x;
    const T* x = logits + row * (int64_t)n;
    const RowSplit<T> sp = split_row<T, V>(x, n);
    float m = -INFINITY, s = 0.f, sx = 0.f;
    auto add1 = [&](float v) __attribute__((always_inline)) {
        sx += v;
        ce_merge(m, s, v, 1.0f);
    };
    if ((int)threadIdx.x < sp.head) add1(Elem<T>::to_f32(x[threadIdx.x]));
    for (int e = sp.tail0 + threadIdx.x; e < n; e += kCeThreads) add1(Elem<T>::to_f32(x[e]));
    const T* body = x + sp.head;
    auto load_vec = [&](int i) __attribute__((always_inline)) -> CeVec<T, V> {
        CeVec<T, V> c;
        if constexpr (V == 1) {
            c.v[0] = body[i];
        } else {
            *reinterpret_cast<u32x4_t*>(&c) =
                __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(body) + i);
        }
        return c;
    };
    auto take_vec = [&](const CeVec<T, V>& c) __attribute__((always_inline)) {
        float f[V];
        float vm = -INFINITY;
#pragma unroll
        for (int j = 0; j < V; ++j) {
            f[j] = Elem<T>::to_f32(c.v[j]);
            vm = fmaxf(vm, f[j]);
            sx += f[j];
        }
        // rescale the running sum only when the maximum moves
        const float mn = fmaxf(m, vm);
        if (mn > m) {
            s *= __builtin_amdgcn_exp2f((m - mn) * 1.4426950408889634f);  // exp2(-inf) = 0
            m = mn;
        }
        if (m != -INFINITY) {
#pragma unroll
            for (int j = 0; j < V; ++j)
                s += __builtin_amdgcn_exp2f((f[j] - m) * 1.4426950408889634f);
        }
    };
    // four loads in flight per thread
    int i = threadIdx.x;
    for (; i + 3 * kCeThreads < sp.nvec; i += 4 * kCeThreads) {
        CeVec<T, V> c[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) c[u] = load_vec(i + u * kCeThreads);
#pragma unroll
        for (int u = 0; u < 4; ++u) take_vec(c[u]);
    }
    for (; i < sp.nvec; i += kCeThreads) take_vec(load_vec(i));
    // block reduction: butterflies inside the wavefront, then the block's wavefronts through LDS
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float m2 = __shfl_xor(m, off, 64);
        const float s2 = __shfl_xor(s, off, 64);
        sx += __shfl_xor(sx, off, 64);
        ce_merge(m, s, m2, s2);
    }
    __shared__ float red[3][kCeThreads / 64];
    if ((threadIdx.x & 63) == 0) {
        red[0][threadIdx.x >> 6] = m;
        red[1][threadIdx.x >> 6] = s;
        red[2][threadIdx.x >> 6] = sx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float mm = red[0][0], ss = red[1][0], xx = red[2][0];
#pragma unroll
        for (int w = 1; w < kCeThreads / 64; ++w) {
            ce_merge(mm, ss, red[0][w], red[1][w]);
            xx += red[2][w];
        }
        m_out[row] = mm;
        s_out[row] = ss;
        sumx_out[row] = xx;
        const int64_t t = target[row] - vocab_start;
        pred_out[row] = (t >= 0 && t < n) ? Elem<T>::to_f32(x[t]) : 0.f;
    }
}

// Backward: grad[row, v] = g[row] (exp(x - M[row]) inv_s[row] - onehot_scale [v == target] - flat)
// with M, inv_s the combined maximum and 1 / sum of the whole vocabulary, onehot_scale =
// 1 - smoothing and flat = smoothing / n (slapo/op/cross_entropy.py:100-122).
template <typename T, int V, int kCeThreads>
__global__ __launch_bounds__(kCeThreads) void ce_bwd_kernel(
    const T* __restrict__ logits, const int64_t* __restrict__ target,
    const float* __restrict__ row_max, const float* __restrict__ inv_sum,
    const float* __restrict__ grad_loss, T* __restrict__ grad, int n, int64_t vocab_start,
    float onehot_scale, float flat) {
    const int64_t row = blockIdx.x;
    const T* x = logits + row * (int64_t)n;
    T* dx = grad + row * (int64_t)n;
    const RowSplit<T> sp = split_row<T, V>(x, n);
    const float mx = row_max[row];
    const float g = grad_loss[row];
    const float isg = inv_sum[row] * g;
    const float flatg = flat * g;
    // (softmax - flat) g; the target's element is corrected after the stream, so that the loop
    // carries no comparison.  v - max first: exact for logits near the maximum even when both
    // sit far from zero.
    auto one = [&](float v) __attribute__((always_inline)) -> float {
        return __builtin_fmaf(__builtin_amdgcn_exp2f((v - mx) * 1.4426950408889634f), isg, -flatg);
    };
    if ((int)threadIdx.x < sp.head)
        dx[threadIdx.x] = Elem<T>::from_f32(one(Elem<T>::to_f32(x[threadIdx.x])));
    for (int e = sp.tail0 + threadIdx.x; e < n; e += kCeThreads)
        dx[e] = Elem<T>::from_f32(one(Elem<T>::to_f32(x[e])));
    const T* body = x + sp.head;
    T* obody = dx + sp.head;
    auto load_vec = [&](int i) __attribute__((always_inline)) -> CeVec<T, V> {
        CeVec<T, V> c;
        if constexpr (V == 1) {
            c.v[0] = body[i];
        } else {
            *reinterpret_cast<u32x4_t*>(&c) =
                __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(body) + i);
        }
        return c;
    };
    auto emit_vec = [&](int i, const CeVec<T, V>& c) __attribute__((always_inline)) {
        CeVec<T, V> o;
#pragma unroll
        for (int j = 0; j < V; ++j) o.v[j] = Elem<T>::from_f32(one(Elem<T>::to_f32(c.v[j])));
        if constexpr (V == 1) {
            obody[i] = o.v[0];
        } else {
            __builtin_nontemporal_store(*reinterpret_cast<const u32x4_t*>(&o),
                                        reinterpret_cast<u32x4_t*>(obody) + i);
        }
    };
    // four loads in flight per thread
    int i = threadIdx.x;
    for (; i + 3 * kCeThreads < sp.nvec; i += 4 * kCeThreads) {
        CeVec<T, V> c[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) c[u] = load_vec(i + u * kCeThreads);
#pragma unroll
        for (int u = 0; u < 4; ++u) emit_vec(i + u * kCeThreads, c[u]);
    }
    for (; i < sp.nvec; i += kCeThreads) emit_vec(i, load_vec(i));
    // the one-hot term of the target, if it lies in this shard: written after every thread of
    // the block has stored its part of the row
    const int64_t t64 = target[row] - vocab_start;
    __syncthreads();
    if (threadIdx.x == 0 && t64 >= 0 && t64 < n)
        dx[t64] = Elem<T>::from_f32(one(Elem<T>::to_f32(x[t64])) - onehot_scale * g);
}

inline bool ce_dims_ok(int64_t rows, int64_t n) {
    return rows > 0 && n > 0 && rows <= 0x7FFFFFFF && n <= 0x7FFFFFFF;
}

template <typename T>
int ce_fwd_dispatch(const void* logits, const int64_t* target, float* m, float* s, float* pred,
                    float* sumx, int64_t rows, int64_t n, int64_t vocab_start, hipStream_t st) {
#define SLAPO_CE_FWD(THREADS)                                                                   \
    hipLaunchKernelGGL((ce_fwd_kernel<T, Elem<T>::kPerVec, THREADS>), dim3((unsigned)rows),     \
                       dim3(THREADS), 0, st, (const T*)logits, target, m, s, pred, sumx, (int)n, \
                       vocab_start)
    if (n >= 16384)
        SLAPO_CE_FWD(512);
    else
        SLAPO_CE_FWD(256);
#undef SLAPO_CE_FWD
    return check_launch();
}

template <typename T>
int ce_bwd_dispatch(const void* logits, const int64_t* target, const float* row_max,
                    const float* inv_sum, const float* grad_loss, void* grad, int64_t rows,
                    int64_t n, int64_t vocab_start, float onehot_scale, float flat,
                    hipStream_t st) {
    // Rows of logits and grad share their misalignment when the two bases are congruent mod 16;
    // otherwise every element goes through the scalar path.
    const bool same = ((reinterpret_cast<uintptr_t>(logits) ^ reinterpret_cast<uintptr_t>(grad)) &
                       15) == 0;
#define SLAPO_CE_BWD(VEC, THREADS)                                                              \
    hipLaunchKernelGGL((ce_bwd_kernel<T, VEC, THREADS>), dim3((unsigned)rows), dim3(THREADS), 0, \
                       st, (const T*)logits, target, row_max, inv_sum, grad_loss, (T*)grad,      \
                       (int)n, vocab_start, onehot_scale, flat)
    if (!same)
        SLAPO_CE_BWD(1, 256);
    else if (n >= 32768)
        SLAPO_CE_BWD(Elem<T>::kPerVec, kCeMaxThreads);
    else if (n >= 8192)
        SLAPO_CE_BWD(Elem<T>::kPerVec, 512);
    else
        SLAPO_CE_BWD(Elem<T>::kPerVec, 256);
#undef SLAPO_CE_BWD
    return check_launch();
}

}  // namespace

extern "C" int slapo_amd_vocab_ce_fwd(const void* logits, const int64_t* target, float* row_max,
                                      float* sum_exp, float* predicted, float* sum_logits,
                                      int64_t rows, int64_t vocab, int64_t vocab_start, int dtype,
                                      void* stream) {
    if (!logits || !target || !row_max || !sum_exp || !predicted || !sum_logits)
        return SLAPO_ERR_ARG;
    if (!ce_dims_ok(rows, vocab)) return SLAPO_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case SLAPO_F32:
            if (reinterpret_cast<uintptr_t>(logits) & 3) return SLAPO_ERR_ALIGN;
            return ce_fwd_dispatch<float>(logits, target, row_max, sum_exp, predicted, sum_logits,
                                          rows, vocab, vocab_start, st);
        case SLAPO_F16:
            if (reinterpret_cast<uintptr_t>(logits) & 1) return SLAPO_ERR_ALIGN;
            return ce_fwd_dispatch<f16_t>(logits, target, row_max, sum_exp, predicted, sum_logits,
                                          rows, vocab, vocab_start, st);
        case SLAPO_BF16:
            if (reinterpret_cast<uintptr_t>(logits) & 1) return SLAPO_ERR_ALIGN;
            return ce_fwd_dispatch<bf16_t>(logits, target, row_max, sum_exp, predicted,
                                           sum_logits, rows, vocab, vocab_start, st);
        default:
            return SLAPO_ERR_DTYPE;
    }
}

extern "C" int slapo_amd_vocab_ce_bwd(const void* logits, const int64_t* target,
                                      const float* row_max, const float* inv_sum_exp,
                                      const float* grad_loss, void* grad_logits, int64_t rows,
                                      int64_t vocab, int64_t vocab_start, double label_smoothing,
                                      int dtype, void* stream) {
    if (!logits || !target || !row_max || !inv_sum_exp || !grad_loss || !grad_logits)
        return SLAPO_ERR_ARG;
    if (!ce_dims_ok(rows, vocab)) return SLAPO_ERR_SHAPE;
    if (!(label_smoothing >= 0.0 && label_smoothing < 1.0)) return SLAPO_ERR_ARG;
    if (label_smoothing > 0.0 && vocab < 2) return SLAPO_ERR_SHAPE;
    // slapo/op/cross_entropy.py:112-116: smoothing = alpha K / (K - 1) with K the shard's size
    const double smoothing =
        label_smoothing > 0.0 ? label_smoothing * (double)vocab / (double)(vocab - 1) : 0.0;
    const float onehot_scale = (float)(1.0 - smoothing);
    const float flat = (float)(smoothing / (double)vocab);
    hipStream_t st = (hipStream_t)stream;
#define CALL(T)                                                                                \
    ce_bwd_dispatch<T>(logits, target, row_max, inv_sum_exp, grad_loss, grad_logits, rows, vocab, \
                       vocab_start, onehot_scale, flat, st)
    switch (dtype) {
        case SLAPO_F32: return CALL(float);
        case SLAPO_F16: return CALL(f16_t);
        case SLAPO_BF16: return CALL(bf16_t);
        default: return SLAPO_ERR_DTYPE;
    }
#undef CALL
}
