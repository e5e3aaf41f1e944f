// Attention forward and backward with fp32 arithmetic throughout (plain FMA, no MFMA): the
// kernels behind dtype == SLAPO_F32, where the parity bar is 1e-5 absolute and reduced-precision
// matrix inputs are not an option.  One thread owns one row (a query in forward and dQ, a key in
// dK / dV) and keeps its row vectors in registers; the other operand streams through LDS in small
// tiles that every thread of the wavefront reads at the same address (broadcast, conflict free).
// They are written for exactness and generality, not speed.
//
// Reference semantics: slapo/op/attention.py:163-181 (attention_bmk) and its autograd.
#include "attn_common.h"

using namespace slapo;

namespace {

constexpr int kRows = 64;   // threads (= owned rows) per block
constexpr int kTile = 16;   // streamed rows per LDS tile

__device__ __forceinline__ float bias_at(const AttnArgs& a, int b, int h, int i, int j) {
    return canonical_bias(
        a.bias[b * a.bs[0] + h * a.bs[1] + (int64_t)i * a.bs[2] + (int64_t)j * a.bs[3]]);
}

__device__ __forceinline__ float drop_scale(const AttnArgs& a, int bh, int i, int j) {
    const uint64_t e = ((uint64_t)bh * a.sq + (uint64_t)i) * (uint64_t)a.sk + (uint64_t)j;
    return dropout_keep1(a.rng, e) ? a.rng.inv_keep : 0.f;
}

// Cooperative load of `kTile` rows x DMAX floats into LDS (zero padded).
template <int DMAX>
__device__ __forceinline__ void load_rows(float (*dst)[DMAX], const float* base, int64_t stride,
                                          int row0, int n_rows, int d) {
    for (int e = threadIdx.x; e < kTile * DMAX; e += kRows) {
        const int r = e / DMAX, c = e % DMAX;
        const int gr = row0 + r;
        dst[r][c] = (gr < n_rows && c < d) ? base[(int64_t)gr * stride + c] : 0.f;
    }
}

template <int DMAX>
__global__ __launch_bounds__(kRows) void attn_f32_fwd_kernel(const AttnArgs a_in) {
    AttnArgs a = a_in;
    if (a.dropout) resolve_device_state(a.rng);
    __shared__ float ks[kTile][DMAX];
    __shared__ float vs[kTile][DMAX];
    const int bh = blockIdx.y, b = bh / a.heads, h = bh % a.heads;
    const int q0 = blockIdx.x * kRows;
    const int i = q0 + threadIdx.x;
    const bool row_ok = i < a.sq;
    const float* qp = reinterpret_cast<const float*>(a.q) + b * a.qs[0] + h * a.qs[2];
    const float* kp = reinterpret_cast<const float*>(a.k) + b * a.ks[0] + h * a.ks[2];
    const float* vp = reinterpret_cast<const float*>(a.v) + b * a.vs[0] + h * a.vs[2];

    float q[DMAX], o[DMAX];
#pragma unroll
    for (int c = 0; c < DMAX; ++c) {
        q[c] = (row_ok && c < a.d) ? qp[(int64_t)i * a.qs[1] + c] * a.scale : 0.f;
        o[c] = 0.f;
    }
    float m = -INFINITY, l = 0.f;

    int j_lo, j_hi;
    key_range(a, q0, min(q0 + kRows, a.sq), j_lo, j_hi);
    for (int j0 = (j_lo / kTile) * kTile; j0 < j_hi; j0 += kTile) {
        __syncthreads();
        load_rows<DMAX>(ks, kp, a.ks[1], j0, a.sk, a.d);
        load_rows<DMAX>(vs, vp, a.vs[1], j0, a.sk, a.d);
        __syncthreads();
        if (!row_ok) continue;
        // One key at a time; the running maximum rarely moves after the first few keys, so the
        // rescale of the accumulator sits behind a branch.
#pragma unroll 1
        for (int jj = 0; jj < kTile; ++jj) {
            const int j = j0 + jj;
            if (!key_visible(a, i, j)) continue;
            float sc = 0.f;
#pragma unroll
            for (int c = 0; c < DMAX; ++c) sc = __builtin_fmaf(q[c], ks[jj][c], sc);
            if (a.has_bias) sc += bias_at(a, b, h, i, j);
            if (sc == -INFINITY) continue;
            if (sc > m) {
                const float alpha = expf(m - sc);
                m = sc;
                l *= alpha;
#pragma unroll
                for (int c = 0; c < DMAX; ++c) o[c] *= alpha;
            }
            float p = expf(sc - m);
            l += p;
            if (a.dropout) p *= drop_scale(a, bh, i, j);
#pragma unroll
            for (int c = 0; c < DMAX; ++c) o[c] = __builtin_fmaf(p, vs[jj][c], o[c]);
        }
    }
    if (!row_ok) return;
    const float inv_l = 1.0f / l;
    float* op = reinterpret_cast<float*>(a.o) + b * a.os[0] + (int64_t)i * a.os[1] + h * a.os[2];
#pragma unroll
    for (int c = 0; c < DMAX; ++c)
        if (c < a.d) op[c] = o[c] * inv_l;
    // a row that saw nothing but masked keys: see canonical_bias
    a.lse[(int64_t)bh * a.sq + i] = m == -kFltMax ? l * kMaskedRowLse : m + logf(l);
}

// dQ: thread = query.  dq_i = scale * sum_j ds_ij k_j,  ds = p (dp - delta),  dp = dO_i . v_j
template <int DMAX>
__global__ __launch_bounds__(kRows) void attn_f32_dq_kernel(const AttnArgs a_in) {
    AttnArgs a = a_in;
    if (a.dropout) resolve_device_state(a.rng);
    __shared__ float ks[kTile][DMAX];
    __shared__ float vs[kTile][DMAX];
    const int bh = blockIdx.y, b = bh / a.heads, h = bh % a.heads;
    const int q0 = blockIdx.x * kRows;
    const int i = q0 + threadIdx.x;
    const bool row_ok = i < a.sq;
    const float* qp = reinterpret_cast<const float*>(a.q) + b * a.qs[0] + h * a.qs[2];
    const float* kp = reinterpret_cast<const float*>(a.k) + b * a.ks[0] + h * a.ks[2];
    const float* vp = reinterpret_cast<const float*>(a.v) + b * a.vs[0] + h * a.vs[2];
    const float* gp = reinterpret_cast<const float*>(a.dout) + b * a.os[0] + h * a.os[2];

    float q[DMAX], go[DMAX], dq[DMAX];
#pragma unroll
    for (int c = 0; c < DMAX; ++c) {
        const bool ok = row_ok && c < a.d;
        q[c] = ok ? qp[(int64_t)i * a.qs[1] + c] * a.scale : 0.f;
        go[c] = ok ? gp[(int64_t)i * a.os[1] + c] : 0.f;
        dq[c] = 0.f;
    }
    const float lse_raw = row_ok ? a.lse[(int64_t)bh * a.sq + i] : 0.f;
    const float lse = lse_reference(lse_raw, 1.0f), inv_n = lse_row_factor(lse_raw);
    const float delta = row_ok ? a.delta[(int64_t)bh * a.sq + i] : 0.f;

    int j_lo, j_hi;
    key_range(a, q0, min(q0 + kRows, a.sq), j_lo, j_hi);
    for (int j0 = (j_lo / kTile) * kTile; j0 < j_hi; j0 += kTile) {
        __syncthreads();
        load_rows<DMAX>(ks, kp, a.ks[1], j0, a.sk, a.d);
        load_rows<DMAX>(vs, vp, a.vs[1], j0, a.sk, a.d);
        __syncthreads();
        if (!row_ok) continue;
#pragma unroll 1
        for (int jj = 0; jj < kTile; ++jj) {
            const int j = j0 + jj;
            if (!key_visible(a, i, j)) continue;
            float s = 0.f, dp = 0.f;
#pragma unroll
            for (int c = 0; c < DMAX; ++c) {
                s = __builtin_fmaf(q[c], ks[jj][c], s);
                dp = __builtin_fmaf(go[c], vs[jj][c], dp);
            }
            if (a.has_bias) s += bias_at(a, b, h, i, j);
            const float p = expf(s - lse) * inv_n;
            if (a.dropout) dp *= drop_scale(a, bh, i, j);
            const float ds = p * (dp - delta);
#pragma unroll
            for (int c = 0; c < DMAX; ++c) dq[c] = __builtin_fmaf(ds, ks[jj][c], dq[c]);
        }
    }
    if (!row_ok) return;
    float* dqp =
        reinterpret_cast<float*>(a.dq) + b * a.dqs[0] + (int64_t)i * a.dqs[1] + h * a.dqs[2];
#pragma unroll
    for (int c = 0; c < DMAX; ++c)
        if (c < a.d) dqp[c] = dq[c] * a.scale;
}

// dK (kWhich == 0) or dV (kWhich == 1): thread = key, queries stream through LDS.
//   dv_j = sum_i pdrop_ij dO_i          dk_j = scale * sum_i ds_ij q_i
template <int DMAX, int kWhich>
__global__ __launch_bounds__(kRows) void attn_f32_dkv_kernel(const AttnArgs a_in) {
    AttnArgs a = a_in;
    if (a.dropout) resolve_device_state(a.rng);
    __shared__ float qs[kTile][DMAX];
    __shared__ float gs[kTile][DMAX];
    __shared__ float lse_s[kTile], inv_n_s[kTile];
    __shared__ float delta_s[kTile];
    const int bh = blockIdx.y, b = bh / a.heads, h = bh % a.heads;
    const int k0 = blockIdx.x * kRows;
    const int j = k0 + threadIdx.x;
    const bool row_ok = j < a.sk;
    const float* qp = reinterpret_cast<const float*>(a.q) + b * a.qs[0] + h * a.qs[2];
    const float* kp = reinterpret_cast<const float*>(a.k) + b * a.ks[0] + h * a.ks[2];
    const float* vp = reinterpret_cast<const float*>(a.v) + b * a.vs[0] + h * a.vs[2];
    const float* gp = reinterpret_cast<const float*>(a.dout) + b * a.os[0] + h * a.os[2];

    float kr[DMAX], vr[kWhich == 0 ? DMAX : 1], acc[DMAX];
#pragma unroll
    for (int c = 0; c < DMAX; ++c) {
        const bool ok = row_ok && c < a.d;
        kr[c] = ok ? kp[(int64_t)j * a.ks[1] + c] * a.scale : 0.f;
        if (kWhich == 0) vr[c] = ok ? vp[(int64_t)j * a.vs[1] + c] : 0.f;
        acc[c] = 0.f;
    }

    int i_lo, i_hi;
    query_range(a, k0, min(k0 + kRows, a.sk), i_lo, i_hi);
    for (int i0 = (i_lo / kTile) * kTile; i0 < i_hi; i0 += kTile) {
        __syncthreads();
        load_rows<DMAX>(qs, qp, a.qs[1], i0, a.sq, a.d);
        load_rows<DMAX>(gs, gp, a.os[1], i0, a.sq, a.d);
        if (threadIdx.x < kTile) {
            const int i = i0 + threadIdx.x;
            const float lse_raw = i < a.sq ? a.lse[(int64_t)bh * a.sq + i] : 0.f;
            lse_s[threadIdx.x] = lse_reference(lse_raw, 1.0f);
            inv_n_s[threadIdx.x] = lse_row_factor(lse_raw);
            delta_s[threadIdx.x] = i < a.sq ? a.delta[(int64_t)bh * a.sq + i] : 0.f;
        }
        __syncthreads();
        if (!row_ok) continue;
#pragma unroll 1
        for (int ii = 0; ii < kTile; ++ii) {
            const int i = i0 + ii;
            if (i >= a.sq || !key_visible(a, i, j)) continue;
            float s = 0.f;
#pragma unroll
            for (int c = 0; c < DMAX; ++c) s = __builtin_fmaf(qs[ii][c], kr[c], s);
            if (a.has_bias) s += bias_at(a, b, h, i, j);
            const float p = expf(s - lse_s[ii]) * inv_n_s[ii];
            const float keep = a.dropout ? drop_scale(a, bh, i, j) : 1.f;
            if (kWhich == 1) {
                const float pd = p * keep;
#pragma unroll
                for (int c = 0; c < DMAX; ++c) acc[c] = __builtin_fmaf(pd, gs[ii][c], acc[c]);
            } else {
                float dp = 0.f;
#pragma unroll
                for (int c = 0; c < DMAX; ++c) dp = __builtin_fmaf(gs[ii][c], vr[c], dp);
                const float ds = p * (dp * keep - delta_s[ii]);
#pragma unroll
                for (int c = 0; c < DMAX; ++c) acc[c] = __builtin_fmaf(ds, qs[ii][c], acc[c]);
            }
        }
    }
    if (!row_ok) return;
    float* outp;
    if (kWhich == 0)
        outp = reinterpret_cast<float*>(a.dk) + b * a.dks[0] + (int64_t)j * a.dks[1] + h * a.dks[2];
    else
        outp = reinterpret_cast<float*>(a.dv) + b * a.dvs[0] + (int64_t)j * a.dvs[1] + h * a.dvs[2];
#pragma unroll
    for (int c = 0; c < DMAX; ++c)
        if (c < a.d) outp[c] = kWhich == 0 ? acc[c] * a.scale : acc[c];
}

template <int DMAX>
int launch_all_fwd(const AttnArgs& a, hipStream_t st) {
    dim3 grid((a.sq + kRows - 1) / kRows, a.batch * a.heads);
    hipLaunchKernelGGL((attn_f32_fwd_kernel<DMAX>), grid, dim3(kRows), 0, st, a);
    return check_launch();
}

template <int DMAX>
int launch_all_bwd(const AttnArgs& a, hipStream_t st) {
    dim3 gq((a.sq + kRows - 1) / kRows, a.batch * a.heads);
    dim3 gk((a.sk + kRows - 1) / kRows, a.batch * a.heads);
    hipLaunchKernelGGL((attn_f32_dq_kernel<DMAX>), gq, dim3(kRows), 0, st, a);
    hipLaunchKernelGGL((attn_f32_dkv_kernel<DMAX, 0>), gk, dim3(kRows), 0, st, a);
    hipLaunchKernelGGL((attn_f32_dkv_kernel<DMAX, 1>), gk, dim3(kRows), 0, st, a);
    return check_launch();
}

}  // namespace

namespace slapo {

int attn_fwd_f32(const AttnArgs& a, hipStream_t st) {
    if (a.batch * a.heads > 65535) return SLAPO_ERR_SHAPE;
    if (a.d <= 32) return launch_all_fwd<32>(a, st);
    if (a.d <= 64) return launch_all_fwd<64>(a, st);
    if (a.d <= 128) return launch_all_fwd<128>(a, st);
    return SLAPO_ERR_SHAPE;
}

int attn_bwd_f32(const AttnArgs& a, hipStream_t st) {
    if (a.batch * a.heads > 65535) return SLAPO_ERR_SHAPE;
    if (a.d <= 32) return launch_all_bwd<32>(a, st);
    if (a.d <= 64) return launch_all_bwd<64>(a, st);
    if (a.d <= 128) return launch_all_bwd<128>(a, st);
    return SLAPO_ERR_SHAPE;
}

}  // namespace slapo
