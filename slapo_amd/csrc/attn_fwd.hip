// Flash-attention forward for gfx950, fp16 / bf16 inputs, fp32 softmax and accumulation.
//
// One workgroup (4 wavefronts) owns 128 consecutive queries of one (batch, head); wavefront w
// owns 32 of them.  Keys/values stream through LDS in tiles of 64 (double buffered, staged
// through registers so the next tile's global loads overlap the current tile's math).
//
// Per tile and wavefront, with lane l, i = l % 32, g = l / 32:
//   S^T = K Q^T      2 x (DPAD/16) MFMA 32x32x16; A = K rows from LDS (row-permuted, 128-bit
//                    reads), B = Q^T fragments held in registers for the whole kernel.
//                    Lane l then holds scores of ONE query (i) against 32 keys, so the row max
//                    and row sum are in-lane reductions plus one exchange with lane l ^ 32,
//                    and m, l, alpha are per-lane scalars.
//   P^T              exp2 of the scaled scores; thanks to the row permutation the accumulator
//                    registers are, in order, the k-slots of the B operand of the next MFMA:
//                    no shuffle, no LDS round trip for P.
//   O^T += V^T P^T   4 x (DPAD/32) MFMA; A = V^T fragments read from the row-major V tile with
//                    the LDS transpose read.
// Masks (causal, local window, key tail) are index arithmetic applied only on tiles that need
// it; an additive bias is broadcast in-kernel; dropout bits are regenerated from Philox in the
// element order of the dense [B*H, Sq, Sk] tensor (4 consecutive keys = one Philox block).
//
// Reference semantics: slapo/op/attention.py:163-181 (attention_bmk), :97-131 (flash_attn_ref).
#include "attn_common.h"

using namespace slapo;

namespace {

constexpr int kFwdWaves = 4;
constexpr int kFwdThreads = kFwdWaves * 64;
constexpr int kFwdBM = kFwdWaves * 32;
constexpr int kFwdBN = 64;

template <typename T, int DPAD>
__global__ __launch_bounds__(kFwdThreads, 2) void attn_fwd_kernel(const AttnArgs a) {
    typedef typename Mma<T>::frag frag_t;
    typedef TileStage<T, DPAD, kFwdBN, kFwdThreads> Stage;
    constexpr int kPitch = Stage::kPitch;
    constexpr int kTileElems = kFwdBN * kPitch;
    constexpr int DK = DPAD / 16;  // k-steps of S^T = K Q^T
    constexpr int DV = DPAD / 32;  // 32-row blocks of O^T

    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    // layout: K[2][tile], V[2][tile]
    T* k_lds = smem;
    T* v_lds = smem + 2 * kTileElems;

    const int n_bh = a.batch * a.heads;
    const int n_qt = (a.sq + kFwdBM - 1) / kFwdBM;
    const int bh = blockIdx.x % n_bh;
    const int qt = n_qt - 1 - blockIdx.x / n_bh;  // heaviest (latest) query tiles first
    const int b = bh / a.heads;
    const int h = bh % a.heads;
    const int q0 = qt * kFwdBM;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int g = lane >> 5;
    const int i_loc = lane & 31;
    const int wq0 = q0 + wave * 32;  // first query of this wavefront
    const int q_row = wq0 + i_loc;

    const T* q_base = reinterpret_cast<const T*>(a.q) + b * a.qs[0] + h * a.qs[2];
    const T* k_base = reinterpret_cast<const T*>(a.k) + b * a.ks[0] + h * a.ks[2];
    const T* v_base = reinterpret_cast<const T*>(a.v) + b * a.vs[0] + h * a.vs[2];

    // Q^T fragments: column i = this lane's query, k-slots = 8 consecutive head-dim elements.
    frag_t qf[DK];
#pragma unroll
    for (int t = 0; t < DK; ++t) {
        u32x4_t v = {0u, 0u, 0u, 0u};
        const int d0 = 16 * t + 8 * g;
        if (q_row < a.sq && d0 < a.d)
            v = *reinterpret_cast<const u32x4_t*>(q_base + (int64_t)q_row * a.qs[1] + d0);
        qf[t] = __builtin_bit_cast(frag_t, v);
    }

    f32x16_t o_acc[DV];
#pragma unroll
    for (int x = 0; x < DV; ++x)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[x][r] = 0.f;
    float m_run = -INFINITY;  // running max (log2 domain)
    float l_run = 0.f;        // this lane's share of the running sum

    int j_lo, j_hi;
    key_range(a, q0, min(q0 + kFwdBM, a.sq), j_lo, j_hi);
    const int t_lo = j_lo / kFwdBN;
    const int t_hi = (j_hi + kFwdBN - 1) / kFwdBN;

    const int wq_last = min(wq0 + 31, a.sq - 1);
    const uint64_t drop_row_base = ((uint64_t)bh * a.sq + (uint64_t)q_row) * (uint64_t)a.sk;
    const float* bias_row = nullptr;
    if (a.has_bias)
        bias_row = a.bias + b * a.bs[0] + h * a.bs[1] + (int64_t)q_row * a.bs[2];

    Stage ks, vs;
    if (t_lo < t_hi) {
        ks.load(k_base, a.ks[1], t_lo * kFwdBN, a.sk, a.d);
        vs.load(v_base, a.vs[1], t_lo * kFwdBN, a.sk, a.d);
        ks.store(k_lds);
        vs.store(v_lds);
    }
    __syncthreads();

    for (int t = t_lo; t < t_hi; ++t) {
        const int buf = (t - t_lo) & 1;
        const T* kt = k_lds + buf * kTileElems;
        const T* vt = v_lds + buf * kTileElems;
        const int j0 = t * kFwdBN;
        const bool have_next = t + 1 < t_hi;
        if (have_next) {
            ks.load(k_base, a.ks[1], j0 + kFwdBN, a.sk, a.d);
            vs.load(v_base, a.vs[1], j0 + kFwdBN, a.sk, a.d);
        }

        // Wavefront-uniform: does this tile hold any visible key for this wavefront's queries?
        bool active = wq0 < a.sq;
        if (a.causal && j0 > wq_last) active = false;
        if (a.window > 0 && wq0 - (j0 + kFwdBN - 1) >= a.window) active = false;

        if (active) {
            // ---- S^T = K Q^T ----
            f32x16_t s_acc[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s_acc[kb][r] = 0.f;
                const T* krow = kt + (kb * 32 + pi_row(i_loc)) * kPitch + 8 * g;
#pragma unroll
                for (int x = 0; x < DK; ++x)
                    s_acc[kb] = Mma<T>::mma32(lds_frag<T>(krow + 16 * x), qf[x], s_acc[kb]);
            }

            // ---- scale, bias, masks (log2 domain) ----
            const bool need_mask = (j0 + kFwdBN > a.sk) || (a.causal && j0 + kFwdBN - 1 > wq0) ||
                                   (a.window > 0 && wq_last - j0 >= a.window);
            float mx = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int key0 = j0 + kb * 32 + acc_row(4 * r4, g);
                    float bv[4] = {0.f, 0.f, 0.f, 0.f};
                    if (a.has_bias) {
                        if (a.bias_vec4 && key0 + 3 < a.sk) {
                            const f32x4_t t4 =
                                *reinterpret_cast<const f32x4_t*>(bias_row + key0);
                            bv[0] = t4.x, bv[1] = t4.y, bv[2] = t4.z, bv[3] = t4.w;
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if (key0 + e < a.sk && q_row < a.sq)
                                    bv[e] = bias_row[(int64_t)(key0 + e) * a.bs[3]];
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float s = s_acc[kb][4 * r4 + e] * a.scale_log2;
                        if (a.has_bias) s = __builtin_fmaf(bv[e], kLog2e, s);
                        if (need_mask && !key_visible(a, q_row, key0 + e)) s = -INFINITY;
                        s_acc[kb][4 * r4 + e] = s;
                        mx = fmaxf(mx, s);
                    }
                }
            }
            mx = fmaxf(mx, xor32(mx));

            // ---- online softmax ----
            const float m_new = fmaxf(m_run, mx);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = fast_exp2(m_run - m_use);
            m_run = m_new;
            float psum = 0.f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float p = fast_exp2(s_acc[kb][r] - m_use);
                    s_acc[kb][r] = p;
                    psum += p;
                }
            l_run = l_run * alpha + psum;
#pragma unroll
            for (int x = 0; x < DV; ++x)
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[x][r] *= alpha;

            // ---- dropout on P (the normaliser keeps the undropped sum) ----
            if (a.dropout) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        const int key0 = j0 + kb * 32 + acc_row(4 * r4, g);
                        uint32_t bits = 0;
                        if (q_row < a.sq && key0 < a.sk) {
                            const uint64_t e0 = drop_row_base + (uint64_t)key0;
                            if (a.dropout_fast) {
                                bits = dropout_keep4(a.rng, e0 >> 2);
                            } else {
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    if (key0 + e < a.sk)
                                        bits |= (dropout_keep1(a.rng, e0 + e) ? 1u : 0u) << e;
                            }
                        }
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float p = s_acc[kb][4 * r4 + e];
                            s_acc[kb][4 * r4 + e] = ((bits >> e) & 1u) ? p * a.rng.inv_keep : 0.f;
                        }
                    }
            }

            // ---- O^T += V^T P^T ----
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4) {
                const int kb = s4 >> 1, hh = s4 & 1;
                u32x4_t pw;
                pw.x = pack2<T>(s_acc[kb][8 * hh + 0], s_acc[kb][8 * hh + 1]);
                pw.y = pack2<T>(s_acc[kb][8 * hh + 2], s_acc[kb][8 * hh + 3]);
                pw.z = pack2<T>(s_acc[kb][8 * hh + 4], s_acc[kb][8 * hh + 5]);
                pw.w = pack2<T>(s_acc[kb][8 * hh + 6], s_acc[kb][8 * hh + 7]);
                const frag_t pf = __builtin_bit_cast(frag_t, pw);
                // source address of the transposing read for this lane
                const T* vsrc = vt + (kb * 32 + 16 * hh + 8 * g + ((lane & 15) >> 2)) * kPitch +
                                ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
#pragma unroll
                for (int x = 0; x < DV; ++x)
                    o_acc[x] = Mma<T>::mma32(lds_frag_tr<T>(vsrc + 32 * x, kPitch), pf, o_acc[x]);
            }
        }

        if (have_next) {
            ks.store(k_lds + (buf ^ 1) * kTileElems);
            vs.store(v_lds + (buf ^ 1) * kTileElems);
        }
        __syncthreads();
    }

    // ---- epilogue ----
    const float l_tot = l_run + xor32(l_run);
    const float inv_l = 1.0f / l_tot;
    if (q_row < a.sq) {
        T* o_row = reinterpret_cast<T*>(a.o) + b * a.os[0] + (int64_t)q_row * a.os[1] + h * a.os[2];
#pragma unroll
        for (int x = 0; x < DV; ++x)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const int d0 = x * 32 + 8 * r4 + 4 * g;
                if (d0 < a.d) {
                    u32x2_t w;
                    w.x = pack2<T>(o_acc[x][4 * r4 + 0] * inv_l, o_acc[x][4 * r4 + 1] * inv_l);
                    w.y = pack2<T>(o_acc[x][4 * r4 + 2] * inv_l, o_acc[x][4 * r4 + 3] * inv_l);
                    *reinterpret_cast<u32x2_t*>(o_row + d0) = w;
                }
            }
        if (g == 0) a.lse[(int64_t)bh * a.sq + q_row] = (m_run + __builtin_log2f(l_tot)) * kLn2;
    }
}

template <typename T, int DPAD>
int launch_fwd(const AttnArgs& a, hipStream_t st) {
    typedef TileStage<T, DPAD, kFwdBN, kFwdThreads> Stage;
    const size_t smem = (size_t)4 * kFwdBN * Stage::kPitch * sizeof(T);
    const int n_qt = (a.sq + kFwdBM - 1) / kFwdBM;
    const int64_t blocks = (int64_t)n_qt * a.batch * a.heads;
    if (blocks <= 0 || blocks > 0x7FFFFFFF) return SLAPO_ERR_SHAPE;
    auto kern = attn_fwd_kernel<T, DPAD>;
    if (smem > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)smem) != hipSuccess)
            return SLAPO_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kFwdThreads), smem, st, a);
    return check_launch();
}

template <typename T>
int dispatch_fwd(const AttnArgs& a, hipStream_t st) {
    if (a.d <= 32) return launch_fwd<T, 32>(a, st);
    if (a.d <= 64) return launch_fwd<T, 64>(a, st);
    if (a.d <= 96) return launch_fwd<T, 96>(a, st);
    if (a.d <= 128) return launch_fwd<T, 128>(a, st);
    return SLAPO_ERR_SHAPE;
}

}  // namespace

namespace slapo {
int attn_fwd_mfma(const AttnArgs& a, int dtype, hipStream_t st) {
    if (dtype == SLAPO_F16) return dispatch_fwd<f16_t>(a, st);
    if (dtype == SLAPO_BF16) return dispatch_fwd<bf16_t>(a, st);
    return SLAPO_ERR_DTYPE;
}
}  // namespace slapo
