// Flash-attention forward for gfx950, fp16 / bf16 inputs, fp32 softmax and accumulation.
//
// One workgroup (4 wavefronts) owns 128 consecutive queries of one (batch, head); wavefront w
// owns 32 of them.  Keys/values stream through LDS in tiles of 64 (K: ring of 2, V: ring of 3;
// global loads for tile t+2 are in flight while tile t is processed).
//
// With lane l, i = l % 32, g = l / 32, per key tile:
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
//
// A wavefront cannot overlap its own matrix and vector instructions unless they are interleaved
// in the instruction stream, so the loop is software pipelined: iteration t issues the MFMAs of
// S(t+1) among the exponentials of tile t, and the bias / mask / row-max work on S(t+1) among the
// MFMAs of P(t) V(t).  The reference point of the exponentials moves lazily (only when a tile
// maximum exceeds it by more than kMaxSlack), which keeps the accumulator rescale off the
// common path.
//
// Masks (causal, local window, key tail) are index arithmetic applied only on tiles that need
// it; an additive bias is broadcast in-kernel; dropout bits are regenerated from Philox in the
// element order of the dense [B*H, Sq, Sk] tensor (4 consecutive keys = one Philox block).
// Bias and dropout are template switches so that the common path carries no flag tests.
//
// Reference semantics: slapo/op/attention.py:163-181 (attention_bmk), :97-131 (flash_attn_ref).
#pragma once
#include <cstdio>
#include <type_traits>

#include "attn_common.h"

namespace slapo {
namespace fwd {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kBM = kWaves * 32;
constexpr int kBN = 64;
constexpr int kKRing = 2;
constexpr int kVRing = 3;

// Running-max hysteresis (log2 units): probabilities are bounded by 2^kMaxSlack before
// normalisation, well inside fp16 / fp32 range.
constexpr float kMaxSlack = 8.0f;

template <typename T, int DPAD, bool kBias, int kDrop>
__global__ __launch_bounds__(kThreads, (DPAD <= 64 ? 2 : 1)) void attn_fwd_kernel(
    const AttnArgs a) {
    typedef typename Mma<T>::frag frag_t;
    typedef TileStage<T, DPAD, kBN, kThreads> Stage;
    constexpr int kPitch = Stage::kPitch;
    constexpr int kTileElems = kBN * kPitch;
    constexpr int DK = DPAD / 16;  // k-steps of S^T = K Q^T
    constexpr int DV = DPAD / 32;  // 32-row blocks of O^T

    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    T* k_lds = smem;                        // K[kKRing][tile]
    T* v_lds = smem + kKRing * kTileElems;  // V[kVRing][tile]

    const int n_bh = a.batch * a.heads;
    const int n_qt = (a.sq + kBM - 1) / kBM;
    const int bh = blockIdx.x % n_bh;
    const int qt = n_qt - 1 - blockIdx.x / n_bh;  // heaviest (latest) query tiles first
    const int b = bh / a.heads;
    const int h = bh % a.heads;
    const int q0 = qt * kBM;

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
    // The loads are issued here and masked after the first K / V tile loads have been issued too,
    // so that all start-up loads of the workgroup are in flight together.
    frag_t qf[DK];
    u32x4_t q_raw[DK];
    {
        const int qr = min(q_row, a.sq - 1);
#pragma unroll
        for (int t = 0; t < DK; ++t)
            q_raw[t] = *reinterpret_cast<const u32x4_t*>(q_base + (int64_t)qr * a.qs[1] +
                                                         min(16 * t + 8 * g, a.d - 8));
    }

    f32x16_t o_acc[DV];
#pragma unroll
    for (int x = 0; x < DV; ++x)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[x][r] = 0.f;
    // Without a bias the scores stay in units of the raw dot product and the scale is folded
    // into the exponential's FMA; with a bias they are converted to log2 units when the bias is
    // added.  m_run is the reference in score units, m_ref = m_run in log2 units (0 if -inf).
    float m_run = -INFINITY;
    float m_ref = 0.f;
    float l_run = 0.f;  // this lane's share of the running sum

    int j_lo, j_hi;
    key_range(a, q0, min(q0 + kBM, a.sq), j_lo, j_hi);
    if constexpr (kBias)  // skip the tiles that hold nothing but padded keys
        j_hi = max(j_lo + 1, min(j_hi, padded_key_limit<kThreads>(
                                           a, b, h, reinterpret_cast<float*>(smem_raw))));
    const int t_lo = j_lo / kBN;
    const int t_hi = (j_hi + kBN - 1) / kBN;
    const int n_tiles = t_hi - t_lo;

    const int wq_last = min(wq0 + 31, a.sq - 1);
    const float c_log2 = a.scale_log2;
    const float slack = kBias ? kMaxSlack : kMaxSlack / c_log2;
    uint64_t drop_row_base = 0;
    if constexpr (kDrop != 0)
        drop_row_base = ((uint64_t)bh * a.sq + (uint64_t)q_row) * (uint64_t)a.sk;
    const float* bias_row = nullptr;
    if constexpr (kBias)
        bias_row = a.bias + b * a.bs[0] + h * a.bs[1] + (int64_t)min(q_row, a.sq - 1) * a.bs[2];

    // per-lane LDS offsets (elements) that do not change from tile to tile
    const int k_off = pi_row(i_loc) * kPitch + 8 * g;
    const int v_off = (8 * g + ((lane & 15) >> 2)) * kPitch + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);

    // Wavefront-uniform: does tile t hold any visible key for this wavefront's queries?
    auto tile_active = [&](int t) __attribute__((always_inline)) {
        if (t < t_lo || t >= t_hi || wq0 >= a.sq) return false;
        const int j0 = t * kBN;
        if (a.causal && j0 > wq_last) return false;
        if (a.window > 0 && wq0 - (j0 + kBN - 1) >= a.window) return false;
        return true;
    };
    auto tile_needs_mask = [&](int t) __attribute__((always_inline)) {
        const int j0 = t * kBN;
        return (j0 + kBN > a.sk) || (a.causal && j0 + kBN - 1 > wq0) ||
               (a.window > 0 && wq_last - j0 >= a.window);
    };

    // ---- stages of the pipeline -------------------------------------------------------------
    // S^T = K Q^T for the tile in ring slot kt
    auto scores = [&](const T* kt, f32x16_t (&s)[2]) __attribute__((always_inline)) {
        frag_t kfr[2][DK];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int x = 0; x < DK; ++x)
                kfr[kb][x] = lds_frag<T>(kt + kb * 32 * kPitch + k_off + 16 * x);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[kb][r] = 0.f;
        // the two accumulators alternate so that no MFMA waits for its predecessor
#pragma unroll
        for (int x = 0; x < DK; ++x)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) s[kb] = Mma<T>::mma32(kfr[kb][x], qf[x], s[kb]);
    };

    // bias, masks and tile maximum of freshly computed scores; returns the row maximum
    // mask_tag: 0 = every key visible, 1 = upper bound only (causal / key tail), 2 = both bounds
    auto finish_scores = [&](f32x16_t (&s)[2], int t, auto mask_tag) __attribute__((always_inline)) -> float {
        constexpr int kMask = decltype(mask_tag)::value;
        const int j0 = t * kBN;
        // register (kb, r) is key j0 + 8 g + c with c = 32 kb + acc_row(r, 0); visible iff
        // c_lo <= c <= c_hi
        int c_lo = 0, c_hi = 0;
        if constexpr (kMask != 0) {
            const int k_max = a.causal ? min(a.sk - 1, q_row) : a.sk - 1;
            c_hi = k_max - j0 - 8 * g;
            if constexpr (kMask == 2) c_lo = q_row - a.window + 1 - j0 - 8 * g;
        }
        float mx = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                if constexpr (kBias) {
                    const int key0 = j0 + kb * 32 + acc_row(4 * r4, g);
                    float bv[4] = {0.f, 0.f, 0.f, 0.f};
                    if (a.bias_vec4 && key0 + 3 < a.sk) {
                        const f32x4_t t4 = *reinterpret_cast<const f32x4_t*>(bias_row + key0);
                        bv[0] = t4.x, bv[1] = t4.y, bv[2] = t4.z, bv[3] = t4.w;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (key0 + e < a.sk) bv[e] = bias_row[(int64_t)(key0 + e) * a.bs[3]];
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        s[kb][4 * r4 + e] =
                            __builtin_fmaf(s[kb][4 * r4 + e], c_log2, bv[e] * kLog2e);
                }
                if constexpr (kMask != 0) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int c = kb * 32 + acc_row(4 * r4, 0) + e;
                        if constexpr (kMask == 2) {
                            if (c > c_hi || c < c_lo) s[kb][4 * r4 + e] = -INFINITY;
                        } else {
                            if (c > c_hi) s[kb][4 * r4 + e] = -INFINITY;
                        }
                    }
                }
                mx = fmaxf(mx, fmaxf(fmaxf(s[kb][4 * r4], s[kb][4 * r4 + 1]),
                                     fmaxf(s[kb][4 * r4 + 2], s[kb][4 * r4 + 3])));
            }
        }
        return max_xor32(mx);
    };
    auto finish_any = [&](f32x16_t (&s)[2], int t) __attribute__((always_inline)) -> float {
        if (!tile_needs_mask(t)) return finish_scores(s, t, std::integral_constant<int, 0>{});
        if (a.window > 0) return finish_scores(s, t, std::integral_constant<int, 2>{});
        return finish_scores(s, t, std::integral_constant<int, 1>{});
    };

    // move the reference point if this tile's maximum calls for it (rare after the first tile)
    auto update_reference = [&](float mx) __attribute__((always_inline)) {
        const bool move = (mx > m_run + slack || m_run == -INFINITY) && mx != -INFINITY;
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(move) != 0, 0)) {
            const float m_new = move ? mx : m_run;
            const float m_new_ref = kBias ? m_new : m_new * c_log2;
            // exp2(old reference - new reference); an unset reference (-inf) scales by 0
            const float alpha = (m_run == -INFINITY) ? 0.f : fast_exp2(m_ref - m_new_ref);
            if (move) {
                m_run = m_new;
                m_ref = m_new_ref;
                l_run *= alpha;
#pragma unroll
                for (int x = 0; x < DV; ++x)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o_acc[x][r] *= alpha;
            }
        }
    };

    // probabilities of the current tile: exp2, row sum, dropout, pack to T
    auto probabilities = [&](f32x16_t (&s)[2], int t, uint32_t (&pw)[16]) __attribute__((always_inline)) {
        float psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float p;
                if constexpr (kBias)
                    p = fast_exp2(s[kb][r] - m_ref);
                else
                    p = fast_exp2(__builtin_fmaf(s[kb][r], c_log2, -m_ref));
                s[kb][r] = p;
                psum += p;
            }
        l_run += psum;
        if constexpr (kDrop != 0) {
            const int j0 = t * kBN;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int key0 = j0 + kb * 32 + acc_row(4 * r4, g);
                    uint32_t bits = 0;
                    if (q_row < a.sq && key0 < a.sk) {
                        const uint64_t e0 = drop_row_base + (uint64_t)key0;
                        if constexpr (kDrop == 1)
                            bits = dropout_keep4_pow2(a.rng, e0 >> 2);
                        else
                            bits = dropout_keep_any(a.rng, e0, min(4, a.sk - key0));
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float p = s[kb][4 * r4 + e];
                        s[kb][4 * r4 + e] = ((bits >> e) & 1u) ? p * a.rng.inv_keep : 0.f;
                    }
                }
        }
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r2 = 0; r2 < 8; ++r2)
                pw[kb * 8 + r2] = pack2<T>(s[kb][2 * r2], s[kb][2 * r2 + 1]);
    };

    // O^T += V^T P^T for the tile in ring slot vt
    auto accumulate = [&](const T* vt, const uint32_t (&pw)[16]) __attribute__((always_inline)) {
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) {
            u32x4_t pq = {pw[4 * s4], pw[4 * s4 + 1], pw[4 * s4 + 2], pw[4 * s4 + 3]};
            const frag_t pf = __builtin_bit_cast(frag_t, pq);
#pragma unroll
            for (int x = 0; x < DV; ++x)
                o_acc[x] = Mma<T>::mma32(
                    lds_frag_tr<T>(vt + 16 * s4 * kPitch + v_off + 32 * x, kPitch), pf, o_acc[x]);
        }
    };

    // ---- prologue: tiles 0 and 1 of this workgroup into LDS, tile 2 in flight -----------------
    // Two register stages alternate: a tile is requested two iterations before it is written to
    // LDS, so a full iteration of math sits between the request and the wait.
    // With two workgroups per CU (DPAD <= 64) one register stage set is enough and leaves the
    // registers to the math; a lone workgroup per CU wants the deeper prefetch of two sets.
    constexpr bool kTwoStages = DPAD > 64;
    Stage ks_a, vs_a, ks_b, vs_b;
    // rows are clamped into the tensor, so the requests are safe whatever n_tiles is
    ks_a.load(k_base, a.ks[1], t_lo * kBN, a.sk, a.d);
    vs_a.load(v_base, a.vs[1], t_lo * kBN, a.sk, a.d);
    ks_b.load(k_base, a.ks[1], (t_lo + 1) * kBN, a.sk, a.d);
    vs_b.load(v_base, a.vs[1], (t_lo + 1) * kBN, a.sk, a.d);
    ks_a.fix(t_lo * kBN, a.sk, a.d);
    vs_a.fix(t_lo * kBN, a.sk, a.d);
    ks_a.store(k_lds);
    vs_a.store(v_lds);
    if (1 < n_tiles) {
        ks_b.fix((t_lo + 1) * kBN, a.sk, a.d);
        vs_b.fix((t_lo + 1) * kBN, a.sk, a.d);
        ks_b.store(k_lds + kTileElems);
        vs_b.store(v_lds + kTileElems);
    }
#pragma unroll
    for (int t = 0; t < DK; ++t)
        qf[t] = __builtin_bit_cast(
            frag_t, keep_or_zero(q_raw[t], q_row < a.sq && 16 * t + 8 * g < a.d));
    if (kTwoStages && 2 < n_tiles) {
        ks_b.load(k_base, a.ks[1], (t_lo + 2) * kBN, a.sk, a.d);
        vs_b.load(v_base, a.vs[1], (t_lo + 2) * kBN, a.sk, a.d);
    }
    __syncthreads();

    // Two score buffers that swap roles every iteration (no register copies).
    f32x16_t s_a[2], s_b[2];
    bool cur_active = tile_active(t_lo);
    if (cur_active) {
        scores(k_lds, s_a);
        const float mx = finish_any(s_a, t_lo);
        update_reference(mx);
    }
    // K slot 0 is overwritten (with tile 2) at the end of iteration 0: every wavefront must have
    // finished reading it for the scores above before any wavefront gets there.
    __syncthreads();

    // iteration r with two stage sets: requests tile r+3 into (k_ld, v_ld), writes tile r+2 from
    // (k_st, v_st); with one: requests tile r+2 at the top and writes it at the bottom
    auto iteration = [&](int r, f32x16_t (&s_cur)[2], f32x16_t (&s_next)[2], Stage& k_ld,
                         Stage& v_ld, Stage& k_st, Stage& v_st) __attribute__((always_inline)) {
        const int t = t_lo + r;
        if constexpr (kTwoStages) {
            if (r + 3 < n_tiles) {
                k_ld.load(k_base, a.ks[1], (t + 3) * kBN, a.sk, a.d);
                v_ld.load(v_base, a.vs[1], (t + 3) * kBN, a.sk, a.d);
            }
        } else {
            if (r + 2 < n_tiles) {
                k_st.load(k_base, a.ks[1], (t + 2) * kBN, a.sk, a.d);
                v_st.load(v_base, a.vs[1], (t + 2) * kBN, a.sk, a.d);
            }
        }
        const bool next_active = tile_active(t + 1);
        const T* k_next = k_lds + ((r + 1) % kKRing) * kTileElems;
        const T* v_cur = v_lds + (r % kVRing) * kTileElems;

        uint32_t pw[16];
        float mx_next = -INFINITY;
        if (cur_active && next_active) {
            // the fused body: MFMAs of S(t+1) among the exponentials of tile t, then the
            // bias / mask / max work on S(t+1) among the MFMAs of P(t) V(t)
            scores(k_next, s_next);
            probabilities(s_cur, t, pw);
            accumulate(v_cur, pw);
            mx_next = finish_any(s_next, t + 1);
        } else if (cur_active) {
            probabilities(s_cur, t, pw);
            accumulate(v_cur, pw);
        } else if (next_active) {
            scores(k_next, s_next);
            mx_next = finish_any(s_next, t + 1);
        }
        if (next_active) update_reference(mx_next);
        cur_active = next_active;

        if (r + 2 < n_tiles) {
            k_st.fix((t + 2) * kBN, a.sk, a.d);
            v_st.fix((t + 2) * kBN, a.sk, a.d);
            k_st.store(k_lds + ((r + 2) % kKRing) * kTileElems);
            v_st.store(v_lds + ((r + 2) % kVRing) * kTileElems);
        }
        __syncthreads();
    };

    for (int r = 0; r < n_tiles; r += 2) {
        if constexpr (kTwoStages) {
            iteration(r, s_a, s_b, ks_a, vs_a, ks_b, vs_b);
            if (r + 1 < n_tiles) iteration(r + 1, s_b, s_a, ks_b, vs_b, ks_a, vs_a);
        } else {
            iteration(r, s_a, s_b, ks_a, vs_a, ks_a, vs_a);
            if (r + 1 < n_tiles) iteration(r + 1, s_b, s_a, ks_a, vs_a, ks_a, vs_a);
        }
    }
    // ---- epilogue ----
    const float l_tot = sum_xor32(l_run);
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
        if (g == 0) {
            const float m_log2 = (m_run == -INFINITY) ? -INFINITY : m_ref;
            a.lse[(int64_t)bh * a.sq + q_row] = (m_log2 + __builtin_log2f(l_tot)) * kLn2;
        }
    }
}

template <typename T, int DPAD, bool kBias, int kDrop>
int launch(const AttnArgs& a, hipStream_t st) {
    typedef TileStage<T, DPAD, kBN, kThreads> Stage;
    const size_t smem = (size_t)(kKRing + kVRing) * kBN * Stage::kPitch * sizeof(T);
    const int n_qt = (a.sq + kBM - 1) / kBM;
    const int64_t blocks = (int64_t)n_qt * a.batch * a.heads;
    if (blocks <= 0 || blocks > 0x7FFFFFFF) return SLAPO_ERR_SHAPE;
    auto kern = attn_fwd_kernel<T, DPAD, kBias, kDrop>;
    if (smem > 48 * 1024) {
        static bool raised = false;  // per instantiation
        if (!raised) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem) != hipSuccess)
                return SLAPO_ERR_LAUNCH;
            raised = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kThreads), smem, st, a);
    return check_launch();
}

template <typename T, int DPAD>
int dispatch_flags(const AttnArgs& a, hipStream_t st) {
    if (a.has_bias) {
        if (a.dropout == 1) return launch<T, DPAD, true, 1>(a, st);
        if (a.dropout == 2) return launch<T, DPAD, true, 2>(a, st);
        return launch<T, DPAD, true, 0>(a, st);
    }
    if (a.dropout == 1) return launch<T, DPAD, false, 1>(a, st);
    if (a.dropout == 2) return launch<T, DPAD, false, 2>(a, st);
    return launch<T, DPAD, false, 0>(a, st);
}

template <typename T>
int dispatch(const AttnArgs& a, hipStream_t st) {
    if (a.d <= 96) return dispatch_flags<T, 96>(a, st);
    if (a.d <= 128) return dispatch_flags<T, 128>(a, st);
    return SLAPO_ERR_SHAPE;
}

}  // namespace fwd
}  // namespace slapo
