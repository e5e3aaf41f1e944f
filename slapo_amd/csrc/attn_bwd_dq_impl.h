// Flash-attention backward, dQ half, for gfx950 (fp16 / bf16 inputs, fp32 accumulation).
//
// The backward is split in two kernels that each recompute the probabilities: this one owns query
// rows and produces dQ, its sibling owns key rows and produces dK / dV.  Neither needs atomics or
// a zero-initialised accumulator, and the result does not depend on scheduling order.  This kernel
// also produces delta = rowsum(dO * O) for its query rows (it holds the dO fragments anyway) and
// stores it for the dK / dV kernel, which therefore has to run after it.
//
// One workgroup (4 wavefronts) owns 128 consecutive queries of one (batch, head); wavefront w
// owns 32 of them and keeps their Q^T and dO^T fragments, lse and delta in registers.  Keys and
// values stream through LDS in tiles of 64, double buffered and staged through registers (the
// global loads of tile t+1 are in flight while tile t is processed).  Per key tile, lane l = query
// i, registers = keys:
//   S^T  = K Q^T, dP^T = V dO^T    A = K / V rows from LDS (row-permuted 128-bit reads); Q carries
//                                  scale * log2(e)
//   P^T  = exp2(S^T - lse), dS^T = P^T * (dP^T - delta)     (at head_dim 64 and 128 the two
//                                  subtractions are done by the matrix pipe: the accumulators
//                                  start from -lse and -delta of the lane's query)
//   dQ^T += K^T dS^T               B = dS^T straight from the accumulator registers, A = K^T read
//                                  from the row-major K tile with the transposing LDS read.
//
// Reference semantics: autograd of slapo/op/attention.py:163-181 (attention_bmk).
#pragma once
#include <type_traits>

#include "attn_common.h"

namespace slapo {
namespace bwd_dq {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kBM = kWaves * 32;
constexpr int kBN = 64;
constexpr int kKRing = 2;
constexpr int kVRing = 2;

// kStagger: see the tile bodies below.  Staggered halves need one workgroup per CU above
// head_dim 64; sequential halves fit two.
// kBias: 0 = no additive bias, 1 = any layout (read from memory per score), 2 = the bias depends on
// the key only (stride 0 over the queries): its 64 values per key tile travel through LDS beside
// the K / V tile, and the tile bodies have neither global loads nor branches for them.
template <typename T, int DPAD, int kBias, int kDrop, bool kStagger, int kSteps>
__global__ __launch_bounds__(kThreads, (kStagger && DPAD > 64 ? 1 : 2)) void attn_bwd_dq_kernel(
    const AttnArgs a_in) {
    AttnArgs a = a_in;
    if constexpr (kDrop == 1 || kDrop == 2) resolve_device_state(a.rng);
    typedef typename Mma<T>::frag frag_t;
    typedef TileStage<T, DPAD, kBN, kThreads> Stage;
    constexpr int kPitch = Stage::kPitch;
    constexpr int kTileElems = kBN * kPitch;
    // k-steps over the head dimension: DPAD / 16, or one fewer where the launcher guarantees
    // head_dim <= 16 * kSteps (head_dim 80 in the 96-wide build)
    constexpr int DK = kSteps;
    constexpr int DV = DPAD / 32;  // 32-row blocks of dQ^T

    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    T* k_lds = smem;                        // K[kKRing][tile]
    T* v_lds = smem + kKRing * kTileElems;  // V[kVRing][tile]
    float* bias_lds = reinterpret_cast<float*>(smem + (kKRing + kVRing) * kTileElems);  // [2][kBN]

    const int n_bh = a.batch * a.heads;
    const int n_qt = (a.sq + kBM - 1) / kBM;
    const int work = work_index(a);
    const int bh = work % n_bh;
    const int qt = n_qt - 1 - work / n_bh;  // heaviest (latest) query tiles first
    const int b = bh / a.heads;
    const int h = bh % a.heads;
    const int q0 = qt * kBM;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wavefront-uniform
    const int g = lane >> 5;
    const int i_loc = lane & 31;
    const int wq0 = q0 + wave * 32;
    const int q_row = wq0 + i_loc;

    const T* q_base = reinterpret_cast<const T*>(a.q) + b * a.qs[0] + h * a.qs[2];
    const T* k_base = reinterpret_cast<const T*>(a.k) + b * a.ks[0] + h * a.ks[2];
    const T* v_base = reinterpret_cast<const T*>(a.v) + b * a.vs[0] + h * a.vs[2];
    const T* g_base = reinterpret_cast<const T*>(a.dout) + b * a.os[0] + h * a.os[2];

    // Start-up loads, all issued before any of them is used: the Q^T and dO^T fragments (column
    // i = this lane's query, k-slots = 8 head-dim elements), lse, delta and the first K / V tile.
    // Addresses are clamped into the tensor; what was clamped is zeroed afterwards.
    Stage ks, vs;
    // The dropout variants at head_dim 128 have no registers to spare for the tile offsets that
    // `load` keeps: they multiply the addresses out (measured 13 % faster there).
    constexpr bool kIndexed = (kDrop == 1 || kDrop == 2) && DPAD > 96;
    if constexpr (!kIndexed) {
        ks.init(a.ks[1], a.d);
        vs.init(a.vs[1], a.d);
    }
    // kBias == 2: thread (x & 63) carries key row0 + (x & 63) of the requested tile (all four
    // wavefronts alike, so that neither request nor store needs a branch)
    const float* bias_keys = nullptr;
    if constexpr (kBias == 2) bias_keys = a.bias + b * a.bs[0] + h * a.bs[1];
    float bias_stage = 0.f;
    auto store_bias = [&](int slot) __attribute__((always_inline)) {
        if constexpr (kBias == 2) bias_lds[slot * kBN + row_slot(lane)] = bias_log2(bias_stage);
    };
    const float* bias_tile = bias_lds;  // the slot of the tile in process
    auto request = [&](int row0) __attribute__((always_inline)) {
        if constexpr (kBias == 2)
            bias_stage = bias_keys[(int64_t)min(row0 + lane, a.sk - 1) * a.bs[3]];
        if constexpr (kIndexed) {
            ks.load_indexed(k_base, a.ks[1], row0, a.sk, a.d);
            vs.load_indexed(v_base, a.vs[1], row0, a.sk, a.d);
        } else {
            ks.load(k_base, a.ks[1], row0, a.sk, a.d);
            vs.load(v_base, a.vs[1], row0, a.sk, a.d);
        }
    };
    int j_lo, j_hi;
    key_range(a, q0, min(q0 + kBM, a.sq), j_lo, j_hi);
    if constexpr (kBias)  // skip the tiles that hold nothing but padded keys
        j_hi = max(j_lo + 1, min(j_hi, padded_key_limit<kThreads>(
                                           a, b, h, reinterpret_cast<float*>(smem_raw))));
    const int t_lo = j_lo / kBN;
    const int t_hi = (j_hi + kBN - 1) / kBN;
    const int n_tiles = t_hi - t_lo;

    frag_t qf[DK], gf[DK];
    float lse2, delta, inv_n = 1.0f;
    {
        const int qr = min(q_row, a.sq - 1);
        const T* o_base = reinterpret_cast<const T*>(a.o) + b * a.os[0] + h * a.os[2];
        u32x4_t qv[DK], gv[DK], ov[DK];
#pragma unroll
        for (int t = 0; t < DK; ++t) {
            const int dc = min(16 * t + 8 * g, a.d - 8);
            qv[t] = *reinterpret_cast<const u32x4_t*>(q_base + (int64_t)qr * a.qs[1] + dc);
            gv[t] = *reinterpret_cast<const u32x4_t*>(g_base + (int64_t)qr * a.os[1] + dc);
            ov[t] = *reinterpret_cast<const u32x4_t*>(o_base + (int64_t)qr * a.os[1] + dc);
        }
        const float lse_raw = a.lse[(int64_t)bh * a.sq + qr];
        request(t_lo * kBN);
        const bool row_ok = q_row < a.sq;
#pragma unroll
        for (int t = 0; t < DK; ++t) {
            const bool keep = row_ok && (16 * t + 8 * g < a.d);
            qf[t] = __builtin_bit_cast(frag_t, keep_or_zero(qv[t], keep));
            gf[t] = __builtin_bit_cast(frag_t, keep_or_zero(gv[t], keep));
        }
        // Q times scale * log2(e), once: the scores leave the matrix pipe in log2 units
#pragma unroll
        for (int t = 0; t < DK; ++t) {
            qf[t] = scale_frag<T>(__builtin_bit_cast(u32x4_t, qf[t]), a.scale_log2);
        }
        // log2 units; +inf for rows past the end so that P = 0 there.  A row that saw nothing
        // but masked keys (bias_log2) stored its row sum n instead: its probabilities are
        // exp2(x + FLT_MAX) / n.  The kernel works with exp2(x + FLT_MAX) and the true delta,
        // and applies 1 / n to the finished dQ row and to the delta that it hands on (the dK / dV
        // kernel scales that row of dO instead).
        lse2 = row_ok ? (kBias ? lse_reference(lse_raw, kLog2e) : lse_raw * kLog2e) : INFINITY;
        if constexpr (kBias) inv_n = lse_row_factor(lse_raw);
        // delta = sum_d dO * O: lanes i and i + 32 hold complementary head-dim slots of row i
        float part = 0.f;
#pragma unroll
        for (int t = 0; t < DK; ++t) {
            const frag_t of = __builtin_bit_cast(frag_t, ov[t]);
#pragma unroll
            for (int j = 0; j < 8; ++j)
                part = __builtin_fmaf((float)gf[t][j], (float)of[j], part);
        }
        delta = sum_xor32(part);  // masked dO slots are zero, so clamped rows / columns add nothing
        if (row_ok && g == 0) a.delta[(int64_t)bh * a.sq + q_row] = delta * inv_n;
    }
    // Where the registers allow it the per-row terms enter through the accumulators: S^T starts
    // from -lse (log2 units) and, without dropout, dP^T from -delta, in all sixteen registers of
    // the lane (= one query).  Measured against explicit subtractions: 130 against 150 us at bf16
    // B4 S2048 H16 D128 causal, 43.5 against 45 us at fp16 B8 S1024 H16 D64; at head_dim 80 / 96
    // the 32 registers cost more than the subtractions (189 against 168 us at B4 S2048 H32 D80).
    constexpr bool kAccInit = DPAD != 96;
    f32x16_t s_init, dp_init;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        s_init[r] = kAccInit ? -lse2 : 0.f;
        dp_init[r] = kAccInit && kDrop == 0 ? -delta : 0.f;
    }
    const float lse_sub = kAccInit ? 0.f : lse2;
    // With dropout dS = P (M dP / (1 - p) - delta) is taken as (P (M dP - delta (1 - p))) / (1 - p):
    // the kept dP stay as they are (dropped ones become +0, two instructions each), delta is
    // scaled once per row and the factor goes onto the dQ rows when they are written.
    const float keep_prob = a.rng.inv_keep > 0.f ? 1.0f / a.rng.inv_keep : 0.f;
    const float delta_sub = kAccInit && kDrop == 0 ? 0.f : (kDrop != 0 ? delta * keep_prob : delta);

    f32x16_t dq_acc[DV];
#pragma unroll
    for (int x = 0; x < DV; ++x)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq_acc[x][r] = 0.f;

    const int wq_last = min(wq0 + 31, a.sq - 1);
    uint64_t drop_row_base = 0;
    if constexpr (kDrop != 0)
        drop_row_base = ((uint64_t)bh * a.sq + (uint64_t)q_row) * (uint64_t)a.sk;
    const float* bias_row = nullptr;
    if constexpr (kBias)
        bias_row = a.bias + b * a.bs[0] + h * a.bs[1] + (int64_t)min(q_row, a.sq - 1) * a.bs[2];

    // per-lane LDS offsets (elements) that do not change from tile to tile
    const int row_off = pi_row(i_loc) * kPitch + 8 * g;
    const int tr_off = tr_lane_off(lane, kPitch);

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

    // The tile is processed as two halves of 32 keys.  With kStagger their stages are staggered,
    // so that the matrix instructions of one half always have independent vector work of the
    // other half around them (a wavefront overlaps the two only when they are interleaved in its
    // instruction stream).  Without it the halves run one after the other: above head_dim 64 that
    // is what fits two workgroups per CU into the register file, and the second resident workgroup
    // hides more latency than the stagger does (measured: 28 % faster at head_dim 80, 2-12 % at
    // 128; only the masked tile bodies of a local window lose, to register spills, at 128).

    // S^T half = K_half Q^T (log2 units)
    auto half_s = [&](const T* kt, int kb, f32x16_t& s) __attribute__((always_inline)) {
        s = Mma<T>::mma32(lds_frag<T>(kt + kb * 32 * kPitch + row_off), qf[0], s_init);
#pragma unroll
        for (int x = 1; x < DK; ++x)
            s = Mma<T>::mma32(lds_frag<T>(kt + kb * 32 * kPitch + row_off + 16 * x), qf[x], s);
    };
    // dP^T half = V_half dO^T
    auto half_dp = [&](const T* vt, int kb, f32x16_t& dp) __attribute__((always_inline)) {
        dp = Mma<T>::mma32(lds_frag<T>(vt + kb * 32 * kPitch + row_off), gf[0], dp_init);
#pragma unroll
        for (int x = 1; x < DK; ++x)
            dp = Mma<T>::mma32(lds_frag<T>(vt + kb * 32 * kPitch + row_off + 16 * x), gf[x], dp);
    };
    // dQ^T += K_half^T dS^T half
    auto half_dq = [&](const T* kt, int kb, const uint32_t (&dw)[8]) __attribute__((always_inline)) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            u32x4_t dq4 = {dw[4 * s2], dw[4 * s2 + 1], dw[4 * s2 + 2], dw[4 * s2 + 3]};
            const frag_t df = __builtin_bit_cast(frag_t, dq4);
#pragma unroll
            for (int x = 0; x < DV; ++x)
                dq_acc[x] = Mma<T>::mma32(
                    lds_frag_tr<T>(kt + (32 * kb + 16 * s2) * kPitch + tr_off + 32 * x, kPitch), df,
                    dq_acc[x]);
        }
    };
    // scores -> probabilities, in place
    // mask_tag: 0 = every key visible, 1 = upper bound only (causal / key tail), 2 = both bounds
    auto half_exp = [&](f32x16_t& s, int t, int kb, auto mask_tag) __attribute__((always_inline)) {
        constexpr int kMask = decltype(mask_tag)::value;
        const int j0 = t * kBN + kb * 32;
        // register r is key j0 + acc_row(r, g) = j0 + kAccGroupStep g + c with c = acc_row(r, 0);
        // visible iff c_lo <= c <= c_hi
        int c_lo = 0, c_hi = 0;
        if constexpr (kMask != 0) {
            const int k_max = a.causal ? min(a.sk - 1, q_row) : a.sk - 1;
            c_hi = k_max - j0 - kAccGroupStep * g;
            if constexpr (kMask == 2) c_lo = q_row - a.window + 1 - j0 - kAccGroupStep * g;
        }
        if constexpr (kBias == 1) {
            // Registers 8 h + e and 8 h + 4 + e are keys 2 g and 2 g + 1 of the aligned group of
            // four keys at j0 + 16 h + 4 e: one 16-byte read per group where the layout allows.
#pragma unroll
            for (int he = 0; he < 8; ++he) {
                const int kg = j0 + 16 * (he >> 2) + 4 * (he & 3);
                float b_lo = 0.f, b_hi = 0.f;
                if (a.bias_vec4 && kg + 3 < a.sk) {
                    const f32x4_t t4 = *reinterpret_cast<const f32x4_t*>(bias_row + kg);
                    b_lo = g ? t4.z : t4.x;
                    b_hi = g ? t4.w : t4.y;
                } else {
                    const int k_lo = kg + 2 * g;
                    if (k_lo < a.sk) b_lo = bias_row[(int64_t)k_lo * a.bs[3]];
                    if (k_lo + 1 < a.sk) b_hi = bias_row[(int64_t)(k_lo + 1) * a.bs[3]];
                }
                s[8 * (he >> 2) + (he & 3)] += bias_log2(b_lo);
                s[8 * (he >> 2) + 4 + (he & 3)] += bias_log2(b_hi);
            }
        }
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if constexpr (kBias == 2) {  // already in log2 units
                const f32x4_t t4 = *reinterpret_cast<const f32x4_t*>(bias_tile + 32 * kb +
                                                                     quad_slot(r4, g));
                bv[0] = t4.x, bv[1] = t4.y, bv[2] = t4.z, bv[3] = t4.w;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float x = s[4 * r4 + e];  // the scale is in already
                if constexpr (!kAccInit) x -= lse_sub;
                if constexpr (kBias == 2) x += bv[e];
                float p = fast_exp2(x);
                if constexpr (kMask != 0) {
                    const int c = acc_row(4 * r4 + e, 0);
                    if constexpr (kMask == 2) {
                        if (c > c_hi || c < c_lo) p = 0.f;
                    } else {
                        if (c > c_hi) p = 0.f;
                    }
                }
                s[4 * r4 + e] = p;
            }
        }
    };
    // dS^T half = P^T (dP^T - delta), packed to T
    // kDrop == 3: the keep bits of this lane's query for one half of 32 keys, as the forward
    // stored them (requested at the top of a tile body, used in half_ds)
    auto mask_word = [&](int t, int kb) __attribute__((always_inline)) -> uint32_t {
        if constexpr (kDrop == 3) {
            const int w = min(2 * t + kb, a.mask_words - 1);
            return a.keep_mask[((int64_t)bh * a.mask_words + w) * a.mask_pitch +
                               min(q_row, a.sq - 1)];
        }
        return 0u;
    };
    auto half_ds = [&](const f32x16_t& p, const f32x16_t& dp, int t, int kb, uint32_t mword,
                       uint32_t (&dw)[8]) __attribute__((always_inline)) {
        const int j0 = t * kBN + kb * 32;
        uint32_t word = mword;  // bit j = keep(key j0 + j)
        if constexpr (kDrop == 1 || kDrop == 2) {
            // Philox blocks cover four consecutive keys; the two lanes of a query (l, l ^ 32)
            // draw the blocks of keys 8 g .. 8 g + 7 of each 16-key group and exchange them.
            word = 0;
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                const int pos = 16 * (blk >> 1) + 8 * g + 4 * (blk & 1);
                const int key0 = j0 + pos;
                uint32_t bits = 0;
                if (q_row < a.sq && key0 < a.sk) {
                    const uint64_t e0 = drop_row_base + (uint64_t)key0;
                    if constexpr (kDrop == 1)
                        bits = dropout_keep4_pow2(a.rng, e0 >> 2);
                    else
                        bits = dropout_keep_any(a.rng, e0, min(4, a.sk - key0));
                }
                word |= bits << pos;
            }
            word = or_xor32(word);
        }
        const uint32_t word_g = word >> (kAccGroupStep * g);
        float dv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float d = dp[r];
            if constexpr (kDrop != 0) d = keep_or_zero(d, word_g, acc_row(r, 0));
            if constexpr (kAccInit && kDrop == 0)
                dv[r] = p[r] * d;  // delta already subtracted by the matrix pipe
            else
                dv[r] = p[r] * (d - delta_sub);
        }
#pragma unroll
        for (int r2 = 0; r2 < 8; ++r2) dw[r2] = pack2<T>(dv[2 * r2], dv[2 * r2 + 1]);
    };
    auto tile_body = [&](const T* kt, const T* vt, int t, auto mask_tag) __attribute__((always_inline)) {
        if constexpr (!kStagger) {
            f32x16_t s0, p0;
            uint32_t dw0[8];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const uint32_t mw = mask_word(t, kb);
                half_s(kt, kb, s0);
                half_dp(vt, kb, p0);
                half_exp(s0, t, kb, mask_tag);
                half_ds(s0, p0, t, kb, mw, dw0);
                half_dq(kt, kb, dw0);
            }
            return;
        }
        f32x16_t s0, s1, p0, p1;
        uint32_t dw0[8], dw1[8];
        const uint32_t mw0 = mask_word(t, 0), mw1 = mask_word(t, 1);
        half_s(kt, 0, s0);
        half_dp(vt, 0, p0);
        half_exp(s0, t, 0, mask_tag);
        half_s(kt, 1, s1);
        half_ds(s0, p0, t, 0, mw0, dw0);
        half_dp(vt, 1, p1);
        half_exp(s1, t, 1, mask_tag);
        half_dq(kt, 0, dw0);
        half_ds(s1, p1, t, 1, mw1, dw1);
        half_dq(kt, 1, dw1);
    };

    // Hand-scheduled version of tile_body for tiles without masks: the LDS operands of each group
    // of matrix instructions are requested one phase before the group runs, and scheduling fences
    // keep the compiler from sinking the requests back down to their uses.
    auto tile_body_fast = [&](const T* kt, const T* vt, int t, auto mask_tag)
                              __attribute__((always_inline)) {
        frag_t kr0[DK], vr0[DK], kr1[DK], vr1[DK], kq0[2 * DV], kq1[2 * DV];
        f32x16_t s0, s1, p0, p1;
        uint32_t dw0[8], dw1[8];
        auto rows = [&](const T* tile, int kb, frag_t (&f)[DK]) __attribute__((always_inline)) {
#pragma unroll
            for (int x = 0; x < DK; ++x)
                f[x] = lds_frag<T>(tile + kb * 32 * kPitch + row_off + 16 * x);
        };
        auto cols = [&](int kb, frag_t (&f)[2 * DV]) __attribute__((always_inline)) {
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
                for (int x = 0; x < DV; ++x)
                    f[s2 * DV + x] =
                        lds_frag_tr<T>(kt + (32 * kb + 16 * s2) * kPitch + tr_off + 32 * x, kPitch);
        };
        auto mma_rows = [&](const frag_t (&f)[DK], const frag_t (&bfr)[DK], const f32x16_t& init,
                            f32x16_t& acc) __attribute__((always_inline)) {
            acc = Mma<T>::mma32(f[0], bfr[0], init);
#pragma unroll
            for (int x = 1; x < DK; ++x) acc = Mma<T>::mma32(f[x], bfr[x], acc);
        };
        auto mma_cols = [&](const frag_t (&f)[2 * DV], const uint32_t (&dw)[8])
                            __attribute__((always_inline)) {
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
                u32x4_t dq4 = {dw[4 * s2], dw[4 * s2 + 1], dw[4 * s2 + 2], dw[4 * s2 + 3]};
                const frag_t df = __builtin_bit_cast(frag_t, dq4);
#pragma unroll
                for (int x = 0; x < DV; ++x)
                    dq_acc[x] = Mma<T>::mma32(f[s2 * DV + x], df, dq_acc[x]);
            }
        };
        const uint32_t mw0 = mask_word(t, 0), mw1 = mask_word(t, 1);
        rows(kt, 0, kr0);
        rows(vt, 0, vr0);
        __builtin_amdgcn_sched_barrier(0);
        rows(kt, 1, kr1);
        mma_rows(kr0, qf, s_init, s0);
        __builtin_amdgcn_sched_barrier(0);
        rows(vt, 1, vr1);
        mma_rows(vr0, gf, dp_init, p0);
        __builtin_amdgcn_sched_barrier(0);
        cols(0, kq0);
        mma_rows(kr1, qf, s_init, s1);
        half_exp(s0, t, 0, mask_tag);
        __builtin_amdgcn_sched_barrier(0);
        cols(1, kq1);
        mma_rows(vr1, gf, dp_init, p1);
        half_ds(s0, p0, t, 0, mw0, dw0);
        __builtin_amdgcn_sched_barrier(0);
        mma_cols(kq0, dw0);
        half_exp(s1, t, 1, mask_tag);
        half_ds(s1, p1, t, 1, mw1, dw1);
        __builtin_amdgcn_sched_barrier(0);
        mma_cols(kq1, dw1);
    };

    // ---- prologue: tile 0 into LDS ----
    if (n_tiles > 0) {
        ks.fix(t_lo * kBN, a.sk, a.d);
        vs.fix(t_lo * kBN, a.sk, a.d);
        ks.store(k_lds);
        vs.store(v_lds);
        store_bias(0);
    }
    __syncthreads();

    // Iteration r: request tile r+1, process tile r, write tile r+1 into the other ring slot.
    // kFast iterations hold tiles that every wavefront of the workgroup sees in full, so their body
    // is one straight block; the others test activity and masks per wavefront.
    auto iteration = [&](int r, auto fast_tag) __attribute__((always_inline)) {
        constexpr bool kFast = decltype(fast_tag)::value;
        const int t = t_lo + r;
        const bool have_next = r + 1 < n_tiles;
        if (have_next) {
            request((t + 1) * kBN);
        }
        const T* kt = k_lds + (r % kKRing) * kTileElems;
        const T* vt = v_lds + (r % kVRing) * kTileElems;
        bias_tile = bias_lds + (r & 1) * kBN;
        if constexpr (kFast) {
            if constexpr (kStagger)
                tile_body_fast(kt, vt, t, std::integral_constant<int, 0>{});
            else
                tile_body(kt, vt, t, std::integral_constant<int, 0>{});
        } else if (tile_active(t)) {
            // One wavefront per SIMD (head_dim 128, 412-484 registers): nothing else hides the
            // latencies of a masked tile, so it runs the hand-scheduled body as well (dQ at bf16 B4
            // S2048 H16 D128, window 256, p 0.1: 90.8 -> 86.5 us).  With two wavefronts per SIMD
            // the extra copies of that body cost registers (246 -> 256 and 16 spilled at head_dim
            // 64) and gain nothing.
            if constexpr (kStagger && DPAD > 96 && kDrop != 2) {
                if (!tile_needs_mask(t))
                    tile_body_fast(kt, vt, t, std::integral_constant<int, 0>{});
                else if (a.window > 0)
                    tile_body_fast(kt, vt, t, std::integral_constant<int, 2>{});
                else
                    tile_body_fast(kt, vt, t, std::integral_constant<int, 1>{});
            } else {
                if (!tile_needs_mask(t))
                    tile_body(kt, vt, t, std::integral_constant<int, 0>{});
                else if (a.window > 0)
                    tile_body(kt, vt, t, std::integral_constant<int, 2>{});
                else
                    tile_body(kt, vt, t, std::integral_constant<int, 1>{});
            }
        }
        if (have_next) {
            ks.fix((t + 1) * kBN, a.sk, a.d);
            vs.fix((t + 1) * kBN, a.sk, a.d);
            ks.store(k_lds + ((r + 1) % kKRing) * kTileElems);
            vs.store(v_lds + ((r + 1) % kVRing) * kTileElems);
            store_bias((r + 1) & 1);
        }
        __syncthreads();
    };
    // leading tiles that need neither mask nor activity test for any of the 128 queries
    int n_fast = 0;
    if (a.window <= 0 && q0 + kBM <= a.sq) {
        n_fast = a.sk / kBN;
        if (a.causal) n_fast = min(n_fast, (q0 + 1) / kBN);
        n_fast = min(n_fast, n_tiles);
    }
    int r = 0;
    for (; r < n_fast; ++r) iteration(r, std::true_type{});
    for (; r < n_tiles; ++r) iteration(r, std::false_type{});
    // ---- epilogue: dQ = scale * dQ^T^T ----
    // every wavefront is past the last barrier of the loop: the K buffers are free, and each
    // wavefront routes its 32 rows through its own quarter of them
    if (wq0 < a.sq) {
        T* dq_row0 =
            reinterpret_cast<T*>(a.dq) + b * a.dqs[0] + (int64_t)wq0 * a.dqs[1] + h * a.dqs[2];
        const float out_scale = (kDrop != 0 ? a.scale * a.rng.inv_keep : a.scale) * inv_n;
        store_block_via_lds<T, DPAD, kPitch>(dq_acc, out_scale, k_lds + wave * 32 * kPitch,
                                             dq_row0, a.dqs[1], a.sq - wq0, a.d);
    }
}

template <typename T, int DPAD, int kBias, int kDrop, bool kStagger, int kSteps>
int launch(const AttnArgs& a, hipStream_t st) {
    typedef TileStage<T, DPAD, kBN, kThreads> Stage;
    const size_t smem = (size_t)(kKRing + kVRing) * kBN * Stage::kPitch * sizeof(T) +
                        (kBias == 2 ? 2 * kBN * sizeof(float) : 0);
    const int n_qt = (a.sq + kBM - 1) / kBM;
    const int64_t blocks = (int64_t)n_qt * a.batch * a.heads;
    if (blocks <= 0 || blocks > 0x7FFFFFFF) return SLAPO_ERR_SHAPE;
    auto kern = attn_bwd_dq_kernel<T, DPAD, kBias, kDrop, kStagger, kSteps>;
    static std::atomic<uint64_t> lds_ready{0};  // per instantiation, one bit per device
    if (allow_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_ready) != SLAPO_OK)
        return SLAPO_ERR_LAUNCH;
    AttnArgs ordered = a;
    set_dispatch_order(&ordered, blocks, (kStagger && DPAD > 64) ? 1 : 2);
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kThreads), smem, st, ordered);
    return check_launch();
}

template <typename T, int DPAD, bool kStagger, int kSteps = DPAD / 16>
int dispatch_flags(const AttnArgs& a, hipStream_t st) {
    if (a.has_bias) {
        if (a.bs[2] == 0) {  // the bias depends on the key only
            if (a.dropout == 1) return launch<T, DPAD, 2, 1, kStagger, kSteps>(a, st);
            if (a.dropout == 2) return launch<T, DPAD, 2, 2, kStagger, kSteps>(a, st);
            if (a.dropout == 3) return launch<T, DPAD, 2, 3, kStagger, kSteps>(a, st);
            return launch<T, DPAD, 2, 0, kStagger, kSteps>(a, st);
        }
        if (a.dropout == 1) return launch<T, DPAD, 1, 1, kStagger, kSteps>(a, st);
        if (a.dropout == 2) return launch<T, DPAD, 1, 2, kStagger, kSteps>(a, st);
        if (a.dropout == 3) return launch<T, DPAD, 1, 3, kStagger, kSteps>(a, st);
        return launch<T, DPAD, 1, 0, kStagger, kSteps>(a, st);
    }
    if (a.dropout == 1) return launch<T, DPAD, 0, 1, kStagger, kSteps>(a, st);
    if (a.dropout == 2) return launch<T, DPAD, 0, 2, kStagger, kSteps>(a, st);
    if (a.dropout == 3) return launch<T, DPAD, 0, 3, kStagger, kSteps>(a, st);
    return launch<T, DPAD, 0, 0, kStagger, kSteps>(a, st);
}

template <typename T>
int dispatch(const AttnArgs& a, hipStream_t st) {
    if (a.d <= 64) return dispatch_flags<T, 64, true>(a, st);
    if (a.d <= 80) return dispatch_flags<T, 96, false, 5>(a, st);  // five k-steps cover head_dim 80
    if (a.d <= 96) return dispatch_flags<T, 96, false>(a, st);
    if (a.d <= 128) {
        // a local window leaves mostly masked tiles, whose bodies spill at two workgroups per CU;
        // so does the body that applies stored dropout bits (163 spilled registers: 188 against
        // 158 us at bf16 B4 S2048 H16 causal, p 0.1)
        if (a.window > 0 || a.dropout == 3) return dispatch_flags<T, 128, true>(a, st);
        return dispatch_flags<T, 128, false>(a, st);
    }
    return SLAPO_ERR_SHAPE;
}

}  // namespace bwd_dq
}  // namespace slapo
