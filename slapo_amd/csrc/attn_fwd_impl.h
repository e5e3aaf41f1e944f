// Flash-attention forward for gfx950 (fp16 / bf16 inputs, fp32 accumulation).
//
// One workgroup (4 wavefronts) owns 128 consecutive queries of one (batch, head); wavefront w owns
// 32 of them, lane l = one query (lanes l and l + 32 share a query and split the registers' keys
// resp. head-dim slots).  Keys and values stream through LDS in tiles of 64, double buffered and
// staged through registers (the global loads of tile t+1 are in flight while tile t is
// processed).  Per key tile, as two halves of 32 keys:
//   S^T  = K Q^T                  A = K rows from LDS (row-permuted 128-bit reads), B = Q^T regs
//   P^T  = exp2(S^T * scale - m)  online softmax with a lazily moved reference point m
//   O^T += V^T P^T                B = P^T straight from the accumulator registers (the row
//                                 permutation of the K reads makes them ordered k-slots), A = V^T
//                                 read from the row-major V tile with the transposing LDS read.
// The loop is deliberately NOT software pipelined across tiles inside a wavefront: one tile is in
// flight per wavefront and leading tiles that no query of the workgroup needs masks for run as
// one straight block.  That keeps the kernel inside 168 registers at head_dim <= 64 (THREE
// workgroups per CU) and inside 256 above (two), and on this hardware resident wavefronts hide
// more latency than a deeper pipeline inside one wavefront does: a pipelined variant with twice
// the registers measured 12 % slower at head_dim 64 and 35-80 % slower at 80 / 128.
//
// Reference semantics: slapo/op/attention.py:163-181 (attention_bmk), :97-131 (flash_attn_ref).
#pragma once
#include <type_traits>

#include "attn_common.h"

namespace slapo {
namespace fwd {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kBM = kWaves * 32;
constexpr int kBN = 64;
constexpr float kMaxSlack = 8.0f;  // hysteresis of the softmax reference, log2 units

template <typename T, int DPAD, int kBias, int kDrop, int kWin, int kSteps>
__global__ __launch_bounds__(kThreads, (DPAD <= 64 && kDrop == 0 ? 3 : 2)) void attn_fwd_kernel(
    const AttnArgs a_in) {
    // kBias: 0 = no additive bias, 1 = any layout (read from memory per score), 2 = the bias
    // depends on the key only (stride 0 over the queries, e.g. a [B,1,1,Sk] padding mask): the 64
    // values of a key tile travel through LDS beside the K / V tile and the tile body has neither
    // global loads nor branches for them (bf16 B4 S2048 H32 D80 causal, every key valid: 241 us
    // with the per-score reads against 169 us without a bias).
    // kWin: 0 = the launcher guarantees window <= 0, 1 = it guarantees window > 0, 2 = either.
    // Folding "no window" in removes the two-sided mask body and the window tests from the
    // kernel, and with them the register spills of the bias-free builds (head_dim 64: 24 spilled
    // registers -> none, 37.8 -> 35.7 us at fp16 B8 S1024 H16 causal; head_dim 128: 69 -> 4,
    // 116 -> 96-109 us at bf16 B4 S2048 H16 causal); folding "window" in leaves one masked body.
    AttnArgs a = a_in;
    if constexpr (kWin == 0) a.window = 0;
    if constexpr (kDrop == 1 || kDrop == 2) resolve_device_state(a.rng);
    typedef typename Mma<T>::frag frag_t;
    typedef TileStage<T, DPAD, kBN, kThreads> Stage;
    constexpr int kPitch = Stage::kPitch;
    constexpr int kTileElems = kBN * kPitch;
    // k-steps of S^T = K Q^T: DPAD / 16, or one fewer where the launcher guarantees head_dim <=
    // 16 * kSteps (head_dim 80 in the 96-wide build: the sixth step would multiply zeros)
    constexpr int DK = kSteps;
    constexpr int DV = DPAD / 32;  // 32-row blocks of O^T

    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* k_lds = reinterpret_cast<T*>(smem_raw);  // K[2][tile]
    T* v_lds = k_lds + 2 * kTileElems;          // V[2][tile]
    float* bias_lds = reinterpret_cast<float*>(v_lds + 2 * kTileElems);  // [2][kBN], kBias == 2

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
    const int wq0 = q0 + wave * 32;  // first query of this wavefront
    const int q_row = wq0 + i_loc;

    const T* q_base = reinterpret_cast<const T*>(a.q) + b * a.qs[0] + h * a.qs[2];
    const T* k_base = reinterpret_cast<const T*>(a.k) + b * a.ks[0] + h * a.ks[2];
    const T* v_base = reinterpret_cast<const T*>(a.v) + b * a.vs[0] + h * a.vs[2];

    int j_lo, j_hi;
    key_range(a, q0, min(q0 + kBM, a.sq), j_lo, j_hi);
    if constexpr (kBias)  // skip the tiles that hold nothing but padded keys
        j_hi = max(j_lo + 1, min(j_hi, padded_key_limit<kThreads>(
                                           a, b, h, reinterpret_cast<float*>(smem_raw))));
    const int t_lo = j_lo / kBN;
    const int t_hi = (j_hi + kBN - 1) / kBN;
    const int n_tiles = t_hi - t_lo;

    // Start-up loads, all issued before any is used: the Q^T fragments (column i = this lane's
    // query, k-slots = 8 consecutive head-dim elements) and the first K / V tile.  Addresses are
    // clamped into the tensors; what was clamped is zeroed afterwards.
    Stage ks, vs;
    ks.init(a.ks[1], a.d);
    vs.init(a.vs[1], a.d);
    frag_t qf[DK];
    {
        u32x4_t q_raw[DK];
        const int qr = min(q_row, a.sq - 1);
#pragma unroll
        for (int t = 0; t < DK; ++t)
            q_raw[t] = *reinterpret_cast<const u32x4_t*>(q_base + (int64_t)qr * a.qs[1] +
                                                         min(16 * t + 8 * g, a.d - 8));
        ks.load(k_base, a.ks[1], t_lo * kBN, a.sk, a.d);
        vs.load(v_base, a.vs[1], t_lo * kBN, a.sk, a.d);
        // Q is multiplied by scale * log2(e) once, here: the scores leave the matrix pipe in log2
        // units and no per-score multiplication is left in the tile body.
#pragma unroll
        for (int t = 0; t < DK; ++t)
            qf[t] = scale_frag<T>(keep_or_zero(q_raw[t], q_row < a.sq && 16 * t + 8 * g < a.d),
                                  a.scale_log2);
    }

    f32x16_t o_acc[DV];
#pragma unroll
    for (int x = 0; x < DV; ++x)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[x][r] = 0.f;
    // Softmax state of this lane's query, in log2 units (Q carries scale * log2(e)): m_run is the
    // reference point of l_run / o_acc (-inf: nothing accumulated yet), moved lazily.
    float m_run = -INFINITY;
    float m_ref = 0.f;  // what the exponentials subtract: m_run, or 0 while m_run is -inf
    float l_run = 0.f;  // this lane's share of the running sum
    // kRefInMma: the matrix pipe subtracts the reference as well.  One more matrix instruction per
    // tile whose A operand is a constant (kRefUnit in k-slot 0, zeros elsewhere) and whose B
    // operand holds -m_ref / kRefUnit in that slot gives the start value of both score
    // accumulators, so that the scores arrive relative to m_ref and a probability is one
    // v_exp_f32.  The reference must then be a number of T: it is rounded to T when it moves (the
    // row's probabilities and their sum share whatever value is subtracted, so the rounding
    // cancels in the output, and the log-sum-exp is formed from the rounded value), kept within
    // T's range (fp16: |m_ref| <= 60000 * 64 log2 units) and away from T's subnormals.
    // Measured: 28 fewer vector instructions per tile (118 -> 90 at head_dim 64) change nothing at
    // head_dim 64 (32.5 us either way at fp16 B8 S1024 H16 causal, 78.7 / 79.2 us with dropout),
    // cost 3 % at head_dim 128 without dropout and 27 % in the window build that reads stored
    // keep bits, and gain 9 % at head_dim 128 where the kernel draws its dropout bits (bf16 B4
    // S2048 H16 causal, p 0.1: 209 -> 190 us): that build has the most live registers, and the
    // subtractions' operands are what it no longer keeps.  Only that build uses it.  (Builds with
    // a bias could not: the masking value -FLT_MAX is no number of T.)
    constexpr bool kRefInMma = kBias == 0 && (kDrop == 1 || kDrop == 2) && kWin == 0 && DPAD > 96;
    constexpr float kRefUnit = std::is_same<T, f16_t>::value ? 64.f : 1.f;
    frag_t ones_frag, ref_frag;
#pragma unroll
    for (int j = 0; j < 8; ++j) ones_frag[j] = (T)0.f, ref_frag[j] = (T)0.f;
    if (g == 0) ones_frag[0] = (T)kRefUnit;

    const int wq_last = min(wq0 + 31, a.sq - 1);
    uint64_t drop_row_base = 0;
    if constexpr (kDrop != 0)
        drop_row_base = ((uint64_t)bh * a.sq + (uint64_t)q_row) * (uint64_t)a.sk;
    const float* bias_row = nullptr;
    if constexpr (kBias)
        bias_row = a.bias + b * a.bs[0] + h * a.bs[1] + (int64_t)min(q_row, a.sq - 1) * a.bs[2];
    // kBias == 2: thread (x & 63) carries key j0 + (x & 63) of the requested tile (all four
    // wavefronts alike, so that neither request nor store needs a branch)
    const float* bias_keys = nullptr;
    if constexpr (kBias == 2) bias_keys = a.bias + b * a.bs[0] + h * a.bs[1];
    float bias_stage = 0.f;
    auto request_bias = [&](int j0) __attribute__((always_inline)) {
        if constexpr (kBias == 2)
            bias_stage = bias_keys[(int64_t)min(j0 + lane, a.sk - 1) * a.bs[3]];
    };
    auto store_bias = [&](int slot) __attribute__((always_inline)) {
        if constexpr (kBias == 2) bias_lds[slot * kBN + row_slot(lane)] = bias_log2(bias_stage);
    };
    const float* bias_tile = bias_lds;  // the slot of the tile in process
    request_bias(t_lo * kBN);

    // per-lane LDS offsets (elements) that do not change from tile to tile
    const int k_off = pi_row(i_loc) * kPitch + 8 * g;
    const int v_off = tr_lane_off(lane, kPitch);

    // Wavefront-uniform: does tile t hold any visible key for this wavefront's queries?
    auto tile_active = [&](int t) __attribute__((always_inline)) {
        if (wq0 >= a.sq) return false;
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

    // S^T half = K_half Q^T, in log2 units
    auto half_scores = [&](const T* kt, int kb, f32x16_t& s) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
        if constexpr (kRefInMma) s = Mma<T>::mma32(ones_frag, ref_frag, s);
#pragma unroll
        for (int x = 0; x < DK; ++x)
            s = Mma<T>::mma32(lds_frag<T>(kt + kb * 32 * kPitch + k_off + 16 * x), qf[x], s);
    };
    // bias, masks and maximum of one half; mask_tag: 0 = every key visible, 1 = upper bound only
    // (causal / key tail), 2 = both bounds (local window).  Returns this lane's maximum.
    auto finish_half = [&](f32x16_t& s, int t, int kb, auto mask_tag)
                           __attribute__((always_inline)) -> float {
        constexpr int kMask = decltype(mask_tag)::value;
        const int j0 = t * kBN + 32 * kb;
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
        float mx = -INFINITY;
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            if constexpr (kBias == 2) {
                const f32x4_t t4 = *reinterpret_cast<const f32x4_t*>(bias_tile + 32 * kb +
                                                                     quad_slot(r4, g));
                s[4 * r4 + 0] += t4.x;
                s[4 * r4 + 1] += t4.y;
                s[4 * r4 + 2] += t4.z;
                s[4 * r4 + 3] += t4.w;
            }
            if constexpr (kMask != 0) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int c = acc_row(4 * r4 + e, 0);
                    if constexpr (kMask == 2) {
                        if (c > c_hi || c < c_lo) s[4 * r4 + e] = -INFINITY;
                    } else {
                        if (c > c_hi) s[4 * r4 + e] = -INFINITY;
                    }
                }
            }
            mx = fmaxf(mx, fmaxf(fmaxf(s[4 * r4], s[4 * r4 + 1]),
                                 fmaxf(s[4 * r4 + 2], s[4 * r4 + 3])));
        }
        return mx;
    };
    // Moves the reference point if this tile's maximum calls for it (rare after a row's first
    // tile): only when the maximum exceeds it by more than kMaxSlack, so that the rescale of the
    // accumulators stays off the common path.  A row that has met nothing but masked keys
    // sits at -FLT_MAX and moves up to the first real key like any other.
    auto update_reference = [&](float mx, f32x16_t& s0, f32x16_t& s1)
                                __attribute__((always_inline)) {
        if constexpr (!kRefInMma) {
            const bool move = mx > m_run + kMaxSlack && mx != -INFINITY;
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(move) != 0, 0)) {
                // exp2(old reference - new reference); an unset reference (-inf) scales by 0
                const float alpha = (m_run == -INFINITY) ? 0.f : fast_exp2(m_run - mx);
                if (move) {
                    m_run = mx;
                    m_ref = mx;
                    l_run *= alpha;
#pragma unroll
                    for (int x = 0; x < DV; ++x)
#pragma unroll
                        for (int r = 0; r < 16; ++r) o_acc[x][r] *= alpha;
                }
            }
        } else {
            // mx is relative to m_ref here (the scores left the matrix pipe that way)
            const bool move = (m_run == -INFINITY) ? mx != -INFINITY : mx > kMaxSlack;
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(move) != 0, 0)) {
                // the new reference as a number of T (times kRefUnit), in range and normal
                constexpr float kTop = std::is_same<T, f16_t>::value ? 60000.f : 3.0e38f;
                constexpr float kTiny = std::is_same<T, f16_t>::value ? 6.2e-5f : 1.2e-38f;
                float x = -(m_ref + mx) * (1.0f / kRefUnit);
                x = fminf(fmaxf(x, -kTop), kTop);
                if (fabsf(x) < kTiny) x = 0.f;
                const T xt = (T)x;
                const float m_new = -(float)xt * kRefUnit;
                const float alpha = (m_run == -INFINITY) ? 0.f : fast_exp2(m_run - m_new);
                if (move) {
                    const float shift = m_new - m_ref;  // this tile's scores move with it
#pragma unroll
                    for (int r = 0; r < 16; ++r) s0[r] -= shift, s1[r] -= shift;
                    m_run = m_new;
                    m_ref = m_new;
                    if (g == 0) ref_frag[0] = xt;
                    l_run *= alpha;
#pragma unroll
                    for (int x2 = 0; x2 < DV; ++x2)
#pragma unroll
                        for (int r = 0; r < 16; ++r) o_acc[x2][r] *= alpha;
                }
            }
        }
    };
    // Keep bits of this lane's query for the 32 keys from j0 on (bit j = key j0 + j), drawn here:
    // Philox blocks cover four consecutive keys; the two lanes of a query (l, l ^ 32) draw the
    // blocks of keys 8 g .. 8 g + 7 of each 16-key group and exchange them.
    auto draw_half = [&](int j0) __attribute__((always_inline)) -> uint32_t {
        uint32_t mine = 0;
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
            mine |= bits << pos;
        }
        return or_xor32(mine);
    };
    // probabilities of one half: exp2, dropout, pack to T, row sum
    // (drop_bits: the keep bits of this lane's query for the 32 keys of the half; kDrop == 3
    // passes in the word that keep_mask_kernel stored, the other modes return the drawn one)
    auto half_prob = [&](f32x16_t& s, int t, int kb, uint32_t (&pw)[8], uint32_t& drop_bits)
                         __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = fast_exp2(kRefInMma ? s[r] : s[r] - m_ref);
        if constexpr (kDrop != 0) {
            float psum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) psum += s[r];
            l_run += psum;
            uint32_t mine = drop_bits;
            if constexpr (kDrop != 3) mine = draw_half(t * kBN + 32 * kb);
            const uint32_t mine_g = mine >> (kAccGroupStep * g);
            // dropped probabilities become +0 (two instructions each); the factor 1 / (1 - p) of
            // the kept ones goes onto the output rows when they are written
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = keep_or_zero(s[r], mine_g, acc_row(r, 0));
            drop_bits = mine;
#pragma unroll
            for (int r2 = 0; r2 < 8; ++r2) pw[r2] = pack2<T>(s[2 * r2], s[2 * r2 + 1]);
        } else {
            // Without dropout the row sum is taken over the rounded probabilities, two per
            // instruction (v_dot2c_f32_{f16,bf16} against a pair of ones): the normaliser then
            // belongs to exactly the numbers that multiply V.
#pragma unroll
            for (int r2 = 0; r2 < 8; ++r2) {
                pw[r2] = pack2<T>(s[2 * r2], s[2 * r2 + 1]);
                l_run = sum2<T>(pw[r2], l_run);
            }
        }
    };
    // O^T += V_half^T P_half^T
    auto half_accumulate = [&](const T* vt, int kb, const uint32_t (&pw)[8])
                               __attribute__((always_inline)) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            u32x4_t pq = {pw[4 * s2], pw[4 * s2 + 1], pw[4 * s2 + 2], pw[4 * s2 + 3]};
            const frag_t pf = __builtin_bit_cast(frag_t, pq);
#pragma unroll
            for (int x = 0; x < DV; ++x)
                o_acc[x] = Mma<T>::mma32(
                    lds_frag_tr<T>(vt + (32 * kb + 16 * s2) * kPitch + v_off + 32 * x, kPitch), pf,
                    o_acc[x]);
        }
    };
    auto tile_body = [&](const T* kt, const T* vt, int t, auto mask_tag)
                         __attribute__((always_inline)) {
        f32x16_t s0, s1;
        uint32_t pw0[8], pw1[8];
        uint32_t bits0 = 0, bits1 = 0;
        if constexpr (kDrop == 3) {
            // the keep bits of this lane's query for the two halves of the tile, drawn by
            // keep_mask_kernel; requested first, used after the scores
            const int w = 2 * t;
            const int64_t base = (int64_t)bh * a.mask_words;
            const int row = min(q_row, a.sq - 1);
            bits0 = a.keep_mask[(base + min(w, a.mask_words - 1)) * a.mask_pitch + row];
            bits1 = a.keep_mask[(base + min(w + 1, a.mask_words - 1)) * a.mask_pitch + row];
        }
        half_scores(kt, 0, s0);
        half_scores(kt, 1, s1);
        const float mx =
            max_xor32(fmaxf(finish_half(s0, t, 0, mask_tag), finish_half(s1, t, 1, mask_tag)));
        update_reference(mx, s0, s1);
        half_prob(s0, t, 0, pw0, bits0);
        half_accumulate(vt, 0, pw0);
        half_prob(s1, t, 1, pw1, bits1);
        half_accumulate(vt, 1, pw1);
        // With dropout and a keep_mask buffer: one word per query and half for the backward.
        // The (wavefront-uniform) branch sits at the end of the tile, where the basic block ends
        // anyway; inside the body it would keep the scheduler from mixing the Philox arithmetic
        // with the matrix instructions (10 % of the forward).
        if constexpr (kDrop == 1 || kDrop == 2) {
            if (a.keep_mask != nullptr) {
                const uint32_t w0 = bits0, w1 = bits1;  // already combined over the lane pair
                uint32_t* row = a.keep_mask +
                                ((int64_t)bh * a.mask_words + 2 * t) * a.mask_pitch + q_row;
                if (g == 0 && q_row < a.sq) {
                    if (t * kBN < a.sk) row[0] = w0;
                    if (t * kBN + 32 < a.sk) row[a.mask_pitch] = w1;
                }
            }
        }
    };

    // ---- prologue: tile 0 into LDS ----
    ks.fix(t_lo * kBN, a.sk, a.d);
    vs.fix(t_lo * kBN, a.sk, a.d);
    ks.store(k_lds);
    vs.store(v_lds);
    store_bias(0);
    __syncthreads();

    // Iteration r: request tile r+1, process tile r, write tile r+1 into the other slot.
    // kFast iterations hold tiles that every wavefront of the workgroup sees in full.
    auto iteration = [&](int r, auto fast_tag) __attribute__((always_inline)) {
        constexpr bool kFast = decltype(fast_tag)::value;
        const int t = t_lo + r;
        const bool have_next = r + 1 < n_tiles;
        // the next tile is requested unconditionally (rows are clamped into the tensor; after the
        // last tile the request is wasted) so that it stays straight-line code.  Requesting it
        // later in the body saves no registers and measures slower.  (Addresses: a scalar tile
        // base plus a per-lane 32-bit offset that is selected, not multiplied out: 2 % faster than
        // the multiplied-out form now that the tile body has no other address arithmetic.)
        ks.load(k_base, a.ks[1], (t + 1) * kBN, a.sk, a.d);
        vs.load(v_base, a.vs[1], (t + 1) * kBN, a.sk, a.d);
        request_bias((t + 1) * kBN);
        const T* kt = k_lds + (r & 1) * kTileElems;
        const T* vt = v_lds + (r & 1) * kTileElems;
        bias_tile = bias_lds + (r & 1) * kBN;
        if constexpr (kFast) {
            tile_body(kt, vt, t, std::integral_constant<int, 0>{});
        } else {
            if (tile_active(t)) {
                if (!tile_needs_mask(t))
                    tile_body(kt, vt, t, std::integral_constant<int, 0>{});
                else if constexpr (kWin == 1)  // one masked body per build: both bounds
                    tile_body(kt, vt, t, std::integral_constant<int, 2>{});
                else if (kWin == 2 && a.window > 0)
                    tile_body(kt, vt, t, std::integral_constant<int, 2>{});
                else
                    tile_body(kt, vt, t, std::integral_constant<int, 1>{});
            }
        }
        if (have_next) {
            ks.fix((t + 1) * kBN, a.sk, a.d);
            vs.fix((t + 1) * kBN, a.sk, a.d);
            ks.store(k_lds + ((r + 1) & 1) * kTileElems);
            vs.store(v_lds + ((r + 1) & 1) * kTileElems);
            store_bias((r + 1) & 1);
        }
        __syncthreads();
    };
    // tiles that need neither mask nor activity test for any of the 128 queries: the leading
    // ones without a local window, a run in the middle of the key range with one
    if constexpr (kWin != 1) {
        int n_fast = 0;
        if (a.window <= 0 && q0 + kBM <= a.sq) {
            n_fast = a.sk / kBN;
            if (a.causal) n_fast = min(n_fast, (q0 + 1) / kBN);
            n_fast = min(n_fast, n_tiles);
        }
        int r = 0;
        for (; r < n_fast; ++r) iteration(r, std::true_type{});
        for (; r < n_tiles; ++r) iteration(r, std::false_type{});
    } else {
        int f_lo = 0, f_hi = 0;  // iterations [f_lo, f_hi) are fast
        if (q0 + kBM <= a.sq) {
            int t_end = a.sk / kBN;  // first tile that is incomplete or hidden from some query
            if (a.causal) t_end = min(t_end, (q0 + 1) / kBN);
            // the last query of the workgroup sees keys >= q0 + kBM - window
            const int t_begin = (max(q0 + kBM - a.window, 0) + kBN - 1) / kBN;
            f_lo = min(max(t_begin - t_lo, 0), n_tiles);
            f_hi = min(max(t_end - t_lo, f_lo), n_tiles);
        }
        for (int r = 0; r < n_tiles; ++r) {
            if (r >= f_lo && r < f_hi)
                iteration(r, std::true_type{});
            else
                iteration(r, std::false_type{});
        }
    }

    // ---- epilogue ----
    const float l_tot = sum_xor32(l_run);
    const float inv_l = kDrop != 0 ? a.rng.inv_keep / l_tot : 1.0f / l_tot;
    // every wavefront is past the last barrier of the loop: the K buffers are free, and each
    // wavefront routes its 32 output rows through its own quarter of them
    if (wq0 < a.sq) {
        T* o_row0 = reinterpret_cast<T*>(a.o) + b * a.os[0] + (int64_t)wq0 * a.os[1] + h * a.os[2];
        store_block_via_lds<T, DPAD, kPitch>(o_acc, inv_l, k_lds + wave * 32 * kPitch, o_row0,
                                             a.os[1], a.sq - wq0, a.d);
    }
    if (q_row < a.sq) {
        // A row that met nothing but masked keys (bias_log2) sits at -FLT_MAX with l_tot = their
        // number: the row sum goes out in place of the log-sum-exp, scaled by 2^100.
        if (g == 0)
            a.lse[(int64_t)bh * a.sq + q_row] = m_run == -kFltMax
                                                    ? l_tot * kMaskedRowLse
                                                    : (m_run + __builtin_log2f(l_tot)) * kLn2;
    }
}

template <typename T, int DPAD, int kBias, int kDrop, int kWin, int kSteps>
int launch(const AttnArgs& a, hipStream_t st) {
    typedef TileStage<T, DPAD, kBN, kThreads> Stage;
    const size_t smem = (size_t)4 * kBN * Stage::kPitch * sizeof(T) +
                        (kBias == 2 ? 2 * kBN * sizeof(float) : 0);
    const int n_qt = (a.sq + kBM - 1) / kBM;
    const int64_t blocks = (int64_t)n_qt * a.batch * a.heads;
    if (blocks <= 0 || blocks > 0x7FFFFFFF) return SLAPO_ERR_SHAPE;
    auto kern = attn_fwd_kernel<T, DPAD, kBias, kDrop, kWin, kSteps>;
    static std::atomic<uint64_t> lds_ready{0};  // per instantiation, one bit per device
    if (allow_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_ready) != SLAPO_OK)
        return SLAPO_ERR_LAUNCH;
    AttnArgs ordered = a;
    // (head groups: not where the kernel draws or applies dropout bits -- its workgroups run twice as
    // long there and a group's late heavy ones become the tail: 314 -> 350 us at bf16 B4 S2048 H32
    // D80 causal, p 0.1, 588 -> 667 us at fp16 B2 S4096 H32 D96)
    set_dispatch_order(&ordered, blocks, (DPAD <= 64 && kDrop == 0) ? 3 : 2, kDrop == 0);
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kThreads), smem, st, ordered);
    return check_launch();
}

template <typename T, int DPAD, int kWin, int kSteps>
int dispatch_nobias(const AttnArgs& a, hipStream_t st) {
    if (a.dropout == 1) return launch<T, DPAD, 0, 1, kWin, kSteps>(a, st);
    if (a.dropout == 2) return launch<T, DPAD, 0, 2, kWin, kSteps>(a, st);
    if (a.dropout == 3) {  // stored keep bits: local-window calls only, see attn_capi.hip
        if constexpr (kWin != 0)
            return launch<T, DPAD, 0, 3, kWin, kSteps>(a, st);
        else
            return SLAPO_ERR_ARG;
    }
    return launch<T, DPAD, 0, 0, kWin, kSteps>(a, st);
}
template <typename T, int DPAD, int kSteps = DPAD / 16>
int dispatch_flags(const AttnArgs& a, hipStream_t st) {
    if (a.has_bias) {
        // one build for both: with a bias the window-free build measured slower (it spills more
        // at head_dim 64 and 96: 266 against 185 us at bf16 B4 S2048 H32 D80 with a padding mask)
        if (a.bs[2] == 0) {  // the bias depends on the key only
            if (a.dropout == 1) return launch<T, DPAD, 2, 1, 2, kSteps>(a, st);
            if (a.dropout == 2) return launch<T, DPAD, 2, 2, 2, kSteps>(a, st);
            if (a.dropout == 3) return launch<T, DPAD, 2, 3, 2, kSteps>(a, st);
            if (a.window <= 0) return launch<T, DPAD, 2, 0, 0, kSteps>(a, st);
            return launch<T, DPAD, 2, 0, 2, kSteps>(a, st);
        }
        if (a.dropout == 1) return launch<T, DPAD, 1, 1, 2, kSteps>(a, st);
        if (a.dropout == 2) return launch<T, DPAD, 1, 2, 2, kSteps>(a, st);
        if (a.dropout == 3) return launch<T, DPAD, 1, 3, 2, kSteps>(a, st);
        return launch<T, DPAD, 1, 0, 2, kSteps>(a, st);
    }
    return a.window > 0 ? dispatch_nobias<T, DPAD, 1, kSteps>(a, st)
                        : dispatch_nobias<T, DPAD, 0, kSteps>(a, st);
}

template <typename T>
int dispatch(const AttnArgs& a, hipStream_t st) {
    if (a.d <= 64) return dispatch_flags<T, 64>(a, st);
    if (a.d <= 80) return dispatch_flags<T, 96, 5>(a, st);  // five k-steps cover head_dim 80
    if (a.d <= 96) return dispatch_flags<T, 96>(a, st);
    if (a.d <= 128) return dispatch_flags<T, 128>(a, st);
    return SLAPO_ERR_SHAPE;
}

}  // namespace fwd
}  // namespace slapo
