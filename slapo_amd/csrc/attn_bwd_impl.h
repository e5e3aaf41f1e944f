// Flash-attention backward, dK / dV half, for gfx950 (fp16 / bf16 inputs, fp32 accumulation).
//
// One workgroup (4 wavefronts) owns 128 consecutive keys of one (batch, head); wavefront w owns
// 32 of them and keeps their K and V fragments in registers for the whole kernel, together with
// its dK^T and dV^T accumulators.  Query tiles of 64 rows (Q, dO, lse, delta) stream through LDS,
// double buffered and staged through registers.  Per 32-query half tile and wavefront (lane l,
// g = l / 32):
//   S  = Q K_w^T, dP = dO V_w^T      A = Q / dO rows from LDS (row-permuted 128-bit reads),
//                                    B = the resident K_w / V_w fragments (K_w carries scale *
//                                    log2(e)).  Lane l holds one KEY column; registers run over
//                                    16 query rows.  The accumulators start from -lse and -delta
//                                    of their query rows (128-bit LDS reads straight into the
//                                    accumulator registers), so that
//   P  = exp2(S), dS = P * dP        cost two vector instructions per score; P is recomputed from
//                                    the saved log-sum-exp; dropout bits regenerated from Philox
//                                    or read back from the forward's keep words.
//   dV_w^T += dO^T P, dK_w^T += Q^T dS    B = P / dS straight from the accumulator registers
//                                    (the row permutation makes them ordered k-slots), A = dO^T /
//                                    Q^T read from the same row-major LDS tiles with the
//                                    transposing LDS read.
// The two halves of a tile are staggered so that the matrix instructions of one half have vector
// work of the other half around them (a wavefront overlaps the two only when they are interleaved
// in its instruction stream).  dQ is produced by the sibling kernel that owns query rows, so
// nothing here is shared between workgroups.  One barrier per query tile.
// Reference semantics: autograd of slapo/op/attention.py:163-181.
#pragma once
#include <type_traits>

#include "attn_common.h"

namespace slapo {
namespace bwd {

constexpr int kBwdWaves = 4;
constexpr int kBwdThreads = kBwdWaves * 64;
constexpr int kBwdBM = 64;  // queries per tile

template <typename T, int DPAD>
struct BwdSmem {
    typedef TileStage<T, DPAD, kBwdBM, kBwdThreads> QStage;
    static constexpr int kPitch = QStage::kPitch;
    static constexpr int kQTile = kBwdBM * kPitch;            // elements
    static constexpr size_t kQBytes = 2 * kQTile * sizeof(T);   // double buffered
    static constexpr size_t kStatBytes = 2 * 2 * kBwdBM * sizeof(float);  // lse, delta; x2 buffers
    // dropout keep bits of a query tile: one word per wavefront (32 keys) and query; x2 buffers
    static constexpr size_t kMaskBytes = 2 * kBwdWaves * kBwdBM * sizeof(uint32_t);
    static constexpr size_t kBytes = 2 * kQBytes + kStatBytes + kMaskBytes;
};

constexpr bool bwd_two_per_cu(int dpad, int drop, int kb) {
    return kb == 1 && (dpad <= 64 || (dpad == 96 && drop != 3));
}

// KB = blocks of 32 keys per wavefront.  KB = 2 halves the LDS operand traffic per matrix
// instruction (every Q / dO fragment read feeds two MFMAs) at the price of twice the resident
// fragments and accumulators, i.e. one wavefront per SIMD instead of two.
template <typename T, int DPAD, int kBias, int kDrop, int KB, int kSteps>
// Two workgroups per CU up to DPAD 96, one at 128 (192 resident accumulator / fragment registers)
// and at 96 with the forward's keep bits (measured 23-35 % slower with two than with one).
__global__ __launch_bounds__(kBwdThreads, (bwd_two_per_cu(DPAD, kDrop, KB) ? 2 : 1)) void attn_bwd_kernel(
    const AttnArgs a_in) {
    AttnArgs a = a_in;
    if constexpr (kDrop == 1 || kDrop == 2) resolve_device_state(a.rng);
    static_assert(kDrop != 3 || KB == 1, "the keep-bit tile holds one word per wavefront and query");
    typedef typename Mma<T>::frag frag_t;
    typedef BwdSmem<T, DPAD> SM;
    typedef typename SM::QStage QStage;
    constexpr int kPitch = SM::kPitch;
    // k-steps over the head dimension: DPAD / 16, or one fewer where the launcher guarantees
    // head_dim <= 16 * kSteps (head_dim 80 in the 96-wide build)
    constexpr int DK = kSteps;
    constexpr int DV = DPAD / 32;          // 32-row blocks of dK^T / dV^T
    constexpr int kWaveKeys = 32 * KB;
    constexpr int kBN = kBwdWaves * kWaveKeys;  // keys per workgroup

    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* q_lds = reinterpret_cast<T*>(smem_raw);
    T* g_lds = reinterpret_cast<T*>(smem_raw + SM::kQBytes);
    float* stat_lds = reinterpret_cast<float*>(smem_raw + 2 * SM::kQBytes);
    uint32_t* mask_lds = reinterpret_cast<uint32_t*>(smem_raw + 2 * SM::kQBytes + SM::kStatBytes);

    const int n_bh = a.batch * a.heads;
    const int work = work_index(a);
    const int bh = work % n_bh;
    const int kt = work / n_bh;  // low key tiles see the most queries under a causal mask
    const int b = bh / a.heads;
    const int h = bh % a.heads;
    const int k0 = kt * kBN;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wavefront-uniform
    const int g = lane >> 5;
    const int c_loc = lane & 31;
    const int kw0 = k0 + wave * kWaveKeys;  // first key of this wavefront
    int key[KB];                            // this lane's key column in each block
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) key[kb] = kw0 + 32 * kb + c_loc;

    const T* q_base = reinterpret_cast<const T*>(a.q) + b * a.qs[0] + h * a.qs[2];
    const T* k_base = reinterpret_cast<const T*>(a.k) + b * a.ks[0] + h * a.ks[2];
    const T* v_base = reinterpret_cast<const T*>(a.v) + b * a.vs[0] + h * a.vs[2];
    const T* g_base = reinterpret_cast<const T*>(a.dout) + b * a.os[0] + h * a.os[2];
    const float* lse_base = a.lse + (int64_t)bh * a.sq;
    const float* delta_base = a.delta + (int64_t)bh * a.sq;
    // With dropout dS = P (M dP / (1 - p) - delta) is taken as (P (M dP - delta (1 - p))) / (1 - p):
    // delta is scaled when it is staged and the factor goes onto the dK rows when they are written.
    const float keep_prob = a.rng.inv_keep > 0.f ? 1.0f / a.rng.inv_keep : 0.f;

    // ---- resident fragments ----
    // Loaded with clamped addresses and masked once the first query tile has been requested too,
    // so that all start-up loads of the workgroup are in flight together.
    frag_t kf[KB][DK], vf[KB][DK];
    u32x4_t k_raw[KB][DK], v_raw[KB][DK];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
        const int kr = min(key[kb], a.sk - 1);
#pragma unroll
        for (int t = 0; t < DK; ++t) {
            const int dc = min(16 * t + 8 * g, a.d - 8);
            k_raw[kb][t] = *reinterpret_cast<const u32x4_t*>(k_base + (int64_t)kr * a.ks[1] + dc);
            v_raw[kb][t] = *reinterpret_cast<const u32x4_t*>(v_base + (int64_t)kr * a.vs[1] + dc);
        }
    }

    f32x16_t dk_acc[KB][DV], dv_acc[KB][DV];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int x = 0; x < DV; ++x)
#pragma unroll
            for (int r = 0; r < 16; ++r) dk_acc[kb][x][r] = 0.f, dv_acc[kb][x][r] = 0.f;

    int i_lo, i_hi;
    query_range(a, k0, min(k0 + kBN, a.sk), i_lo, i_hi);
    if constexpr (kBias) {  // a workgroup that owns nothing but padded keys has dK = dV = 0
        if (k0 >= padded_key_limit<kBwdThreads>(a, b, h, reinterpret_cast<float*>(smem_raw)))
            i_hi = i_lo;
    }
    const int t_lo = i_lo / kBwdBM;
    const int t_hi = (i_hi + kBwdBM - 1) / kBwdBM;

    // kBias: 0 = none, 1 = any layout (read from memory per score), 2 = the launcher guarantees a
    // bias that does not depend on the query (stride 0 over the queries, the compact [B,1,1,Sk]
    // layout): one register per lane and key block.
    constexpr bool bias_per_key = kBias == 2;
    float bias_k[KB];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
        bias_k[kb] = 0.f;
        if constexpr (kBias) {
            if (bias_per_key && key[kb] < a.sk)
                bias_k[kb] =
                    bias_log2(a.bias[b * a.bs[0] + h * a.bs[1] + (int64_t)key[kb] * a.bs[3]]);
        }
    }
    // per-lane LDS offsets (elements) that do not change from tile to tile
    const int a_off = pi_row(c_loc) * kPitch + 8 * g;
    const int t_off = tr_lane_off(lane, kPitch);

    // Registers through which a query tile (Q, dO rows, lse / delta, keep bits) travels from
    // global memory to LDS.
    struct TileRegs {
        QStage q, g;
        float stat;
        uint32_t mask;
        float row_lse;  // kBias: lse of tile row (thread & 63), in every wavefront
    };
    TileRegs regs;
    regs.q.init(a.qs[1], a.d);
    regs.g.init(a.os[1], a.d);
    regs.stat = 0.f, regs.mask = 0u;
    regs.row_lse = 0.f;
    int masked_pending = 0, masked_tile[2] = {0, 0};  // staged tiles that sync_staged must fix
    // lse / delta of a query tile: threads 0..63 fetch lse, threads 64..127 delta.
    const float* stat_src = (threadIdx.x < kBwdBM) ? lse_base : delta_base;
    // Requests tile t.  Unconditional: rows are clamped into the tensor (past the last tile the
    // request is wasted), so it stays straight-line code; nothing is touched until stage_tile.
    auto request_tile = [&](TileRegs& r, int t) __attribute__((always_inline)) {
        const int i0 = t * kBwdBM;
        r.q.load(q_base, a.qs[1], i0, a.sq, a.d);
        r.g.load(g_base, a.os[1], i0, a.sq, a.d);
        // every thread loads (the upper half of the workgroup a duplicate that stage_tile drops):
        // a branch here would end the basic block in the middle of a tile body, and the
        // exponentials of the body then sink below it, away from the matrix instructions that
        // are meant to run beside them (bf16 B4 S2048 H32 D80 causal: 289 -> 263 us; head_dim 128
        // with dropout: 236 -> 221 us; head_dim 64: 1-3 %).  Only head_dim 128 without dropout,
        // which requests at the top of the body, measured better with the branch (659 against
        // 697 us at S 4096) and keeps it.
        if (!(DPAD > 96 && kDrop == 0) || threadIdx.x < 2 * kBwdBM)
            r.stat = stat_src[min(i0 + (int)(threadIdx.x & (kBwdBM - 1)), a.sq - 1)];
        if constexpr (kBias) r.row_lse = lse_base[min(i0 + (int)(threadIdx.x & 63), a.sq - 1)];
        if constexpr (kDrop == 3) {
            // the keep bits that the forward stored: thread (w, row) of the workgroup fetches the
            // word of query row i0 + row for the 32 keys of wavefront w
            const int w = min((k0 >> 5) + (int)(threadIdx.x >> 6), a.mask_words - 1);
            const int row = min(i0 + (int)(threadIdx.x & 63), a.mask_pitch - 1);
            r.mask = a.keep_mask[((int64_t)bh * a.mask_words + w) * a.mask_pitch + row];
        }
    };
    // Writes the requested tile t into its LDS buffer (tiles alternate between two buffers).
    auto stage_tile = [&](TileRegs& r, int t) __attribute__((always_inline)) {
        const int buf = (t - t_lo) & 1;
        const int i0 = t * kBwdBM;
        r.q.fix(i0, a.sq, a.d);
        r.g.fix(i0, a.sq, a.d);
        if constexpr (kBias) {
            // Every wavefront holds the 64 lse values of the tile, one per lane, so all of them
            // agree on whether the tile has a row that saw nothing but masked keys; see
            // sync_staged for what happens then.
            if (__builtin_amdgcn_ballot_w64(masked_row_lse(r.row_lse)) != 0)
                masked_pending |= 1 << buf, masked_tile[buf] = t;
        }
        r.q.store(q_lds + buf * SM::kQTile);
        r.g.store(g_lds + buf * SM::kQTile);
        if (threadIdx.x < 2 * kBwdBM) {
            const bool ok = i0 + (int)(threadIdx.x & (kBwdBM - 1)) < a.sq;
            // what the accumulators start from: -lse in log2 units (-inf past the end, so that
            // P = 0 there) and, without dropout, -delta; kept at row_slot so that one 128-bit
            // read returns the values of four accumulator registers in order
            const float v = (threadIdx.x < kBwdBM)
                                ? (ok ? -(kBias ? lse_reference(r.stat, kLog2e) : r.stat * kLog2e)
                                      : -INFINITY)
                                : (ok ? (kDrop == 0 ? -r.stat : r.stat * keep_prob) : 0.f);
            stat_lds[buf * 2 * kBwdBM + (threadIdx.x & kBwdBM) + row_slot(threadIdx.x & (kBwdBM - 1))] = v;
        }
        if constexpr (kDrop == 3)
            mask_lds[buf * kBwdThreads + (threadIdx.x & ~63) + row_slot(threadIdx.x & 63)] = r.mask;
    };
    // The barrier after a stage_tile.  Rows that saw nothing but masked keys (bias_log2) have
    // probabilities exp2(x + FLT_MAX) / n: the division goes onto their row of dO (and, in the dQ
    // kernel, onto the delta it stored), which puts it into dV, dP and dS alike.  It is applied to
    // the staged tile in LDS, each thread on the chunks it wrote, behind a test that is uniform
    // over the workgroup and false for every tile of an ordinary call.
    auto sync_staged = [&]() __attribute__((always_inline)) {
        __syncthreads();
        if constexpr (kBias) {
            if (__builtin_expect(masked_pending != 0, 0)) {
#pragma unroll 1
                for (int buf = 0; buf < 2; ++buf) {
                    if (!(masked_pending >> buf & 1)) continue;
                    const int i0 = masked_tile[buf] * kBwdBM;
                    T* tile = g_lds + buf * SM::kQTile;
#pragma unroll
                    for (int u = 0; u < QStage::kPerThread; ++u) {
                        const int c = threadIdx.x + u * kBwdThreads;
                        if (QStage::kChunks % kBwdThreads != 0 && c >= QStage::kChunks) continue;
                        const int row = c / QStage::kChunksPerRow, cc = c % QStage::kChunksPerRow;
                        const float f = lse_row_factor(lse_base[min(i0 + row, a.sq - 1)]);
                        u32x4_t* p = reinterpret_cast<u32x4_t*>(tile + row * kPitch + cc * 8);
                        *p = __builtin_bit_cast(u32x4_t, scale_frag<T>(*p, f));
                    }
                }
                masked_pending = 0;
                __syncthreads();
            }
        }
    };
    auto tile_fast = [&](int t) __attribute__((always_inline)) {
        const int i0 = t * kBwdBM;
        // every (query, key) pair of the tile is visible: the first query sees the last key
        // (causal), the last query still sees the first key (local window)
        return k0 + kBN <= a.sk && i0 + kBwdBM <= a.sq && (!a.causal || i0 >= k0 + kBN - 1) &&
               (a.window <= 0 || i0 + kBwdBM - 1 - k0 < a.window);
    };
    // Two generic (diagonal / tail) tiles in a row are processed together, see generic_step; when
    // the kernel starts with such a pair, both tiles are requested at once.
    // (Measured: 3.5 % on the kernel at head_dim 128, 15 % with a local window; at 64 the second
    // register set spills and costs more than the pairing saves, at 80 it is a wash.)
    constexpr bool kPairGeneric = DPAD > 96;
    const bool pair_first =
        kPairGeneric && t_lo + 1 < t_hi && !tile_fast(t_lo) && !tile_fast(t_lo + 1);
    TileRegs second = regs;  // same lane offsets

    request_tile(regs, t_lo);
    if constexpr (kPairGeneric) request_tile(second, t_lo + 1);
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int t = 0; t < DK; ++t) {
            const bool keep = key[kb] < a.sk && 16 * t + 8 * g < a.d;
            // K times scale * log2(e), once: the scores leave the matrix pipe in log2 units
            kf[kb][t] = scale_frag<T>(keep_or_zero(k_raw[kb][t], keep), a.scale_log2);
            vf[kb][t] = __builtin_bit_cast(frag_t, keep_or_zero(v_raw[kb][t], keep));
        }
    if (t_lo < t_hi) stage_tile(regs, t_lo);
    if constexpr (kPairGeneric) {
        if (pair_first) stage_tile(second, t_lo + 1);
    }
    sync_staged();

    // wavefront-uniform: does the 32-query half tile at ih0 see any key of this wavefront?
    auto half_active = [&](int ih0) __attribute__((always_inline)) {
        const int i_last = min(ih0 + 32, a.sq) - 1;
        if (kw0 >= a.sk || ih0 >= a.sq) return false;
        if (a.causal && kw0 > i_last) return false;
        if (a.window > 0 && ih0 - (kw0 + kWaveKeys - 1) >= a.window) return false;
        return true;
    };
    auto half_needs_mask = [&](int ih0) __attribute__((always_inline)) {
        const int i_last = min(ih0 + 32, a.sq) - 1;
        return (kw0 + kWaveKeys > a.sk) || (a.causal && kw0 + kWaveKeys - 1 > ih0) ||
               (a.window > 0 && i_last - kw0 >= a.window);
    };

    // ---- stages of one half tile (32 queries at ih0 = i0 + 32 hf) ----
    // S = Q_h K_w^T, dP = dO_h V_w^T: every Q / dO fragment read feeds KB matrix instructions
    auto half_sp = [&](const T* qt, const T* gt, const float* lse_h, const float* delta_h, int hf,
                       f32x16_t (&s)[KB], f32x16_t (&dp)[KB]) __attribute__((always_inline)) {
        f32x16_t s_init, dp_init;
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const f32x4_t l4 = *reinterpret_cast<const f32x4_t*>(lse_h + quad_slot(r4, g));
            f32x4_t d4 = {0.f, 0.f, 0.f, 0.f};
            if constexpr (kDrop == 0) d4 = *reinterpret_cast<const f32x4_t*>(delta_h + quad_slot(r4, g));
#pragma unroll
            for (int e = 0; e < 4; ++e) s_init[4 * r4 + e] = l4[e], dp_init[4 * r4 + e] = d4[e];
        }
        const T* qrow = qt + 32 * hf * kPitch + a_off;
        const T* grow = gt + 32 * hf * kPitch + a_off;
#pragma unroll
        for (int x = 0; x < DK; ++x) {
            const frag_t qa = lds_frag<T>(qrow + 16 * x);
            const frag_t ga = lds_frag<T>(grow + 16 * x);
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                s[kb] = Mma<T>::mma32(qa, kf[kb][x], x == 0 ? s_init : s[kb]);
                dp[kb] = Mma<T>::mma32(ga, vf[kb][x], x == 0 ? dp_init : dp[kb]);
            }
        }
    };
    // scores -> probabilities in place.  mask_tag: 0 = all visible, 1 = lower bound on the query
    // only (causal / key tail), 2 = both bounds (local window)
    auto half_exp = [&](f32x16_t (&s)[KB], const float* lse_h, int ih0, auto mask_tag)
                        __attribute__((always_inline)) {
        constexpr int kMask = decltype(mask_tag)::value;
        // register r is query ih0 + acc_row(r, g) = ih0 + kAccGroupStep g + c with
        // c = acc_row(r, 0); visible iff c_lo <= c <= c_hi
        int c_lo[KB], c_hi[KB];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            c_lo[kb] = 0, c_hi[kb] = 0;
            if constexpr (kMask != 0) {
                c_lo[kb] = (key[kb] < a.sk)
                               ? (a.causal ? key[kb] - ih0 - kAccGroupStep * g : -1)
                               : 64;
                if constexpr (kMask == 2)
                    c_hi[kb] = key[kb] + a.window - 1 - ih0 - kAccGroupStep * g;
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                float x = s[kb][r];  // scale and lse are in already
                if constexpr (kBias == 2) {
                    x += bias_k[kb];
                } else if constexpr (kBias == 1) {
                    const int i = ih0 + acc_row(r, g);
                    if (i < a.sq && key[kb] < a.sk)
                        x += bias_log2(a.bias[b * a.bs[0] + h * a.bs[1] + (int64_t)i * a.bs[2] +
                                              (int64_t)key[kb] * a.bs[3]]);
                }
                float p = fast_exp2(x);
                if constexpr (kMask != 0) {
                    const int c = acc_row(r, 0);
                    if constexpr (kMask == 2) {
                        if (c < c_lo[kb] || c > c_hi[kb]) p = 0.f;
                    } else {
                        if (c < c_lo[kb]) p = 0.f;
                    }
                }
                s[kb][r] = p;
            }
        }
    };
    // Keep-bits of one key block of a half tile: wq[e] bit 4 * r4 belongs to register 4 * r4 + e.
    // (kDrop == 3 reads the stored words in half_ds instead.)
    auto keep_bits_half = [&](int kcol, int ih0, uint32_t (&wq)[4])
                              __attribute__((always_inline)) {
        if constexpr (kDrop == 1) {
            // The four lanes of a quad hold four consecutive keys, i.e. one Philox block per query
            // row.  Lane j of the quad draws the blocks of the rows held in registers j, j+4, j+8,
            // j+12 and the quad exchanges them: 4 blocks per lane instead of 16.
            const int qpos = lane & 3;
            uint32_t mine = 0;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const int i = ih0 + acc_row(4 * r4 + qpos, g);
                if (i < a.sq && kcol < a.sk) {
                    const uint64_t el =
                        ((uint64_t)bh * a.sq + (uint64_t)i) * (uint64_t)a.sk + (uint64_t)(kcol & ~3);
                    mine |= dropout_keep4_pow2(a.rng, el >> 2) << (4 * r4);
                }
            }
            wq[0] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0x00, 0xF, 0xF, false) >> qpos;
            wq[1] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0x55, 0xF, 0xF, false) >> qpos;
            wq[2] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0xAA, 0xF, 0xF, false) >> qpos;
            wq[3] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0xFF, 0xF, 0xF, false) >> qpos;
        } else if constexpr (kDrop == 2) {
            uint32_t mask16 = 0;  // bit r <-> register r
#pragma unroll 1
            for (int r = 0; r < 16; ++r) {
                const int i = ih0 + acc_row(r, g);
                if (i < a.sq && kcol < a.sk) {
                    const uint64_t el =
                        ((uint64_t)bh * a.sq + (uint64_t)i) * (uint64_t)a.sk + (uint64_t)kcol;
                    if (dropout_keep1(a.rng, el)) mask16 |= 1u << r;
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) wq[e] = mask16 >> e;
        }
    };
    // P (after dropout) and dS = P (dP - delta), packed to T
    auto half_ds = [&](const f32x16_t (&p)[KB], const f32x16_t (&dp)[KB], const float* delta_h,
                       const uint32_t* mask_h, int ih0, uint32_t (&pw)[KB][8],
                       uint32_t (&dw)[KB][8]) __attribute__((always_inline)) {
        uint32_t wq[KB][4];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
            for (int e = 0; e < 4; ++e) wq[kb][e] = 0u;
            keep_bits_half(key[kb], ih0, wq[kb]);
        }
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            f32x4_t del4 = {0.f, 0.f, 0.f, 0.f};  // no dropout: already subtracted
            u32x4_t w4 = {0u, 0u, 0u, 0u};
            if constexpr (kDrop != 0)
                del4 = *reinterpret_cast<const f32x4_t*>(delta_h + quad_slot(r4, g));
            // kDrop == 3: the stored words of four queries (bit j = key j of this wavefront)
            if constexpr (kDrop == 3)
                w4 = *reinterpret_cast<const u32x4_t*>(mask_h + quad_slot(r4, g));
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                float pv[4], dv[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float pe = p[kb][4 * r4 + e];
                    float d = dp[kb][4 * r4 + e];
                    float pd = pe;
                    if constexpr (kDrop != 0) {
                        // dropped pairs become +0; dV and dK take the factor 1 / (1 - p) when
                        // they are written (the staged delta carries 1 - p instead)
                        const uint32_t bits = kDrop == 3 ? w4[e] : wq[kb][e];
                        const uint32_t pos = kDrop == 3 ? (uint32_t)c_loc : 4u * r4;
                        pd = keep_or_zero(pe, bits, pos);
                        d = keep_or_zero(d, bits, pos);
                    }
                    pv[e] = pd;
                    dv[e] = pe * (d - del4[e]);
                }
                pw[kb][2 * r4] = pack2<T>(pv[0], pv[1]);
                pw[kb][2 * r4 + 1] = pack2<T>(pv[2], pv[3]);
                dw[kb][2 * r4] = pack2<T>(dv[0], dv[1]);
                dw[kb][2 * r4 + 1] = pack2<T>(dv[2], dv[3]);
            }
        }
    };
    // dV^T += dO_h^T P, dK^T += Q_h^T dS: every transposed fragment read feeds KB instructions
    auto half_out = [&](const T* qt, const T* gt, int hf, const uint32_t (&pw)[KB][8],
                        const uint32_t (&dw)[KB][8]) __attribute__((always_inline)) {
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            frag_t pf[KB], df[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                u32x4_t pq = {pw[kb][4 * hh], pw[kb][4 * hh + 1], pw[kb][4 * hh + 2],
                              pw[kb][4 * hh + 3]};
                u32x4_t dq4 = {dw[kb][4 * hh], dw[kb][4 * hh + 1], dw[kb][4 * hh + 2],
                               dw[kb][4 * hh + 3]};
                pf[kb] = __builtin_bit_cast(frag_t, pq);
                df[kb] = __builtin_bit_cast(frag_t, dq4);
            }
            const int off = (32 * hf + 16 * hh) * kPitch + t_off;
#pragma unroll
            for (int x = 0; x < DV; ++x) {
                const frag_t gta = lds_frag_tr<T>(gt + off + 32 * x, kPitch);
                const frag_t qta = lds_frag_tr<T>(qt + off + 32 * x, kPitch);
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) {
                    dv_acc[kb][x] = Mma<T>::mma32(gta, pf[kb], dv_acc[kb][x]);
                    dk_acc[kb][x] = Mma<T>::mma32(qta, df[kb], dk_acc[kb][x]);
                }
            }
        }
    };

    // The two halves of a fast tile one after the other.  At DPAD 96 this is what fits two
    // workgroups per CU (11-51 spilled registers); the second resident workgroup is worth more
    // than the stagger: 319 -> 287 us at bf16 B4 S2048 H32 D80 causal, 638 -> 503 us when the
    // backward regenerates the dropout mask.  With the forward's keep bits it is the other way
    // round (370 -> 455 us), so that variant keeps one workgroup and the staggered body.
    auto sequential_tile = [&](int t) __attribute__((always_inline)) {
        const int buf = (t - t_lo) & 1;
        const T* qt = q_lds + buf * SM::kQTile;
        const T* gt = g_lds + buf * SM::kQTile;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int ih0 = t * kBwdBM + 32 * hf;
            const float* lse_h = stat_lds + buf * 2 * kBwdBM + 32 * hf;
            const float* delta_h = lse_h + kBwdBM;
            const uint32_t* mask_h = mask_lds + buf * kBwdThreads + wave * kBwdBM + 32 * hf;
            f32x16_t s[KB], dp[KB];
            uint32_t pw[KB][8], dw[KB][8];
            half_sp(qt, gt, lse_h, delta_h, hf, s, dp);
            half_exp(s, lse_h, ih0, std::integral_constant<int, 0>{});
            half_ds(s, dp, delta_h, mask_h, ih0, pw, dw);
            half_out(qt, gt, hf, pw, dw);
        }
    };
    // Fast iteration t (every key of the workgroup sees every query of the tile): request tile
    // t+1, process tile t as one straight block, write tile t+1 into the other buffer.
    // The two halves of tile t with their stages staggered (mask_tag as in half_exp; only fast
    // tiles, tag 0, run this body: a second copy with the causal bound for the diagonal tiles
    // changed the register allocation of the first and measured 6 % slower overall).
    // kRequestInside: tile t+1 is requested in the middle, once the score registers of the first
    // half are dead, which keeps the staging registers out of the busiest stretch.  (No
    // scheduling fences around the request: with the body in one basic block they only kept the
    // exponentials of the second half away from the matrix instructions of the first half's
    // outputs; without them the kernel needs 214 registers instead of 254 and measures the same.)
    auto staggered_tile = [&](int t, auto mask_tag, auto request_inside)
                              __attribute__((always_inline)) {
        constexpr bool kRequestInside = decltype(request_inside)::value;
        const int buf = (t - t_lo) & 1;
        const T* qt = q_lds + buf * SM::kQTile;
        const T* gt = g_lds + buf * SM::kQTile;
        const float* lse_t = stat_lds + buf * 2 * kBwdBM;
        const float* delta_t = lse_t + kBwdBM;
        const uint32_t* mask_t = mask_lds + buf * kBwdThreads + wave * kBwdBM;
        const int i0 = t * kBwdBM;
        f32x16_t s0[KB], s1[KB], p0[KB], p1[KB];
        uint32_t pw0[KB][8], dw0[KB][8], pw1[KB][8], dw1[KB][8];
        half_sp(qt, gt, lse_t, delta_t, 0, s0, p0);
        half_exp(s0, lse_t, i0, mask_tag);
        half_sp(qt, gt, lse_t + 32, delta_t + 32, 1, s1, p1);
        half_ds(s0, p0, delta_t, mask_t, i0, pw0, dw0);
        half_exp(s1, lse_t + 32, i0 + 32, mask_tag);
        if constexpr (kRequestInside) {
            request_tile(regs, t + 1);
        }
        half_out(qt, gt, 0, pw0, dw0);
        half_ds(s1, p1, delta_t + 32, mask_t + 32, i0 + 32, pw1, dw1);
        half_out(qt, gt, 1, pw1, dw1);
    };
    // Fast iteration t (every key of the workgroup sees every query of the tile): request tile
    // t+1, process tile t as one straight block, write tile t+1 into the other buffer.
    auto fast_iteration = [&](int t) __attribute__((always_inline)) {
        constexpr bool kLateRequest = DPAD <= 64;  // two workgroups share a CU: registers scarce
        if constexpr (!kLateRequest) request_tile(regs, t + 1);
        if constexpr (DPAD == 96 && bwd_two_per_cu(DPAD, kDrop, KB))
            sequential_tile(t);
        else
            staggered_tile(t, std::integral_constant<int, 0>{},
                       std::integral_constant<bool, kLateRequest>{});
        // stage the next query tile (its buffer was last read before the previous barrier)
        if (t + 1 < t_hi) stage_tile(regs, t + 1);
        sync_staged();
    };

    // Diagonal / window / tail tiles: activity and masks are tested per wavefront and half tile.
    // The half tiles of `n` tiles (1 or 2) that sit in LDS are walked by one rolled loop.
    auto generic_tiles = [&](int t, int n) __attribute__((always_inline)) {
#pragma unroll 1
        for (int j = 0; j < 2 * n; ++j) {
            const int tt = t + (j >> 1), hf = j & 1;
            const int ih0 = tt * kBwdBM + 32 * hf;
            if (!half_active(ih0)) continue;
            const int buf = (tt - t_lo) & 1;
            const T* qt = q_lds + buf * SM::kQTile;
            const T* gt = g_lds + buf * SM::kQTile;
            const float* lse_h = stat_lds + buf * 2 * kBwdBM + 32 * hf;
            const float* delta_h = lse_h + kBwdBM;
            const uint32_t* mask_h = mask_lds + buf * kBwdThreads + wave * kBwdBM + 32 * hf;
            f32x16_t s[KB], dp[KB];
            uint32_t pw[KB][8], dw[KB][8];
            half_sp(qt, gt, lse_h, delta_h, hf, s, dp);
            if (!half_needs_mask(ih0))
                half_exp(s, lse_h, ih0, std::integral_constant<int, 0>{});
            else if (a.window > 0)
                half_exp(s, lse_h, ih0, std::integral_constant<int, 2>{});
            else
                half_exp(s, lse_h, ih0, std::integral_constant<int, 1>{});
            half_ds(s, dp, delta_h, mask_h, ih0, pw, dw);
            half_out(qt, gt, hf, pw, dw);
        }
    };
    // Generic step at tile t (in LDS, nothing requested); returns the number of tiles done.  Two
    // generic tiles in a row -- the two diagonal tiles of a causal mask -- are taken together:
    // the wavefronts have very different numbers of visible half tiles in each of them, and with
    // both tiles in LDS no wavefront waits at a barrier in between for the busiest one.
    auto generic_step = [&](int t) __attribute__((always_inline)) -> int {
        const bool pair = kPairGeneric && t + 1 < t_hi && !tile_fast(t + 1);
        if (!pair) {
            request_tile(regs, t + 1);
            generic_tiles(t, 1);
            if (t + 1 < t_hi) stage_tile(regs, t + 1);
            sync_staged();
            return 1;
        }
        if (!(pair_first && t == t_lo)) {  // otherwise the start-up has staged tile t+1 already
            request_tile(regs, t + 1);
            stage_tile(regs, t + 1);  // the other buffer: last read before the previous barrier
            sync_staged();
        }
        request_tile(regs, t + 2);
        generic_tiles(t, 2);
        __syncthreads();  // tile t+2 goes where tile t was
        if (t + 2 < t_hi) stage_tile(regs, t + 2);
        sync_staged();
        return 2;
    };
    {
        int t = t_lo;
        while (t < t_hi && !tile_fast(t)) t += generic_step(t);
        for (; t < t_hi && tile_fast(t); ++t) fast_iteration(t);
        while (t < t_hi) t += generic_step(t);
    }
    // ---- write dK, dV ----
    // every wavefront is past the last barrier of the loop: the tile buffers are free, and each
    // wavefront routes its rows through its own part of them (dK through the Q buffers, dV
    // through the dO buffers)
    static_assert(KB == 1, "the output staging assumes 32 keys per wavefront");
    if (kw0 < a.sk) {
        T* dk_row0 =
            reinterpret_cast<T*>(a.dk) + b * a.dks[0] + (int64_t)kw0 * a.dks[1] + h * a.dks[2];
        T* dv_row0 =
            reinterpret_cast<T*>(a.dv) + b * a.dvs[0] + (int64_t)kw0 * a.dvs[1] + h * a.dvs[2];
        store_block_via_lds<T, DPAD, kPitch>(dk_acc[0],
                                             kDrop != 0 ? a.scale * a.rng.inv_keep : a.scale,
                                             q_lds + wave * 32 * kPitch,
                                             dk_row0, a.dks[1], a.sk - kw0, a.d);
        // with dropout: the factor 1 / (1 - p) that half_ds left out of P
        store_block_via_lds<T, DPAD, kPitch>(dv_acc[0], kDrop != 0 ? a.rng.inv_keep : 1.0f,
                                             g_lds + wave * 32 * kPitch, dv_row0, a.dvs[1],
                                             a.sk - kw0, a.d);
    }
}

template <typename T, int DPAD, int kBias, int kDrop, int KB, int kSteps>
int launch(const AttnArgs& a, hipStream_t st) {
    typedef BwdSmem<T, DPAD> SM;
    const size_t smem = SM::kBytes;
    constexpr int kBN = kBwdWaves * 32 * KB;
    const int n_kt = (a.sk + kBN - 1) / kBN;
    const int64_t blocks = (int64_t)n_kt * a.batch * a.heads;
    if (blocks <= 0 || blocks > 0x7FFFFFFF) return SLAPO_ERR_SHAPE;
    auto kern = attn_bwd_kernel<T, DPAD, kBias, kDrop, KB, kSteps>;
    static std::atomic<uint64_t> lds_ready{0};  // per instantiation, one bit per device
    if (allow_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_ready) != SLAPO_OK)
        return SLAPO_ERR_LAUNCH;
    AttnArgs ordered = a;
    set_dispatch_order(&ordered, blocks, bwd_two_per_cu(DPAD, kDrop, KB) ? 2 : 1);
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kBwdThreads), smem, st, ordered);
    return check_launch();
}

// Two key blocks per wavefront (KB = 2, one wavefront per SIMD) measured slower than KB = 1 with two
// wavefronts per SIMD on MI355X (92 us against 70 us at fp16 B8 S1024 H16 D64 causal): the second
// resident wavefront hides more latency than the halved LDS traffic saves.  Only KB = 1 is built.
template <typename T, int DPAD, int kBias, int kDrop, int kSteps>
int launch_kb(const AttnArgs& a, hipStream_t st) {
    return launch<T, DPAD, kBias, kDrop, 1, kSteps>(a, st);
}

template <typename T, int DPAD, int kBias, int kSteps>
int dispatch_drop(const AttnArgs& a, hipStream_t st) {
    if (a.dropout == 1) return launch_kb<T, DPAD, kBias, 1, kSteps>(a, st);
    if (a.dropout == 2) return launch_kb<T, DPAD, kBias, 2, kSteps>(a, st);
    if (a.dropout == 3) return launch_kb<T, DPAD, kBias, 3, kSteps>(a, st);
    return launch_kb<T, DPAD, kBias, 0, kSteps>(a, st);
}

template <typename T, int DPAD, int kSteps = DPAD / 16>
int dispatch_flags(const AttnArgs& a, hipStream_t st) {
    if (!a.has_bias) return dispatch_drop<T, DPAD, 0, kSteps>(a, st);
    return a.bs[2] == 0 ? dispatch_drop<T, DPAD, 2, kSteps>(a, st)
                        : dispatch_drop<T, DPAD, 1, kSteps>(a, st);
}

template <typename T>
int dispatch(const AttnArgs& a, hipStream_t st) {
    if (a.d <= 64) return dispatch_flags<T, 64>(a, st);
    if (a.d <= 80) return dispatch_flags<T, 96, 5>(a, st);  // five k-steps cover head_dim 80
    if (a.d <= 96) return dispatch_flags<T, 96>(a, st);
    if (a.d <= 128) return dispatch_flags<T, 128>(a, st);
    return SLAPO_ERR_SHAPE;
}

}  // namespace bwd
}  // namespace slapo
