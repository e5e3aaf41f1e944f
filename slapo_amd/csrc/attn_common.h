// Pieces shared by the attention kernels: MFMA wrappers for fp16/bf16 on gfx950, the LDS
// transpose read, tile staging (global -> registers -> LDS), masks and the kernel argument block.
//
// MFMA v_mfma_f32_32x32x16_{f16,bf16} (one wavefront, lane l, g = l / 32):
//   A operand: lane holds row (l % 32), 8 consecutive k-slots of lane-group g;
//   B operand: lane holds column (l % 32), the same 8 k-slots;
//   C/D:       register r of lane l is element (row 8*(r/4) + 4*g + r%4, column l % 32).
// The k-slot <-> data mapping is free as long as A and B agree, and the row <-> data mapping of
// the A operand is free as well; both freedoms are used below to keep every fragment a plain
// 128-bit LDS read or two transposing 64-bit reads.
#pragma once
#include "common.h"

namespace slapo {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

template <typename T>
struct Mma;

template <>
struct Mma<f16_t> {
    typedef f16x8_t frag;
    typedef f16x4_t half_frag;
    static __device__ __forceinline__ f32x16_t mma32(frag a, frag b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4_t mma16(frag a, frag b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Mma<bf16_t> {
    typedef bf16x8_t frag;
    typedef bf16x4_t half_frag;
    static __device__ __forceinline__ f32x16_t mma32(frag a, frag b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4_t mma16(frag a, frag b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};

typedef short i16x4_t __attribute__((ext_vector_type(4)));

// LDS transpose read (ds_read_b64_tr_b16).  Within each block of 16 lanes, lane n receives
// element e = 0..3 from source lane (4*e + n/4), 16-bit word (n % 4) of that lane's 8 bytes.
// With source lane i pointing at row (i/4), columns 4*(i%4).. of a row-major tile, lane n gets
// the four rows of column n: a 4x16 -> 16x4 transpose.
__device__ __forceinline__ u32x2_t lds_read_tr16(const void* lds_ptr) {
    i16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (i16x4_t __attribute__((address_space(3)))*)(uintptr_t)(
            (uint32_t)(uintptr_t)lds_ptr));
    return __builtin_bit_cast(u32x2_t, v);
}

// Fragment made of two transposing reads: slots 0..3 from rows r0, r0+4, r0+8, r0+12 and slots 4..7
// from the rows one below them (the lane offset of tr_lane_off supplies the row stride of 4; see
// pi_row for why the four rows of one read are four rows apart).
template <typename T>
__device__ __forceinline__ typename Mma<T>::frag lds_frag_tr(const T* tile, int pitch) {
    const u32x2_t lo = lds_read_tr16(tile);
    const u32x2_t hi = lds_read_tr16(tile + pitch);
    u32x4_t v = {lo.x, lo.y, hi.x, hi.y};
    return __builtin_bit_cast(typename Mma<T>::frag, v);
}
// Per-lane element offset of such a fragment inside a block of 16 tile rows whose columns
// 32 x .. 32 x + 31 form the 32 rows of the A operand: lane-group g starts at row 2 g, the four
// source lanes of a column quad are four rows apart, 16-lane block b takes columns 16 b ..
__device__ __forceinline__ int tr_lane_off(int lane, int pitch) {
    return (2 * (lane >> 5) + 4 * ((lane & 15) >> 2)) * pitch + ((lane >> 4) & 1) * 16 +
           4 * (lane & 3);
}

template <typename T>
__device__ __forceinline__ typename Mma<T>::frag lds_frag(const T* p) {
    return *reinterpret_cast<const typename Mma<T>::frag*>(p);
}

// Row permutation applied when a 32-row A operand is gathered: MFMA row rho takes data row
// pi(rho).  Accumulator register r of lane-group g is MFMA row 8 (r / 4) + 4 g + r % 4; with
// rho = [h][u][g][e1 e0] (bits 4..0) the data row is [h][e1 e0][g][u].  Two properties follow:
//  * registers 8 h .. 8 h + 7 of lane-group g are, in order, the eight k-slots of a B operand of
//    the next MFMA whose A operand comes from transposing LDS reads of the same tile;
//  * the four k-slots of one transposing read (e = 0..3) are data rows FOUR apart.  With a row
//    pitch of DPAD + 8 elements four rows are 64 bytes (mod 256) apart, so the 4 rows x 64 bytes
//    that 32 lanes read in one LDS cycle fall into 64 different banks.  With consecutive rows
//    the same reads collide two-fold at head_dim 64 / 96 and four-fold at 128 (measured: 437 and
//    851 ns against 247 ns per 128 KB and CU).
__device__ __forceinline__ int pi_row(int rho) {
    return (rho & 16) | ((rho & 3) << 2) | (((rho >> 2) & 1) << 1) | ((rho >> 3) & 1);
}
// Data row (0..31) held by accumulator register r of lane-group g under that permutation.
__device__ __forceinline__ constexpr int acc_row(int r, int g) {
    return ((r >> 3) << 4) + ((r & 3) << 2) + (g << 1) + ((r >> 2) & 1);
}
constexpr int kAccGroupStep = 2;  // acc_row(r, g) = acc_row(r, 0) + kAccGroupStep * g
// Per-row values (bias, lse, delta, keep words) of a 32-row block are kept in LDS at position
// row_slot(row), so that ONE 128-bit read at quad_slot(r4, g) returns the values of registers
// 4 r4 .. 4 r4 + 3 of lane-group g in order.
__device__ __forceinline__ constexpr int row_slot(int row) {
    return (row & ~15) | ((row & 3) << 2) | ((row >> 2) & 3);
}
__device__ __forceinline__ constexpr int quad_slot(int r4, int g) {
    return ((r4 >> 1) << 4) + (g << 3) + ((r4 & 1) << 2);
}

// Two floats -> one packed register of T, round to nearest even (v_cvt_pk_{f16,bf16}_f32).
template <typename T>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    typedef T pair_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    f32x2_t v = {a, b};
    pair_t p = __builtin_convertvector(v, pair_t);
    return __builtin_bit_cast(uint32_t, p);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// acc + lo + hi of a packed pair of T, in fp32 (v_dot2c_f32_{f16,bf16} against a pair of ones).
template <typename T>
__device__ __forceinline__ float sum2(uint32_t pair, float acc);
template <>
__device__ __forceinline__ float sum2<f16_t>(uint32_t pair, float acc) {
    const f16x2_t ones = {(f16_t)1.f, (f16_t)1.f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, pair), ones, acc, false);
}
template <>
__device__ __forceinline__ float sum2<bf16_t>(uint32_t pair, float acc) {
    const bf16x2_t ones = {(bf16_t)1.f, (bf16_t)1.f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pair), ones, acc, false);
}

// Masking values.  A bias at or below kMaskBias (-5e8: "-1e9", also after rounding to bf16,
// "-1e30", finfo.min of bf16 / fp32 are what models add to hide a key) is taken as THE masking
// value and becomes -FLT_MAX exactly;
// a true -inf is left alone.  Added to a score in fp32 such a bias swallows the score in the
// reference too, so a query row that sees nothing but masked keys gets a uniform softmax over them
// there and here.  For such a row the kernels keep m = -FLT_MAX as the softmax reference point
// (masked scores minus it are exactly 0) and the row sum n = number of those keys; the usual
// log-sum-exp m + log n cannot hold n beside m, so the forward stores n * 2^100 in its place
// (no real log-sum-exp comes near 6e29) and the backward decodes it: probabilities are
// exp(x - m) / n.
constexpr float kMaskBias = -5e8f;
constexpr float kFltMax = 3.4028234663852886e38f;
constexpr float kMaskedRowLse = 1.2676506002282294e30f;  // 2^100
__device__ __forceinline__ float canonical_bias(float b) {
    return (b <= kMaskBias && b != -INFINITY) ? -kFltMax : b;
}
// An additive bias in log2 units.
__device__ __forceinline__ float bias_log2(float b) {
    return (b <= kMaskBias && b != -INFINITY) ? -kFltMax : b * kLog2e;
}
// What the forward stores as log-sum-exp of a row with reference point m (any units) and row sum l.
__device__ __forceinline__ bool masked_row_lse(float lse) {
    return lse >= 0.5f * kMaskedRowLse && lse < INFINITY;
}
// The reference point that exp subtracts for a stored log-sum-exp, times `unit` (1 for natural
// units, log2(e) for log2 units), and the factor 1 / n that goes with it (1 for ordinary rows).
__device__ __forceinline__ float lse_reference(float lse, float unit) {
    return masked_row_lse(lse) ? -kFltMax : lse * unit;
}
__device__ __forceinline__ float lse_row_factor(float lse) {
    return masked_row_lse(lse) ? kMaskedRowLse / lse : 1.0f;
}

// Fragment of 8 elements times a scalar, rounded back to T.
template <typename T>
__device__ __forceinline__ typename Mma<T>::frag scale_frag(u32x4_t raw, float c) {
    typename Mma<T>::frag f = __builtin_bit_cast(typename Mma<T>::frag, raw);
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = (T)((float)f[j] * c);
    return f;
}

// Exchange with lane l ^ 32 through v_permlane32_swap (upper half of the first register <-> lower
// half of the second).  Starting from two copies of v, the first register ends up holding the lower
// half's values on all lanes and the second the upper half's.  Written as inline assembly, with the
// wait states the instruction needs after a VALU write of its operands.
__device__ __forceinline__ void swap32(float v, float& lo_val, float& hi_val) {
    float a = v, b = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    lo_val = a;
    hi_val = b;
}
// OR of a value with that of lane l ^ 32
__device__ __forceinline__ uint32_t or_xor32(uint32_t v) {
    float a, b;
    swap32(__builtin_bit_cast(float, v), a, b);
    return __builtin_bit_cast(uint32_t, a) | __builtin_bit_cast(uint32_t, b);
}
__device__ __forceinline__ float max_xor32(float v) {
    float a, b;
    swap32(v, a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float sum_xor32(float v) {
    float a, b;
    swap32(v, a, b);
    return a + b;
}

// 16 bytes of a row fragment, or zeros when `keep` is false.  Written as a mask so that it stays
// straight-line code: a branch here would make the compiler wait for the load on the spot, and
// the start-up loads of a workgroup must all be in flight together.
__device__ __forceinline__ u32x4_t keep_or_zero(u32x4_t v, bool keep) {
    const uint32_t m = keep ? 0xFFFFFFFFu : 0u;
    return u32x4_t{v.x & m, v.y & m, v.z & m, v.w & m};
}

// v where bit `pos` of `bits` is set, +0 elsewhere: the bit, sign-extended to a whole word
// (v_bfe_i32), masks the float.  Two instructions per value where a test, a compare and a select
// take three.
__device__ __forceinline__ float keep_or_zero(float v, uint32_t bits, uint32_t pos) {
    const uint32_t m = (uint32_t)__builtin_amdgcn_sbfe((int)bits, pos, 1u);
    return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v) & m);
}

// Kernel argument block (filled by the host dispatcher from slapo_attn_params).
struct AttnArgs {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    const void* dout;
    void* dq;  // element type of the tensors
    void* dk;
    void* dv;
    const float* bias;
    float* lse;
    float* delta;
    int64_t qs[3], ks[3], vs[3], os[3], dqs[3], dks[3], dvs[3];
    int64_t bs[4];
    int batch, heads, sq, sk, d;
    int causal, window;
    int has_bias, bias_vec4;  // bias_vec4: s3 == 1, s2 == 0 rows 16B-aligned
    // dropout: 0 = off, 1 = fast mask geometry (plan.vec >= 4, power-of-two thread count and
    // sk % 4 == 0: one Philox block per aligned group of four keys), 2 = any geometry,
    // 3 = keep bits read from keep_mask (drawn by keep_mask_kernel ahead of the forward)
    int dropout;
    // Keep bits of the dropout mask, when not null: uint32 words
    // [batch*heads][mask_words][mask_pitch], bit j of word (bh, w, i) = keep(query i, key 32 w + j)
    uint32_t* keep_mask;
    int mask_words, mask_pitch;
    float scale, scale_log2;
    DropoutState rng;
    // Dispatch order, see work_index: the first `snake_rows` rows of `snake_len` workgroups each
    // are walked in alternating directions.  n_cus is host-side only (0: unknown).
    int snake_len, snake_rows;
    // head_group > 0: an XCD works through its heads `head_group` at a time (all tiles of one
    // group before the next group), so that the K / V of the heads in flight fit its L2
    int head_group;
    int n_cus;
};

// Which unit of work a workgroup takes.  The kernels order their work heaviest first (under a
// causal mask a workgroup's loop has 2 to 2 S / 128 tiles), and the hardware hands the
// first workgroups out one per CU, row after row of n_cus workgroups, until every CU holds as
// many as fit; the rest follow as workgroups finish.  With every row in descending order the CU
// that got the heaviest workgroup of row 0 also gets the heaviest of rows 1, 2: at fp16 B8
// S1024 H16 D64 half of the CUs then hold 16 + 12 tiles of the dK/dV kernel and the other half
// 14 + 10, the latter get the next-heaviest workgroups as well, and the launch ends with CUs at
// 34 to 40 tiles (43 to 53 us).  Walking the odd rows backwards (in groups of eight, so that a
// workgroup stays on the XCD it would have had: workgroup i runs on XCD i % 8, and the heads are
// spread over the XCDs the same way) evens the sums out.
__device__ __forceinline__ int work_index(const AttnArgs& a) {
    int idx = (int)blockIdx.x;
    if (a.snake_rows > 0) {
        const int row = idx / a.snake_len;
        if (row < a.snake_rows && (row & 1)) {
            const int pos = idx - row * a.snake_len;
            idx = row * a.snake_len + (a.snake_len / 8 - 1 - pos / 8) * 8 + (pos & 7);
        }
    }
    if (a.head_group > 0) {
        // Workgroup i runs on XCD i % 8.  Position j = i / 8 in that XCD's sequence takes, group
        // after group of `head_group` heads (head = XCD + 8 * its index on the XCD), the tiles of
        // the group heaviest first; the host checked batch * heads % 8 == 0.
        const int n_bh = a.batch * a.heads;
        const int xcd = idx & 7, j = idx >> 3;
        const int per_xcd = n_bh >> 3;
        const int n_levels = (int)gridDim.x / n_bh;
        const int full = per_xcd / a.head_group;             // groups of full size
        const int span = a.head_group * n_levels;            // workgroups per full group
        int group = j / span, r = j - group * span, size = a.head_group;
        if (group >= full) {                                 // the last, smaller group
            group = full, r = j - full * span, size = per_xcd - full * a.head_group;
        }
        const int level = r / size, head = group * a.head_group + (r - level * size);
        idx = level * n_bh + xcd + 8 * head;
    }
    return idx;
}
// Host: `per_cu` workgroups of the kernel fit a CU at a time; rows that the grid does not fill
// are left alone.
inline void set_dispatch_order(AttnArgs* a, int64_t blocks, int per_cu, bool group_heads = false) {
    a->snake_len = a->n_cus & ~7;
    a->snake_rows = 0;
    a->head_group = 0;
    if (group_heads && a->n_cus >= 8) {
        // K and V of one head against the L2 of an XCD (4 MB; three quarters of it budgeted).
        // Heads are grouped only where a group fills the XCD's resident workgroups by itself (else
        // several groups are in flight anyway) and the launch is at least four such fillings deep
        // (a group's heavy workgroups start late; in a shallow launch they become its tail).
        // Measured at bf16 B4 S2048 H32 D80 (groups of 4 of the 16 heads of an XCD), clocks
        // settled: forward 132 -> 127 us with a padding mask, 146 -> 141 us without, 252 -> 236 us
        // without the causal mask; dQ unchanged (163 us), dK/dV 222 -> 234 us: only the forward
        // asks for it.  Without the two conditions: fp16 B8 S1024 H16 D64 forward 34 -> 42 us, bf16
        // B4 S2048 H16 D128 forward 90 -> 100 us, S4096 306 -> 340 us.
        const int64_t n_bh = (int64_t)a->batch * a->heads;
        const int64_t head_bytes = 2 * (int64_t)a->sk * a->d * 2;
        const int64_t fit = (3 << 20) / (head_bytes > 0 ? head_bytes : 1);
        const int64_t levels = n_bh > 0 ? blocks / n_bh : 0;
        const int64_t xcd_slots = (int64_t)(a->n_cus / 8) * per_cu;
        if (n_bh % 8 == 0 && blocks % n_bh == 0 && fit >= 1 && fit < n_bh / 8 &&
            fit * levels >= xcd_slots && blocks >= 4 * 8 * xcd_slots) {
            a->head_group = (int)fit;
            return;  // the order inside a group is heaviest first
        }
    }
    if (a->snake_len < 8 || !a->causal) return;
    const int64_t full_rows = blocks / a->snake_len;
    a->snake_rows = (int)(full_rows < per_cu ? full_rows : per_cu);
}

__device__ __forceinline__ bool key_visible(const AttnArgs& a, int i, int j) {
    return j < a.sk && (!a.causal || j <= i) && (a.window <= 0 || i - j < a.window);
}

// First / one-past-last key that any query in [q_lo, q_hi) may see.
__device__ __forceinline__ void key_range(const AttnArgs& a, int q_lo, int q_hi, int& j_lo,
                                          int& j_hi) {
    j_hi = a.causal ? min(a.sk, q_hi) : a.sk;
    j_lo = a.window > 0 ? max(0, q_lo - a.window + 1) : 0;
}
// First / one-past-last query that can see any key in [k_lo, k_hi).
__device__ __forceinline__ void query_range(const AttnArgs& a, int k_lo, int k_hi, int& i_lo,
                                            int& i_hi) {
    i_lo = a.causal ? min(k_lo, a.sq) : 0;
    i_hi = a.window > 0 ? min(a.sq, k_hi - 1 + a.window) : a.sq;
}

// Key-padding masks arrive as an additive bias that does not depend on the query
// ([B,1,1,Sk] with a large negative value on padded keys).  Keys past the last unmasked one
// contribute exp(-huge) = 0 exactly to every row that sees at least one unmasked key, so whole
// tiles of them can be skipped.  Returns one past the last key worth visiting (a.sk when the
// shortcut does not apply): only per-key biases, no local window, and key 0 unmasked, which
// guarantees an unmasked visible key for every query row under a causal or full mask.
// Called by all threads of the workgroup; `scratch` is 4 floats of LDS that nothing else uses
// until the call returns.
constexpr float kMaskedBias = -30000.f;  // below fp16's most negative value, far beyond any score
template <int THREADS>
__device__ __forceinline__ int padded_key_limit(const AttnArgs& a, int b, int h, float* scratch) {
    if (!a.has_bias || a.bs[2] != 0 || a.window > 0) return a.sk;
    const float* brow = a.bias + b * a.bs[0] + h * a.bs[1];
    if (!(brow[0] > kMaskedBias)) return a.sk;
    int last = 0;
    for (int j = threadIdx.x; j < a.sk; j += THREADS)
        if (brow[(int64_t)j * a.bs[3]] > kMaskedBias) last = j;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) last = max(last, __shfl_xor(last, off, 64));
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = __int_as_float(last);
    __syncthreads();
    int limit = 0;
#pragma unroll
    for (int w = 0; w < THREADS / 64; ++w) limit = max(limit, __float_as_int(scratch[w]));
    __syncthreads();
    return limit + 1;
}

// Writes a wavefront's 32 x d block of results to global memory with full-line stores.  The
// block arrives transposed in accumulator registers (acc[x][4 r4 + e] of lane (i, g) is element
// (row i, column 32 x + 8 r4 + 4 g + e)), goes through `wave_lds` (32 rows of PITCH elements that
// only this wavefront touches) and leaves as 16 bytes per lane, eight or more lanes per row.
// Storing straight from the registers would write 8 bytes per lane to 32 different rows per
// instruction: sixteen-byte pieces of 128-byte lines.
template <typename T, int DPAD, int PITCH>
__device__ __forceinline__ void store_block_via_lds(const f32x16_t (&acc)[DPAD / 32], float mul,
                                                    T* wave_lds, T* out_row0, int64_t row_stride,
                                                    int n_rows, int d) {
    const int lane = threadIdx.x & 63;
    const int i = lane & 31, g = lane >> 5;
#pragma unroll
    for (int x = 0; x < DPAD / 32; ++x)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            u32x2_t w;
            w.x = pack2<T>(acc[x][4 * r4 + 0] * mul, acc[x][4 * r4 + 1] * mul);
            w.y = pack2<T>(acc[x][4 * r4 + 2] * mul, acc[x][4 * r4 + 3] * mul);
            *reinterpret_cast<u32x2_t*>(wave_lds + i * PITCH + 32 * x + 8 * r4 + 4 * g) = w;
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    constexpr int kChunksPerRow = DPAD / 8;
#pragma unroll
    for (int pass = 0; pass < 32 * kChunksPerRow / 64; ++pass) {
        const int idx = pass * 64 + lane;
        const int row = idx / kChunksPerRow, c = idx % kChunksPerRow;
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(wave_lds + row * PITCH + 8 * c);
        if (row < n_rows && 8 * c < d)
            *reinterpret_cast<u32x4_t*>(out_row0 + (int64_t)row * row_stride + 8 * c) = v;
    }
}

// Stage a [ROWS x DPAD] tile of T (rows row0.., zero beyond n_rows / beyond d) through registers.
// The global loads are unconditional (out-of-range rows are clamped to the last valid row and
// zeroed when the tile is written to LDS), so they stay in the caller's basic block and the
// compiler can leave them in flight across the math that follows.
template <typename T, int DPAD, int ROWS, int THREADS>
struct TileStage {
    static constexpr int kChunksPerRow = DPAD / 8;
    static constexpr int kChunks = ROWS * kChunksPerRow;
    static constexpr int kPerThread = (kChunks + THREADS - 1) / THREADS;
    static constexpr int kPitch = DPAD + 8;
    u32x4_t r[kPerThread];

    // Where THREADS is a multiple of the chunks per row, a lane's chunks sit in one column, kRowStep
    // rows apart, and one offset pair serves them all; otherwise each chunk keeps its own.
    static constexpr bool kOneColumn = THREADS % kChunksPerRow == 0;
    static constexpr int kRowStep = THREADS / kChunksPerRow;
    static constexpr int kOffsets = kOneColumn ? 1 : kPerThread;
    // Byte offsets inside a tile, set once by `init`: own[u] = chunk u at its own row, col[u] =
    // its column part alone.
    uint32_t own[kOffsets], col[kOffsets];

    // Needs 0 <= row_stride < 2^24 elements (host-checked): offsets inside a tile fit 32 bits.
    __device__ __forceinline__ void init(int64_t row_stride, int d) {
        const uint32_t stride_b = (uint32_t)row_stride * (uint32_t)sizeof(T);
#pragma unroll
        for (int u = 0; u < kOffsets; ++u) {
            const int c = threadIdx.x + u * THREADS;
            col[u] = (uint32_t)min((c % kChunksPerRow) * 8, d - 8) * (uint32_t)sizeof(T);
            own[u] = (uint32_t)(c / kChunksPerRow) * stride_b + col[u];
            // opaque to the optimiser, which would otherwise turn the select in `load` back into
            // a multiplication per tile
            asm volatile("" : "+v"(own[u]));
        }
    }
    // Requests the tile that starts at row0.  Rows past the end are clamped to the last row (row0
    // itself may lie past the end: the request is then wasted but safe).  The address is a
    // wavefront-uniform tile base plus an unsigned 32-bit byte offset per lane, which the
    // hardware adds for free (scalar base + vector offset addressing); the offset of a clamped
    // row is selected, not multiplied out.
    __device__ __forceinline__ void load(const T* base, int64_t row_stride, int row0, int n_rows,
                                         int d) {
        (void)d;
        const int row0c = min(row0, n_rows - 1);
        const char* tile = reinterpret_cast<const char*>(base + (int64_t)row0c * row_stride);
        const int last = n_rows - 1 - row0c;  // tile row that the clamped rows read, >= 0
        const uint32_t stride_b = (uint32_t)row_stride * (uint32_t)sizeof(T);
        const uint32_t last_b = (uint32_t)last * stride_b;
#pragma unroll
        for (int u = 0; u < kPerThread; ++u) {
            const int c = threadIdx.x + u * THREADS;
            const int row = c / kChunksPerRow;
            uint32_t off;
            if constexpr (kOneColumn)
                off = row <= last ? own[0] + (uint32_t)(u * kRowStep) * stride_b : last_b + col[0];
            else
                off = row <= last ? own[u] : last_b + col[u];
            if (kChunks % THREADS == 0 || c < kChunks)
                r[u] = *reinterpret_cast<const u32x4_t*>(tile + off);
        }
    }
    // The same request with every address multiplied out per lane: more vector instructions, no
    // `init`, fewer scalar ones.  The forward kernel measures 5 % faster with this form at
    // head_dim 64 (causal), the backward kernels 2-8 % faster with `load`.
    __device__ __forceinline__ void load_indexed(const T* base, int64_t row_stride, int row0,
                                                 int n_rows, int d) {
#pragma unroll
        for (int u = 0; u < kPerThread; ++u) {
            const int c = threadIdx.x + u * THREADS;
            const int row = c / kChunksPerRow;
            const int cc = c % kChunksPerRow;
            const int gr = min(row0 + row, n_rows - 1);
            if (kChunks % THREADS == 0 || c < kChunks)
                r[u] = *reinterpret_cast<const u32x4_t*>(base + (int64_t)gr * row_stride +
                                                         min(cc * 8, d - 8));
        }
    }
    // Zero what `load` clamped: rows past n_rows and columns past d.
    __device__ __forceinline__ void fix(int row0, int n_rows, int d) {
        if (row0 + ROWS <= n_rows && d == DPAD) return;  // uniform: whole tile valid
#pragma unroll
        for (int u = 0; u < kPerThread; ++u) {
            const int c = threadIdx.x + u * THREADS;
            const int row = c / kChunksPerRow;
            const int cc = c % kChunksPerRow;
            if (row0 + row >= n_rows || cc * 8 >= d) r[u] = u32x4_t{0u, 0u, 0u, 0u};
        }
    }
    // Chunk u times f[u] (one factor per row that the thread holds a chunk of), rounded back to T.
    __device__ __forceinline__ void scale_rows(const float (&f)[kPerThread]) {
#pragma unroll
        for (int u = 0; u < kPerThread; ++u)
            r[u] = __builtin_bit_cast(u32x4_t, scale_frag<T>(r[u], f[u]));
    }
    // Tile row of chunk u of this thread.
    static __device__ __forceinline__ int row_of(int u) {
        return (threadIdx.x + u * THREADS) / kChunksPerRow;
    }
    __device__ __forceinline__ void store(T* lds) const {
#pragma unroll
        for (int u = 0; u < kPerThread; ++u) {
            const int c = threadIdx.x + u * THREADS;
            if (kChunks % THREADS != 0 && c >= kChunks) continue;
            const int row = c / kChunksPerRow;
            const int cc = c % kChunksPerRow;
            *reinterpret_cast<u32x4_t*>(lds + row * kPitch + cc * 8) = r[u];
        }
    }
};

}  // namespace slapo
