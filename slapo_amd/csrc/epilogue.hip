// FusedMLP epilogues for gfx950: bias+GeLU(tanh) and bias+dropout(+residual), forward and
// backward.  All four are single-pass, HBM-bound streaming kernels: every tensor element is
// read or written exactly once through 128-bit accesses; the dropout mask is never stored
// (it is regenerated from the Philox state), and the bias gradient is a deterministic two-stage
// column reduction (per-block fp32 partials, then a tiny finishing kernel) -- no atomics.
//
// Formulas follow slapo/op/fused_bias.py:18-34 (bias_gelu / bias_gelu_back) and :67-74
// (bias_dropout); math is fp32 inside, storage in the tensor dtype.
#include "common.h"

using namespace slapo;

namespace {

// gelu_tanh(x) = 0.5 x (1 + tanh(a)) with a = 0.79788456 x (1 + 0.044715 x^2)
//             = x * sigma(2a),   sigma(z) = 1 / (1 + exp(-z)).
// exp(-2a) = exp2(x * (K1 + K2 x^2)),  K1 = -2 log2(e) 0.79788456,  K2 = K1 * 0.044715.
constexpr float kGeluK1 = -2.0f * 1.4426950408889634f * 0.79788456f;
constexpr float kGeluK2 = kGeluK1 * 0.044715f;

__device__ __forceinline__ float sigma2a(float x) {
    const float t = x * x;
    const float e = __builtin_amdgcn_exp2f(x * __builtin_fmaf(t, kGeluK2, kGeluK1));
    return __builtin_amdgcn_rcpf(1.0f + e);
}

__device__ __forceinline__ float gelu_fwd(float x) { return x * sigma2a(x); }

// d/dx: with t = tanh(a) = 2 s - 1:  0.5 (1 + t) = s,  1 - t^2 = 4 s (1 - s), so
// ff = 0.5 x (1 - t^2)(0.79788456 + 0.1070322243 x^2) + 0.5 (1 + t)
//    = s + 2 x s (1 - s)(0.79788456 + 0.1070322243 x^2).
__device__ __forceinline__ float gelu_grad(float x) {
    const float s = sigma2a(x);
    const float poly = __builtin_fmaf(x * x, 0.1070322243f, 0.79788456f);
    return __builtin_fmaf(2.0f * x * s * (1.0f - s), poly, s);
}

// V consecutive elements of T: V == Elem<T>::kPerVec uses one 128-bit access, V == 1 scalar.
template <typename T, int V>
struct Chunk {
    T v[V];
};

template <typename T, int V>
__device__ __forceinline__ Chunk<T, V> load_chunk(const T* p) {
    Chunk<T, V> c;
    if constexpr (V == 1) {
        c.v[0] = *p;
    } else {
        static_assert(sizeof(Chunk<T, V>) == 16, "vector chunk must be 16 bytes");
        *reinterpret_cast<u32x4_t*>(&c) =
            __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    }
    return c;
}
template <typename T, int V>
__device__ __forceinline__ Chunk<T, V> load_chunk_cached(const T* p) {
    Chunk<T, V> c;
    if constexpr (V == 1) {
        c.v[0] = *p;
    } else {
        *reinterpret_cast<u32x4_t*>(&c) = *reinterpret_cast<const u32x4_t*>(p);
    }
    return c;
}
template <typename T, int V>
__device__ __forceinline__ void store_chunk(T* p, const Chunk<T, V>& c) {
    if constexpr (V == 1) {
        *p = c.v[0];
    } else {
        __builtin_nontemporal_store(*reinterpret_cast<const u32x4_t*>(&c),
                                    reinterpret_cast<u32x4_t*>(p));
    }
}

// Keep-bits for V consecutive elements starting at element index e0 (e0 % V == 0).
// kDrop: 1 = shift-only mask geometry (vec >= 4, power-of-two thread count), 2 = any geometry.
template <int V, int kDrop>
__device__ __forceinline__ uint32_t keep_bits(const DropoutState& s, uint64_t e0) {
    uint32_t bits = 0;
    if constexpr (kDrop == 1) {
        static_assert(V % 4 == 0, "the fast geometry needs whole Philox blocks per chunk");
#pragma unroll
        for (int g = 0; g < V / 4; ++g) bits |= dropout_keep4_pow2(s, e0 / 4 + g) << (4 * g);
        return bits;
    }
    if constexpr (V % 4 == 0) {
        if (s.vec >= 4) {
#pragma unroll
            for (int g = 0; g < V / 4; ++g) bits |= dropout_keep4(s, e0 / 4 + g) << (4 * g);
            return bits;
        }
    }
#pragma unroll
    for (int i = 0; i < V; ++i) bits |= (dropout_keep1(s, e0 + i) ? 1u : 0u) << i;
    return bits;
}

// ----------------------------------------------------------------------------------------
// Forward kernels: flat over chunks; a block covers kUnroll * 256 consecutive chunks.
// ----------------------------------------------------------------------------------------
constexpr int kUnroll = 1;  // chunks per thread (more did not help on MI355X)

template <typename T, int V>
__global__ __launch_bounds__(256) void bias_gelu_fwd_kernel(const T* __restrict__ y,
                                                            const T* __restrict__ bias,
                                                            T* __restrict__ out,
                                                            uint64_t n_chunks,
                                                            uint32_t chunks_per_row,
                                                            uint32_t row_mask) {
    const uint64_t base = (uint64_t)blockIdx.x * (256 * kUnroll) + threadIdx.x;
    Chunk<T, V> in[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const uint64_t c = base + (uint64_t)u * 256;
        if (c < n_chunks) in[u] = load_chunk<T, V>(y + c * V);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const uint64_t c = base + (uint64_t)u * 256;
        if (c >= n_chunks) continue;
        const uint32_t col =
            row_mask ? ((uint32_t)c & row_mask) : (uint32_t)(c % chunks_per_row);
        const Chunk<T, V> b = load_chunk_cached<T, V>(bias + (uint64_t)col * V);
        Chunk<T, V> o;
#pragma unroll
        for (int i = 0; i < V; ++i) {
            const float x = Elem<T>::to_f32(in[u].v[i]) + Elem<T>::to_f32(b.v[i]);
            o.v[i] = Elem<T>::from_f32(gelu_fwd(x));
        }
        store_chunk<T, V>(out + c * V, o);
    }
}

// kDU = 16-byte chunks per thread: 2 without dropout (four loads in flight per thread: 8.6 us at
// bf16 8192 x 1024 with a residual, where any three-stream kernel of this size measures 9.6 us or
// more with one), 1 with it.  With dropout the Philox rounds (two blocks per 8 elements) are as
// much vector work as the kernel has memory time to hide it in, and wavefronts that all request
// first and draw second leave the memory system idle while they draw: odd wavefronts draw their
// bits BEFORE they request their data, even ones after, so that at any time half of a SIMD's
// wavefronts keep the vector ALU busy while the other half has requests in flight (12.1 -> 11.0 us
// at p = 0.1).
template <typename T, int V, bool kResidual, int kDrop, int kDU>
__global__ __launch_bounds__(256) void bias_dropout_residual_fwd_kernel(
    const T* __restrict__ x, const T* __restrict__ bias, const T* __restrict__ residual,
    T* __restrict__ out, uint64_t n_chunks, uint32_t chunks_per_row, uint32_t row_mask,
    DropoutState s) {
    if constexpr (kDrop != 0) resolve_device_state(s);
    const uint64_t base = (uint64_t)blockIdx.x * (256 * kDU) + threadIdx.x;
    Chunk<T, V> in[kDU];
    Chunk<T, V> res[kDU];
    uint32_t bits_u[kDU];
#pragma unroll
    for (int u = 0; u < kDU; ++u) bits_u[u] = 0xFFFFFFFFu;
    const bool draw_first = (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6) & 1) != 0;
    if constexpr (kDrop != 0) {
        if (draw_first) {
#pragma unroll
            for (int u = 0; u < kDU; ++u) {
                const uint64_t c = base + (uint64_t)u * 256;
                if (c < n_chunks) bits_u[u] = keep_bits<V, kDrop>(s, c * V);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int u = 0; u < kDU; ++u) {
        const uint64_t c = base + (uint64_t)u * 256;
        if (c < n_chunks) {
            in[u] = load_chunk<T, V>(x + c * V);
            if constexpr (kResidual) res[u] = load_chunk<T, V>(residual + c * V);
        }
    }
    if constexpr (kDrop != 0) {
        if (!draw_first) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < kDU; ++u) {
                const uint64_t c = base + (uint64_t)u * 256;
                if (c < n_chunks) bits_u[u] = keep_bits<V, kDrop>(s, c * V);
            }
        }
    }
#pragma unroll
    for (int u = 0; u < kDU; ++u) {
        const uint64_t c = base + (uint64_t)u * 256;
        if (c >= n_chunks) continue;
        const uint32_t col =
            row_mask ? ((uint32_t)c & row_mask) : (uint32_t)(c % chunks_per_row);
        const Chunk<T, V> b = load_chunk_cached<T, V>(bias + (uint64_t)col * V);
        const uint32_t bits = bits_u[u];
        Chunk<T, V> o;
#pragma unroll
        for (int i = 0; i < V; ++i) {
            float v = Elem<T>::to_f32(in[u].v[i]) + Elem<T>::to_f32(b.v[i]);
            if constexpr (kDrop != 0) v = ((bits >> i) & 1u) ? v * s.inv_keep : 0.0f;
            if constexpr (kResidual) v += Elem<T>::to_f32(res[u].v[i]);
            o.v[i] = Elem<T>::from_f32(v);
        }
        store_chunk<T, V>(out + c * V, o);
    }
}

// ----------------------------------------------------------------------------------------
// Backward kernels: a block is 64 column-chunks x 4 row-lanes and walks kRowsPerBlock rows,
// keeping per-thread fp32 column sums; the 4 row-lanes are combined through LDS and written
// as one fp32 partial row per block.
// ----------------------------------------------------------------------------------------
constexpr int kRowsPerBlock = 64;  // at most; see colsum_rows_per_block
constexpr int kRowLanes = 4;
constexpr int kColLanes = 64;

// Rows that one block walks: 64 where that still gives the device four blocks per CU or more,
// else 32 or 16 (a block's rows run one after the other, so a narrow matrix in few blocks is
// bound by latency: bf16 8192 x 1024 in 256 blocks of 64 rows took 15.7 us for 33.6 MB).  The
// choice depends on the shape alone, so that the workspace size and the finishing kernel agree
// with the launch.
inline int colsum_rows_per_block(int64_t rows, int64_t cols) {
    const int64_t col_blocks = (cols + 8 * kColLanes - 1) / (8 * kColLanes);
    int rpb = kRowsPerBlock;
    while (rpb > 16 && col_blocks * ((rows + rpb - 1) / rpb) < 1024) rpb /= 2;
    return rpb;
}

template <typename T, int V, typename F>
__device__ __forceinline__ void colsum_walk(int64_t rows, int64_t cols, float* __restrict__ partial,
                                            bool want_sum, int rows_per_block, F&& body) {
    const int cx = threadIdx.x % kColLanes;
    const int ry = threadIdx.x / kColLanes;
    const int64_t chunk_col = (int64_t)blockIdx.x * kColLanes + cx;
    const int64_t col0 = chunk_col * V;
    const bool active = col0 < cols;
    float acc[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = 0.f;
    const int64_t r_begin = (int64_t)blockIdx.y * rows_per_block;
    if (active) {
        if (r_begin + rows_per_block <= rows) {
            // a whole block of rows: no test between the iterations, so that the loads of an
            // unrolled group of four rows are requested together
#pragma unroll 4
            for (int it = 0; it < rows_per_block / kRowLanes; ++it)
                body(r_begin + ry + (int64_t)it * kRowLanes, col0, acc);
        } else {
            for (int it = 0; it < rows_per_block / kRowLanes; ++it) {
                const int64_t r = r_begin + ry + (int64_t)it * kRowLanes;
                if (r < rows) body(r, col0, acc);
            }
        }
    }
    if (!want_sum) return;
    __shared__ float red[kRowLanes][kColLanes][V + 1];
#pragma unroll
    for (int i = 0; i < V; ++i) red[ry][cx][i] = acc[i];
    __syncthreads();
    if (ry == 0 && active) {
#pragma unroll
        for (int i = 0; i < V; ++i) {
            float t = red[0][cx][i];
#pragma unroll
            for (int k = 1; k < kRowLanes; ++k) t += red[k][cx][i];
            partial[(int64_t)blockIdx.y * cols + col0 + i] = t;
        }
    }
}

template <typename T, int V>
__global__ __launch_bounds__(256) void bias_gelu_bwd_kernel(const T* __restrict__ grad,
                                                            const T* __restrict__ y,
                                                            const T* __restrict__ bias,
                                                            T* __restrict__ dx,
                                                            float* __restrict__ partial,
                                                            int64_t rows, int64_t cols,
                                                            int want_sum, int rows_per_block) {
    Chunk<T, V> b;
    {
        const int64_t col0 = ((int64_t)blockIdx.x * kColLanes + threadIdx.x % kColLanes) * V;
        if (col0 < cols) b = load_chunk_cached<T, V>(bias + col0);
    }
    colsum_walk<T, V>(rows, cols, partial, want_sum != 0, rows_per_block,
                      [&](int64_t r, int64_t col0, float* acc) {
                          const int64_t off = r * cols + col0;
                          const Chunk<T, V> g = load_chunk<T, V>(grad + off);
                          const Chunk<T, V> yy = load_chunk<T, V>(y + off);
                          Chunk<T, V> o;
#pragma unroll
                          for (int i = 0; i < V; ++i) {
                              const float x =
                                  Elem<T>::to_f32(yy.v[i]) + Elem<T>::to_f32(b.v[i]);
                              const float d = gelu_grad(x) * Elem<T>::to_f32(g.v[i]);
                              o.v[i] = Elem<T>::from_f32(d);
                              acc[i] += d;
                          }
                          store_chunk<T, V>(dx + off, o);
                      });
}

template <typename T, int V, int kDrop>
__global__ __launch_bounds__(256) void bias_dropout_bwd_kernel(const T* __restrict__ grad,
                                                               T* __restrict__ dx,
                                                               float* __restrict__ partial,
                                                               int64_t rows, int64_t cols,
                                                               int want_sum, int write_dx,
                                                               int rows_per_block,
                                                               DropoutState s) {
    if constexpr (kDrop != 0) resolve_device_state(s);
    colsum_walk<T, V>(rows, cols, partial, want_sum != 0, rows_per_block,
                      [&](int64_t r, int64_t col0, float* acc) {
                          const int64_t off = r * cols + col0;
                          const Chunk<T, V> g = load_chunk<T, V>(grad + off);
                          uint32_t bits = 0xFFFFFFFFu;
                          if constexpr (kDrop != 0) bits = keep_bits<V, kDrop>(s, (uint64_t)off);
                          Chunk<T, V> o;
#pragma unroll
                          for (int i = 0; i < V; ++i) {
                              float d = Elem<T>::to_f32(g.v[i]);
                              if constexpr (kDrop != 0)
                                  d = ((bits >> i) & 1u) ? d * s.inv_keep : 0.0f;
                              o.v[i] = Elem<T>::from_f32(d);
                              acc[i] += d;
                          }
                          if (write_dx) store_chunk<T, V>(dx + off, o);
                      });
}

// Second stage of the column reduction: a block owns 16 columns; its 16 row-lanes walk the partial
// rows with a stride of 16 (64-byte segments; the whole partial matrix is a few MB), then combine
// through LDS.  Many small blocks: the stage is latency bound, not bandwidth bound.
constexpr int kFinCols = 16;
constexpr int kFinRows = 16;
constexpr int kFinWide = 32;  // loads in flight per thread in the wide stage of a finishing kernel
template <typename T>
__global__ __launch_bounds__(256) void colsum_finish_kernel(const float* __restrict__ partial,
                                                            T* __restrict__ dbias,
                                                            int64_t n_partials, int64_t cols) {
    __shared__ float red[kFinRows][kFinCols + 1];
    const int cx = threadIdx.x % kFinCols;
    const int ry = threadIdx.x / kFinCols;
    const int64_t c = (int64_t)blockIdx.x * kFinCols + cx;
    float t = 0.f;
    if (c < cols) {
        float t0 = 0.f, t1 = 0.f, t2 = 0.f, t3 = 0.f;
        int64_t k = ry;
        // many partial rows (narrow matrices in blocks of 16 rows): 32 loads in flight per thread,
        // the stage is a chain of memory round trips (bias-dropout backward at bf16 8192 x 1024:
        // 14.5 -> 13.2 us with its finishing kernel)
        for (; k + (kFinWide - 1) * kFinRows < n_partials; k += kFinWide * kFinRows) {
            float v[kFinWide];
#pragma unroll
            for (int j = 0; j < kFinWide; ++j) v[j] = partial[(k + j * kFinRows) * cols + c];
#pragma unroll
            for (int j = 0; j < kFinWide; j += 4)
                t0 += v[j], t1 += v[j + 1], t2 += v[j + 2], t3 += v[j + 3];
        }
        for (; k + 3 * kFinRows < n_partials; k += 4 * kFinRows) {
            t0 += partial[k * cols + c];
            t1 += partial[(k + kFinRows) * cols + c];
            t2 += partial[(k + 2 * kFinRows) * cols + c];
            t3 += partial[(k + 3 * kFinRows) * cols + c];
        }
        for (; k < n_partials; k += kFinRows) t0 += partial[k * cols + c];
        t = (t0 + t1) + (t2 + t3);
    }
    red[ry][cx] = t;
    __syncthreads();
    if (ry == 0 && c < cols) {
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < kFinRows; ++r) sum += red[r][cx];
        dbias[c] = Elem<T>::from_f32(sum);
    }
}

// ----------------------------------------------------------------------------------------
// bias + dropout + residual + LayerNorm (the fusion pattern of tests/test_fusion.py:157-204:
// layer_norm(dropout(x + bias) + residual)).
//
// A row is owned by TPR threads: one wavefront (TPR = 64) up to 64 * V * 2 columns, the
// whole block (TPR = 256) above, so that every row value stays in registers between the two
// passes of the statistics and is read from memory once.  z = dropout(x + bias) + residual is
// rounded to T first and the statistics are taken from the rounded values, i.e. exactly what the
// unfused modules compute from the stored sum; z is also what the backward reads.
// ----------------------------------------------------------------------------------------
constexpr int kLnChunks = 4;         // 16-byte chunks per thread and row (guarded against cols)
constexpr int kLnRowsPerBlock = 16;  // backward: rows walked by one block (column partial sums)

// Sum over the 64 lanes, on every lane, without LDS traffic: butterflies inside the 16-lane
// rows through DPP (quad permutes, row rotations), then the four row sums through v_readlane.
template <int kCtrl>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xF, 0xF, false));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_move<0x124>(v);  // row_ror 4
    v += dpp_move<0x128>(v);  // row_ror 8
    const float r0 = __builtin_bit_cast(
        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float r1 = __builtin_bit_cast(
        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    const float r2 = __builtin_bit_cast(
        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    const float r3 = __builtin_bit_cast(
        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (r0 + r1) + (r2 + r3);
}
// Sum over the TPR threads of a row.  red: 4 floats of LDS that no other reduction in flight uses
// (TPR == 256 only; every thread of the block has to call).
template <int TPR>
__device__ __forceinline__ float row_sum(float v, float* red) {
    v = wave_sum(v);
    if constexpr (TPR == 256) {
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
        __syncthreads();
        v = (red[0] + red[1]) + (red[2] + red[3]);
    }
    return v;
}

template <typename T, int V, int TPR, int kDrop>
__global__ __launch_bounds__(256) void bias_dropout_residual_ln_fwd_kernel(
    const T* __restrict__ x, const T* __restrict__ bias, const T* __restrict__ residual,
    const T* __restrict__ gamma, const T* __restrict__ beta, T* __restrict__ z_out,
    T* __restrict__ y, float* __restrict__ mean_out, float* __restrict__ rstd_out, int64_t rows,
    int cols, float eps, DropoutState s) {
    if constexpr (kDrop != 0) resolve_device_state(s);
    constexpr int kRows = 256 / TPR;  // rows per block
    __shared__ float red[2][4];
    const int sub = threadIdx.x % TPR;
    const int64_t row = (int64_t)blockIdx.x * kRows + threadIdx.x / TPR;
    const bool row_ok = row < rows;  // uniform per wavefront
    float zf[kLnChunks][V];
    float sum = 0.f;
    // odd wavefronts draw their dropout bits before they request their data, even ones after (see
    // bias_dropout_residual_fwd_kernel)
    uint32_t bits_u[kLnChunks];
#pragma unroll
    for (int u = 0; u < kLnChunks; ++u) bits_u[u] = 0xFFFFFFFFu;
    const bool draw_first = (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6) & 1) != 0;
    if constexpr (kDrop != 0) {
        if (draw_first) {
#pragma unroll
            for (int u = 0; u < kLnChunks; ++u) {
                const int col0 = (sub + u * TPR) * V;
                if (row_ok && col0 < cols)
                    bits_u[u] = keep_bits<V, kDrop>(s, (uint64_t)(row * cols + col0));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int u = 0; u < kLnChunks; ++u) {
        const int col0 = (sub + u * TPR) * V;
#pragma unroll
        for (int i = 0; i < V; ++i) zf[u][i] = 0.f;
        if (row_ok && col0 < cols) {
            const int64_t off = row * cols + col0;
            const Chunk<T, V> xin = load_chunk<T, V>(x + off);
            Chunk<T, V> b, r;
            if (bias) b = load_chunk_cached<T, V>(bias + col0);
            if (residual) r = load_chunk<T, V>(residual + off);
            uint32_t bits = bits_u[u];
            if constexpr (kDrop != 0) {
                if (!draw_first) bits = keep_bits<V, kDrop>(s, (uint64_t)off);
            }
            Chunk<T, V> zc;
#pragma unroll
            for (int i = 0; i < V; ++i) {
                float v = Elem<T>::to_f32(xin.v[i]);
                if (bias) v += Elem<T>::to_f32(b.v[i]);
                if constexpr (kDrop != 0) v = ((bits >> i) & 1u) ? v * s.inv_keep : 0.0f;
                if (residual) v += Elem<T>::to_f32(r.v[i]);
                zc.v[i] = Elem<T>::from_f32(v);
                zf[u][i] = Elem<T>::to_f32(zc.v[i]);
                sum += zf[u][i];
            }
            if (z_out) store_chunk<T, V>(z_out + off, zc);
        }
    }
    const float inv_n = 1.0f / (float)cols;
    const float mean = row_sum<TPR>(sum, red[0]) * inv_n;
    float sq = 0.f;
#pragma unroll
    for (int u = 0; u < kLnChunks; ++u) {
        if ((sub + u * TPR) * V < cols) {
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const float d = zf[u][i] - mean;
                sq = __builtin_fmaf(d, d, sq);
            }
        }
    }
    const float var = row_sum<TPR>(sq, red[1]) * inv_n;
    const float rstd = 1.0f / __builtin_sqrtf(var + eps);
    if (!row_ok) return;
#pragma unroll
    for (int u = 0; u < kLnChunks; ++u) {
        const int col0 = (sub + u * TPR) * V;
        if (col0 < cols) {
            const Chunk<T, V> g = load_chunk_cached<T, V>(gamma + col0);
            const Chunk<T, V> be = load_chunk_cached<T, V>(beta + col0);
            Chunk<T, V> o;
#pragma unroll
            for (int i = 0; i < V; ++i)
                o.v[i] = Elem<T>::from_f32(__builtin_fmaf((zf[u][i] - mean) * rstd,
                                                          Elem<T>::to_f32(g.v[i]),
                                                          Elem<T>::to_f32(be.v[i])));
            store_chunk<T, V>(y + row * cols + col0, o);
        }
    }
    if (sub == 0) {
        if (mean_out) mean_out[row] = mean;
        if (rstd_out) rstd_out[row] = rstd;
    }
}

// Backward of the above.  With xh = (z - mean) rstd and g = dy gamma:
//   dz = rstd (g - mean_c(g) - xh mean_c(g xh)),  dresidual = dz,  dx = dz keep / (1 - p),
//   dgamma = sum_r dy xh,  dbeta = sum_r dy,  dbias = sum_r dx.
// A block walks kLnRowsPerBlock rows and keeps the three column sums of its threads in
// registers; they leave as one fp32 partial row triple per block ([block][3][cols]: dgamma, dbeta,
// dbias) for ln_finish_kernel.  No atomics: the result does not depend on scheduling.
// NV = 16-byte chunks per thread and row (1, 2 or 4, the smallest that covers cols): the column
// sums cost 3 * NV * V registers, and registers decide how many rows a CU has in flight.  The
// loads of the next two rows are issued before the current row is reduced.
template <typename T, int V, int NV, int TPR, int kDrop, int kThreads>
__global__ __launch_bounds__(kThreads, (kThreads == 512 && kDrop != 2) ? 4 : 1)
void bias_dropout_residual_ln_bwd_kernel(
    const T* __restrict__ dy, const T* __restrict__ z, const float* __restrict__ mean,
    const float* __restrict__ rstd, const T* __restrict__ gamma, T* __restrict__ dx,
    T* __restrict__ dres, float* __restrict__ partial, int64_t rows, int cols, DropoutState s) {
    if constexpr (kDrop != 0) resolve_device_state(s);
    static_assert(TPR == 256 ? kThreads == 256 : (kThreads == 256 || kThreads == 512),
                  "a block is one wide row, or four or eight wavefront rows");
    constexpr int kRows = kThreads / TPR;  // rows in flight per block
    constexpr int kIters = kLnRowsPerBlock / kRows;
    constexpr int kCombCols = TPR == 64 ? 64 * V * NV : 1;
    __shared__ float red[2][2][4];
    __shared__ float comb[4 * 3 * kCombCols];
    const int sub = threadIdx.x % TPR;
    const int rr = threadIdx.x / TPR;
    Chunk<T, V> gm[NV];
    float acc_g[NV][V], acc_b[NV][V], acc_x[NV][V];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int col0 = (sub + u * TPR) * V;
        if (col0 < cols) gm[u] = load_chunk_cached<T, V>(gamma + col0);
#pragma unroll
        for (int i = 0; i < V; ++i) acc_g[u][i] = 0.f, acc_b[u][i] = 0.f, acc_x[u][i] = 0.f;
    }
    const float inv_n = 1.0f / (float)cols;
    const int64_t row0 = (int64_t)blockIdx.x * kLnRowsPerBlock + rr;

    // rows it + 1 and it + 2 are in flight while row it is processed
    Chunk<T, V> gy[NV], zz[NV], gy_n1[NV], zz_n1[NV], gy_n2[NV], zz_n2[NV];
    float m = 0.f, rs = 0.f, m_n1 = 0.f, rs_n1 = 0.f, m_n2 = 0.f, rs_n2 = 0.f;
    auto request = [&](int64_t row, Chunk<T, V> (&g)[NV], Chunk<T, V> (&zc)[NV], float& mm,
                       float& rr_) __attribute__((always_inline)) {
        if (row < rows) {  // uniform per wavefront
            mm = mean[row];
            rr_ = rstd[row];
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                const int col0 = (sub + u * TPR) * V;
                if (col0 < cols) {
                    g[u] = load_chunk<T, V>(dy + row * cols + col0);
                    zc[u] = load_chunk<T, V>(z + row * cols + col0);
                }
            }
        }
    };
    request(row0, gy, zz, m, rs);
    if (kIters > 1) request(row0 + kRows, gy_n1, zz_n1, m_n1, rs_n1);
#pragma unroll 1
    for (int it = 0; it < kIters; ++it) {
        const int64_t row = row0 + it * kRows;
        const bool row_ok = row < rows;  // uniform per wavefront
        if (it + 2 < kIters) request(row + 2 * kRows, gy_n2, zz_n2, m_n2, rs_n2);
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int col0 = (sub + u * TPR) * V;
            if (row_ok && col0 < cols) {
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const float d = Elem<T>::to_f32(gy[u].v[i]);
                    const float xh = (Elem<T>::to_f32(zz[u].v[i]) - m) * rs;
                    const float g = d * Elem<T>::to_f32(gm[u].v[i]);
                    s1 += g;
                    s2 = __builtin_fmaf(g, xh, s2);
                    acc_g[u][i] = __builtin_fmaf(d, xh, acc_g[u][i]);
                    acc_b[u][i] += d;
                }
            }
        }
        const float c1 = row_sum<TPR>(s1, red[it & 1][0]) * inv_n;
        const float c2 = row_sum<TPR>(s2, red[it & 1][1]) * inv_n;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int col0 = (sub + u * TPR) * V;
            if (row_ok && col0 < cols) {
                const int64_t off = row * cols + col0;
                uint32_t bits = 0xFFFFFFFFu;
                if constexpr (kDrop != 0) bits = keep_bits<V, kDrop>(s, (uint64_t)off);
                Chunk<T, V> oz, ox;
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const float xh = (Elem<T>::to_f32(zz[u].v[i]) - m) * rs;
                    const float g = Elem<T>::to_f32(gy[u].v[i]) * Elem<T>::to_f32(gm[u].v[i]);
                    const float dz = rs * (g - c1 - xh * c2);
                    float d = dz;
                    if constexpr (kDrop != 0) d = ((bits >> i) & 1u) ? dz * s.inv_keep : 0.0f;
                    oz.v[i] = Elem<T>::from_f32(dz);
                    ox.v[i] = Elem<T>::from_f32(d);
                    acc_x[u][i] += d;
                }
                if (dres) store_chunk<T, V>(dres + off, oz);
                if (dx) store_chunk<T, V>(dx + off, ox);
            }
        }
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            gy[u] = gy_n1[u], zz[u] = zz_n1[u];
            gy_n1[u] = gy_n2[u], zz_n1[u] = zz_n2[u];
        }
        m = m_n1, rs = rs_n1, m_n1 = m_n2, rs_n1 = rs_n2;
    }
    if (!partial) return;
    float* out = partial + (int64_t)blockIdx.x * 3 * cols;
    if constexpr (TPR == 256) {
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int col0 = (sub + u * TPR) * V;
            if (col0 < cols) {
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    out[col0 + i] = acc_g[u][i];
                    out[cols + col0 + i] = acc_b[u][i];
                    out[2 * cols + col0 + i] = acc_x[u][i];
                }
            }
        }
    } else {
        // every wavefront (row group) parks its sums in LDS, then the block adds the four copies
        // column by column and writes the partial row with consecutive lanes on consecutive
        // columns
        float* mine = comb + (rr & 3) * 3 * kCombCols;
        if constexpr (kRows == 8) {
            // the upper four wavefronts hand their sums to the lower four first, so that the
            // parking area stays at four copies
            if (rr >= 4) {
#pragma unroll
                for (int u = 0; u < NV; ++u) {
                    const int col0 = (sub + u * TPR) * V;
                    if (col0 < cols) {
#pragma unroll
                        for (int i = 0; i < V; ++i) {
                            mine[col0 + i] = acc_g[u][i];
                            mine[kCombCols + col0 + i] = acc_b[u][i];
                            mine[2 * kCombCols + col0 + i] = acc_x[u][i];
                        }
                    }
                }
            }
            __syncthreads();
            if (rr < 4) {
#pragma unroll
                for (int u = 0; u < NV; ++u) {
                    const int col0 = (sub + u * TPR) * V;
                    if (col0 < cols) {
#pragma unroll
                        for (int i = 0; i < V; ++i) {
                            acc_g[u][i] += mine[col0 + i];
                            acc_b[u][i] += mine[kCombCols + col0 + i];
                            acc_x[u][i] += mine[2 * kCombCols + col0 + i];
                        }
                    }
                }
            }
            __syncthreads();
        }
        if (rr < 4) {
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                const int col0 = (sub + u * TPR) * V;
                if (col0 < cols) {
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        mine[col0 + i] = acc_g[u][i];
                        mine[kCombCols + col0 + i] = acc_b[u][i];
                        mine[2 * kCombCols + col0 + i] = acc_x[u][i];
                    }
                }
            }
        }
        __syncthreads();
        for (int c = threadIdx.x; c < 3 * cols; c += kThreads) {
            const int which = c / cols;
            const int idx = which * kCombCols + (c - which * cols);
            out[c] = (comb[idx] + comb[3 * kCombCols + idx]) +
                     (comb[6 * kCombCols + idx] + comb[9 * kCombCols + idx]);
        }
    }
}

// Second stage: partial is [n_partials][3 * cols]; column c of it belongs to dgamma (c < cols),
// dbeta or dbias.  A block owns kFC columns and kFR row-lanes (kFC * kFR = 256): narrow tiles for
// small matrices (many blocks, the stage is a chain of L2 round trips), 256-byte segments for
// large ones (the stage is then bound by reading the partials).
template <typename T, int kFC, int kFR>
__global__ __launch_bounds__(256) void ln_finish_kernel(const float* __restrict__ partial,
                                                        T* __restrict__ dgamma,
                                                        T* __restrict__ dbeta,
                                                        T* __restrict__ dbias, int64_t n_partials,
                                                        int cols) {
    static_assert(kFC * kFR == 256, "one thread per (column, row-lane)");
    __shared__ float red[kFR][kFC + 1];
    const int cx = threadIdx.x % kFC;
    const int ry = threadIdx.x / kFC;
    const int64_t cols3 = 3 * (int64_t)cols;
    const int64_t c = (int64_t)blockIdx.x * kFC + cx;
    float t = 0.f;
    if (c < cols3) {
        // 32 loads in flight per thread while that many rows are left, then eight
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        int64_t k = ry;
        for (; k + (kFinWide - 1) * kFR < n_partials; k += kFinWide * kFR) {
            float v[kFinWide];
#pragma unroll
            for (int j = 0; j < kFinWide; ++j) v[j] = partial[(k + j * kFR) * cols3 + c];
#pragma unroll
            for (int j = 0; j < kFinWide; ++j) acc[j & 7] += v[j];
        }
        for (; k + 7 * kFR < n_partials; k += 8 * kFR) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = partial[(k + j * kFR) * cols3 + c];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] += v[j];
        }
        for (; k < n_partials; k += kFR) acc[0] += partial[k * cols3 + c];
        t = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
    }
    red[ry][cx] = t;
    __syncthreads();
    if (ry == 0 && c < cols3) {
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < kFR; ++r) sum += red[r][cx];
        const int which = (int)(c / cols);
        T* dst = which == 0 ? dgamma : which == 1 ? dbeta : dbias;
        if (dst) dst[c - (int64_t)which * cols] = Elem<T>::from_f32(sum);
    }
}

// ----------------------------------------------------------------------------------------
// Host dispatch
// ----------------------------------------------------------------------------------------
struct RowGeom {
    uint64_t n_chunks;
    uint32_t chunks_per_row;
    uint32_t row_mask;
    unsigned blocks;
};

inline bool flat_geom(int64_t rows, int64_t cols, int v, RowGeom* g, int unroll = kUnroll) {
    const int64_t cpr = cols / v;
    if (cpr > 0x7FFFFFFF) return false;
    g->chunks_per_row = (uint32_t)cpr;
    g->n_chunks = (uint64_t)rows * (uint64_t)cpr;
    g->row_mask = (cpr & (cpr - 1)) == 0 ? (uint32_t)(cpr - 1) : 0u;
    if (cpr == 1) g->row_mask = 0;  // mask 0 means "use modulo"; modulo by 1 is fine
    const uint64_t per_block = 256ull * (uint64_t)unroll;
    const uint64_t blocks = (g->n_chunks + per_block - 1) / per_block;
    if (blocks > 0x7FFFFFFFull) return false;
    g->blocks = (unsigned)blocks;
    return true;
}

template <typename T>
inline bool vector_ok(int64_t cols, std::initializer_list<const void*> ptrs) {
    if (cols % Elem<T>::kPerVec != 0) return false;
    for (const void* p : ptrs)
        if (p && !aligned16(p)) return false;
    return true;
}

template <typename T>
int gelu_fwd_dispatch(const void* y, const void* bias, void* out, int64_t rows, int64_t cols,
                      hipStream_t st) {
    RowGeom g;
    if (vector_ok<T>(cols, {y, bias, out})) {
        constexpr int V = Elem<T>::kPerVec;
        if (!flat_geom(rows, cols, V, &g)) return SLAPO_ERR_SHAPE;
        hipLaunchKernelGGL((bias_gelu_fwd_kernel<T, V>), dim3(g.blocks), dim3(256), 0, st,
                           (const T*)y, (const T*)bias, (T*)out, g.n_chunks, g.chunks_per_row,
                           g.row_mask);
    } else {
        if (!flat_geom(rows, cols, 1, &g)) return SLAPO_ERR_SHAPE;
        hipLaunchKernelGGL((bias_gelu_fwd_kernel<T, 1>), dim3(g.blocks), dim3(256), 0, st,
                           (const T*)y, (const T*)bias, (T*)out, g.n_chunks, g.chunks_per_row,
                           g.row_mask);
    }
    return check_launch();
}

template <typename T, int V>
int dropres_fwd_launch(const void* x, const void* bias, const void* residual, void* out,
                       int64_t rows, int64_t cols, bool dropout, const DropoutState& s,
                       hipStream_t st) {
    RowGeom g;
    if (!flat_geom(rows, cols, V, &g, dropout ? 1 : 2)) return SLAPO_ERR_SHAPE;
#define SLAPO_LAUNCH_DR(RES, DROP)                                                             \
    hipLaunchKernelGGL((bias_dropout_residual_fwd_kernel<T, V, RES, DROP, (DROP == 0 ? 2 : 1)>), \
                       dim3(g.blocks), dim3(256), 0, st, (const T*)x, (const T*)bias,          \
                       (const T*)residual, (T*)out, g.n_chunks, g.chunks_per_row, g.row_mask, s)
    // dropout mode: the shift-only geometry needs whole Philox blocks per chunk
    const int mode = !dropout ? 0 : (V % 4 == 0 && s.g_shift >= 0 && s.t_shift >= 0) ? 1 : 2;
    if (residual) {
        if (mode == 0) SLAPO_LAUNCH_DR(true, 0);
        if constexpr (V % 4 == 0) {
            if (mode == 1) SLAPO_LAUNCH_DR(true, 1);
        }
        if (mode == 2) SLAPO_LAUNCH_DR(true, 2);
    } else {
        if (mode == 0) SLAPO_LAUNCH_DR(false, 0);
        if constexpr (V % 4 == 0) {
            if (mode == 1) SLAPO_LAUNCH_DR(false, 1);
        }
        if (mode == 2) SLAPO_LAUNCH_DR(false, 2);
    }
#undef SLAPO_LAUNCH_DR
    return check_launch();
}

inline bool bwd_grid(int64_t rows, int64_t cols, int v, dim3* grid) {
    const int64_t chunk_cols = (cols + v - 1) / v;
    const int64_t gx = (chunk_cols + kColLanes - 1) / kColLanes;
    const int rpb = colsum_rows_per_block(rows, cols);
    const int64_t gy = (rows + rpb - 1) / rpb;
    if (gx > 0x7FFFFFFF || gy > 65535) return false;
    *grid = dim3((unsigned)gx, (unsigned)gy);
    return true;
}

template <typename T>
int finish_colsum(const float* partial, void* dbias, int64_t rows, int64_t cols, hipStream_t st) {
    const int rpb = colsum_rows_per_block(rows, cols);
    const int64_t n_partials = (rows + rpb - 1) / rpb;
    const unsigned blocks = (unsigned)((cols + kFinCols - 1) / kFinCols);
    hipLaunchKernelGGL((colsum_finish_kernel<T>), dim3(blocks), dim3(256), 0, st, partial,
                       (T*)dbias, n_partials, cols);
    return check_launch();
}

template <typename T>
int gelu_bwd_dispatch(const void* grad, const void* y, const void* bias, void* dx, void* dbias,
                      void* ws, int64_t rows, int64_t cols, hipStream_t st) {
    dim3 grid;
    const int want = dbias ? 1 : 0;
    if (vector_ok<T>(cols, {grad, y, bias, dx})) {
        constexpr int V = Elem<T>::kPerVec;
        if (!bwd_grid(rows, cols, V, &grid)) return SLAPO_ERR_SHAPE;
        hipLaunchKernelGGL((bias_gelu_bwd_kernel<T, V>), grid, dim3(256), 0, st, (const T*)grad,
                           (const T*)y, (const T*)bias, (T*)dx, (float*)ws, rows, cols, want,
                           colsum_rows_per_block(rows, cols));
    } else {
        if (!bwd_grid(rows, cols, 1, &grid)) return SLAPO_ERR_SHAPE;
        hipLaunchKernelGGL((bias_gelu_bwd_kernel<T, 1>), grid, dim3(256), 0, st, (const T*)grad,
                           (const T*)y, (const T*)bias, (T*)dx, (float*)ws, rows, cols, want,
                           colsum_rows_per_block(rows, cols));
    }
    int rc = check_launch();
    if (rc != SLAPO_OK || !dbias) return rc;
    return finish_colsum<T>((const float*)ws, dbias, rows, cols, st);
}

template <typename T, int V>
int dropres_bwd_launch(const void* grad, void* dx, void* ws, int64_t rows, int64_t cols,
                       bool dropout, int want, const DropoutState& s, hipStream_t st) {
    dim3 grid;
    if (!bwd_grid(rows, cols, V, &grid)) return SLAPO_ERR_SHAPE;
    const int write_dx = dx ? 1 : 0;
#define SLAPO_LAUNCH_DB(MODE)                                                                  \
    hipLaunchKernelGGL((bias_dropout_bwd_kernel<T, V, MODE>), grid, dim3(256), 0, st,          \
                       (const T*)grad, (T*)dx, (float*)ws, rows, cols, want, write_dx,            \
                       colsum_rows_per_block(rows, cols), s)
    const int mode = !dropout ? 0 : (V % 4 == 0 && s.g_shift >= 0 && s.t_shift >= 0) ? 1 : 2;
    if (mode == 0) SLAPO_LAUNCH_DB(0);
    if constexpr (V % 4 == 0) {
        if (mode == 1) SLAPO_LAUNCH_DB(1);
    }
    if (mode == 2) SLAPO_LAUNCH_DB(2);
#undef SLAPO_LAUNCH_DB
    return check_launch();
}

template <typename T>
int dropres_fwd_dispatch(const void* x, const void* bias, const void* residual, void* out,
                         int64_t rows, int64_t cols, bool dropout, const DropoutState& s,
                         hipStream_t st) {
    if (vector_ok<T>(cols, {x, bias, residual, out}))
        return dropres_fwd_launch<T, Elem<T>::kPerVec>(x, bias, residual, out, rows, cols,
                                                       dropout, s, st);
    return dropres_fwd_launch<T, 1>(x, bias, residual, out, rows, cols, dropout, s, st);
}

template <typename T>
int dropres_bwd_dispatch(const void* grad, void* dx, void* dbias, void* ws, int64_t rows,
                         int64_t cols, bool dropout, const DropoutState& s, hipStream_t st) {
    const int want = dbias ? 1 : 0;
    int rc;
    if (vector_ok<T>(cols, {grad, dx}))
        rc = dropres_bwd_launch<T, Elem<T>::kPerVec>(grad, dx, ws, rows, cols, dropout, want, s,
                                                     st);
    else
        rc = dropres_bwd_launch<T, 1>(grad, dx, ws, rows, cols, dropout, want, s, st);
    if (rc != SLAPO_OK || !dbias) return rc;
    return finish_colsum<T>((const float*)ws, dbias, rows, cols, st);
}

template <typename T>
inline int ln_geometry(int64_t rows, int64_t cols, bool* wide) {
    constexpr int V = Elem<T>::kPerVec;
    if (cols % V != 0) return SLAPO_ERR_ALIGN;
    if (cols > 256 * V * kLnChunks) return SLAPO_ERR_SHAPE;
    *wide = cols > 64 * V * 2;  // a wavefront per row up to two chunks per lane, a block above
    if (rows > 0x7FFFFFFF) return SLAPO_ERR_SHAPE;
    return SLAPO_OK;
}

template <typename T>
int ln_fwd_dispatch(const void* x, const void* bias, const void* residual, const void* gamma,
                    const void* beta, void* z, void* y, float* mean, float* rstd, int64_t rows,
                    int64_t cols, float eps, bool dropout, const DropoutState& s,
                    hipStream_t st) {
    constexpr int V = Elem<T>::kPerVec;
    bool wide = false;
    int rc = ln_geometry<T>(rows, cols, &wide);
    if (rc != SLAPO_OK) return rc;
    for (const void* p : {x, bias, residual, gamma, beta, (const void*)z, (const void*)y})
        if (p && !aligned16(p)) return SLAPO_ERR_ALIGN;
    const int mode = !dropout ? 0 : (s.g_shift >= 0 && s.t_shift >= 0) ? 1 : 2;
#define SLAPO_LAUNCH_LN(TPR, MODE)                                                              \
    hipLaunchKernelGGL((bias_dropout_residual_ln_fwd_kernel<T, V, TPR, MODE>),                  \
                       dim3((unsigned)((rows + (256 / TPR) - 1) / (256 / TPR))), dim3(256), 0,  \
                       st, (const T*)x, (const T*)bias, (const T*)residual, (const T*)gamma,    \
                       (const T*)beta, (T*)z, (T*)y, mean, rstd, rows, (int)cols, eps, s)
    if (wide) {
        if (mode == 0) SLAPO_LAUNCH_LN(256, 0);
        if (mode == 1) SLAPO_LAUNCH_LN(256, 1);
        if (mode == 2) SLAPO_LAUNCH_LN(256, 2);
    } else {
        if (mode == 0) SLAPO_LAUNCH_LN(64, 0);
        if (mode == 1) SLAPO_LAUNCH_LN(64, 1);
        if (mode == 2) SLAPO_LAUNCH_LN(64, 2);
    }
#undef SLAPO_LAUNCH_LN
    return check_launch();
}

template <typename T>
int ln_bwd_dispatch(const void* dy, const void* z, const float* mean, const float* rstd,
                    const void* gamma, void* dx, void* dres, void* dgamma, void* dbeta,
                    void* dbias, void* ws, int64_t rows, int64_t cols, bool dropout,
                    const DropoutState& s, hipStream_t st) {
    constexpr int V = Elem<T>::kPerVec;
    bool wide = false;
    int rc = ln_geometry<T>(rows, cols, &wide);
    if (rc != SLAPO_OK) return rc;
    for (const void* p : {dy, z, gamma, (const void*)dx, (const void*)dres})
        if (p && !aligned16(p)) return SLAPO_ERR_ALIGN;
    const bool want_sums = dgamma || dbeta || dbias;
    const int64_t n_blocks = (rows + kLnRowsPerBlock - 1) / kLnRowsPerBlock;
    float* partial = want_sums ? (float*)ws : nullptr;
    const int mode = !dropout ? 0 : (s.g_shift >= 0 && s.t_shift >= 0) ? 1 : 2;
#define SLAPO_LAUNCH_LNB(NV, TPR, MODE)                                                         \
    hipLaunchKernelGGL(                                                                         \
        (bias_dropout_residual_ln_bwd_kernel<T, V, NV, TPR, MODE, (TPR == 64 ? 512 : 256)>),    \
        dim3((unsigned)n_blocks), dim3(TPR == 64 ? 512 : 256), 0, st, (const T*)dy,             \
        (const T*)z, mean, rstd, (const T*)gamma, (T*)dx, (T*)dres, partial, rows, (int)cols, s)
#define SLAPO_LAUNCH_LNB_MODE(NV, TPR)            \
    do {                                          \
        if (mode == 0) SLAPO_LAUNCH_LNB(NV, TPR, 0); \
        if (mode == 1) SLAPO_LAUNCH_LNB(NV, TPR, 1); \
        if (mode == 2) SLAPO_LAUNCH_LNB(NV, TPR, 2); \
    } while (0)
    const int tpr = wide ? 256 : 64;
    const int chunks = (int)((cols / V + tpr - 1) / tpr);  // per thread and row, 1..kLnChunks
    if (wide) {
        if (chunks <= 1)
            SLAPO_LAUNCH_LNB_MODE(1, 256);
        else if (chunks <= 2)
            SLAPO_LAUNCH_LNB_MODE(2, 256);
        else
            SLAPO_LAUNCH_LNB_MODE(4, 256);
    } else {
        if (chunks <= 1)
            SLAPO_LAUNCH_LNB_MODE(1, 64);
        else
            SLAPO_LAUNCH_LNB_MODE(2, 64);
    }
#undef SLAPO_LAUNCH_LNB_MODE
#undef SLAPO_LAUNCH_LNB
    rc = check_launch();
    if (rc != SLAPO_OK || !want_sums) return rc;
    if (3 * cols >= 6144) {
        hipLaunchKernelGGL((ln_finish_kernel<T, 64, 4>), dim3((unsigned)((3 * cols + 63) / 64)),
                           dim3(256), 0, st, partial, (T*)dgamma, (T*)dbeta, (T*)dbias, n_blocks,
                           (int)cols);
    } else {
        hipLaunchKernelGGL((ln_finish_kernel<T, 16, 16>), dim3((unsigned)((3 * cols + 15) / 16)),
                           dim3(256), 0, st, partial, (T*)dgamma, (T*)dbeta, (T*)dbias, n_blocks,
                           (int)cols);
    }
    return check_launch();
}

inline bool dims_ok(int64_t rows, int64_t cols) {
    return rows > 0 && cols > 0 && rows <= (int64_t)1 << 40 && cols <= (int64_t)1 << 30;
}

}  // namespace

#define SLAPO_DISPATCH_DTYPE(dtype, CALL)   \
    switch (dtype) {                        \
        case SLAPO_F32: return CALL(float); \
        case SLAPO_F16: return CALL(f16_t); \
        case SLAPO_BF16: return CALL(bf16_t); \
        default: return SLAPO_ERR_DTYPE;    \
    }

extern "C" size_t slapo_amd_colsum_workspace_bytes(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    const int rpb = colsum_rows_per_block(rows, cols);
    const int64_t n_partials = (rows + rpb - 1) / rpb;
    return (size_t)n_partials * (size_t)cols * sizeof(float);
}

extern "C" int slapo_amd_bias_gelu_fwd(const void* y, const void* bias, void* out, int64_t rows,
                                       int64_t cols, int dtype, void* stream) {
    if (!y || !bias || !out) return SLAPO_ERR_ARG;
    if (!dims_ok(rows, cols)) return SLAPO_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
#define CALL(T) gelu_fwd_dispatch<T>(y, bias, out, rows, cols, st)
    SLAPO_DISPATCH_DTYPE(dtype, CALL)
#undef CALL
}

extern "C" int slapo_amd_bias_gelu_bwd(const void* grad, const void* y, const void* bias,
                                       void* dx, void* dbias, void* workspace,
                                       size_t workspace_bytes, int64_t rows, int64_t cols,
                                       int dtype, void* stream) {
    if (!grad || !y || !bias || !dx) return SLAPO_ERR_ARG;
    if (!dims_ok(rows, cols)) return SLAPO_ERR_SHAPE;
    if (dbias && (!workspace || workspace_bytes < slapo_amd_colsum_workspace_bytes(rows, cols)))
        return SLAPO_ERR_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
#define CALL(T) gelu_bwd_dispatch<T>(grad, y, bias, dx, dbias, workspace, rows, cols, st)
    SLAPO_DISPATCH_DTYPE(dtype, CALL)
#undef CALL
}

extern "C" int slapo_amd_bias_dropout_residual_fwd(const void* x, const void* bias,
                                                   const void* residual, void* out, int64_t rows,
                                                   int64_t cols, int dtype, double p,
                                                   uint64_t seed, uint64_t offset,
                                                   const slapo_dropout_plan* plan, void* stream) {
    if (!x || !bias || !out) return SLAPO_ERR_ARG;
    if (!dims_ok(rows, cols)) return SLAPO_ERR_SHAPE;
    if (!(p >= 0.0 && p <= 1.0)) return SLAPO_ERR_ARG;
    const bool dropout = p > 0.0;
    DropoutState s = {};
    if (dropout) {
        if (!plan_ok(plan, rows * cols)) return SLAPO_ERR_ARG;
        s = make_dropout_state(*plan, p, seed, offset);
    }
    hipStream_t st = (hipStream_t)stream;
#define CALL(T) dropres_fwd_dispatch<T>(x, bias, residual, out, rows, cols, dropout, s, st)
    SLAPO_DISPATCH_DTYPE(dtype, CALL)
#undef CALL
}

extern "C" int slapo_amd_bias_dropout_residual_bwd(const void* grad, void* dx, void* dbias,
                                                   void* workspace, size_t workspace_bytes,
                                                   int64_t rows, int64_t cols, int dtype,
                                                   double p, uint64_t seed, uint64_t offset,
                                                   const slapo_dropout_plan* plan, void* stream) {
    if (!grad || (!dx && !dbias)) return SLAPO_ERR_ARG;
    if (!dims_ok(rows, cols)) return SLAPO_ERR_SHAPE;
    if (!(p >= 0.0 && p <= 1.0)) return SLAPO_ERR_ARG;
    if (dbias && (!workspace || workspace_bytes < slapo_amd_colsum_workspace_bytes(rows, cols)))
        return SLAPO_ERR_WORKSPACE;
    const bool dropout = p > 0.0;
    DropoutState s = {};
    if (dropout) {
        if (!plan_ok(plan, rows * cols)) return SLAPO_ERR_ARG;
        s = make_dropout_state(*plan, p, seed, offset);
    }
    hipStream_t st = (hipStream_t)stream;
#define CALL(T) dropres_bwd_dispatch<T>(grad, dx, dbias, workspace, rows, cols, dropout, s, st)
    SLAPO_DISPATCH_DTYPE(dtype, CALL)
#undef CALL
}

extern "C" size_t slapo_amd_ln_bwd_workspace_bytes(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    const int64_t n_blocks = (rows + kLnRowsPerBlock - 1) / kLnRowsPerBlock;
    return (size_t)n_blocks * 3 * (size_t)cols * sizeof(float);
}

extern "C" int slapo_amd_bias_dropout_residual_ln_fwd(
    const void* x, const void* bias, const void* residual, const void* gamma, const void* beta,
    void* z, void* y, float* mean, float* rstd, int64_t rows, int64_t cols, int dtype,
    double eps, double p, uint64_t seed, uint64_t offset, const slapo_dropout_plan* plan,
    void* stream) {
    if (!x || !gamma || !beta || !y) return SLAPO_ERR_ARG;
    if (!dims_ok(rows, cols)) return SLAPO_ERR_SHAPE;
    if (!(p >= 0.0 && p <= 1.0) || !(eps >= 0.0)) return SLAPO_ERR_ARG;
    const bool dropout = p > 0.0;
    DropoutState s = {};
    if (dropout) {
        if (!plan_ok(plan, rows * cols)) return SLAPO_ERR_ARG;
        s = make_dropout_state(*plan, p, seed, offset);
    }
    hipStream_t st = (hipStream_t)stream;
#define CALL(T)                                                                                \
    ln_fwd_dispatch<T>(x, bias, residual, gamma, beta, z, y, mean, rstd, rows, cols, (float)eps, \
                       dropout, s, st)
    SLAPO_DISPATCH_DTYPE(dtype, CALL)
#undef CALL
}

extern "C" int slapo_amd_bias_dropout_residual_ln_bwd(
    const void* grad_y, const void* z, const float* mean, const float* rstd, const void* gamma,
    void* dx, void* dresidual, void* dgamma, void* dbeta, void* dbias, void* workspace,
    size_t workspace_bytes, int64_t rows, int64_t cols, int dtype, double p, uint64_t seed,
    uint64_t offset, const slapo_dropout_plan* plan, void* stream) {
    if (!grad_y || !z || !mean || !rstd || !gamma) return SLAPO_ERR_ARG;
    if (!dx && !dresidual && !dgamma && !dbeta && !dbias) return SLAPO_ERR_ARG;
    if (!dims_ok(rows, cols)) return SLAPO_ERR_SHAPE;
    if (!(p >= 0.0 && p <= 1.0)) return SLAPO_ERR_ARG;
    if ((dgamma || dbeta || dbias) &&
        (!workspace || workspace_bytes < slapo_amd_ln_bwd_workspace_bytes(rows, cols)))
        return SLAPO_ERR_WORKSPACE;
    const bool dropout = p > 0.0;
    DropoutState s = {};
    if (dropout) {
        if (!plan_ok(plan, rows * cols)) return SLAPO_ERR_ARG;
        s = make_dropout_state(*plan, p, seed, offset);
    }
    hipStream_t st = (hipStream_t)stream;
#define CALL(T)                                                                               \
    ln_bwd_dispatch<T>(grad_y, z, mean, rstd, gamma, dx, dresidual, dgamma, dbeta, dbias,    \
                       workspace, rows, cols, dropout, s, st)
    SLAPO_DISPATCH_DTYPE(dtype, CALL)
#undef CALL
}
