// Row-wise building blocks: embedding rows into the fp32 residual stream, the weighted sum of residual streams fused with the
// RMS norms that read it, the polynomial-of-normalised-powers activation, the sigmoid top-k router and the bookkeeping of a
// mixture of experts (bucketing pairs by expert, summing the pairs' results back into the stream).  All reductions fp32.
#include <string.h>

#include "pb_common.h"

static thread_local char g_err[512] = "";

void pcb_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

PCB_EXPORT int pcb_version(void) { return PCB_ABI_VERSION; }
PCB_EXPORT const char* pcb_last_error_string(void) { return g_err; }

namespace {
using namespace pcb;

// block-wide sum of NV values per thread; every thread gets the totals.  red: [waves * NV]
template <int NV>
__device__ __forceinline__ void block_sum(float (&v)[NV], float* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = wave_sum(v[i]);
    __syncthreads();
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < NV; ++i) red[wave * NV + i] = v[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        float t = 0.0f;
        for (int w = 0; w < waves; ++w) t += red[w * NV + i];
        v[i] = t;
    }
}

template <typename E>
__global__ __launch_bounds__(256) void embed_rows_kernel(const E* __restrict__ table, const int32_t* __restrict__ ids,
                                                         float* __restrict__ out, int width, int vocab, float scale = 1.0f) {
    const int r = blockIdx.x;
    int id = ids[r];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const E* src = table + (int64_t)id * width;
    for (int c = threadIdx.x; c < width; c += 256) out[(int64_t)r * width + c] = scale * to_f32(src[c]);
}

// one workgroup per output row; the row is held in LDS between the sum and the norms (width * 4 bytes of dynamic LDS)
template <typename E>
__global__ __launch_bounds__(1024) void mix_norm_kernel(pcb_mix_norm_args a) {
    extern __shared__ float row[];
    __shared__ float red[16];
    const int r = blockIdx.x;
    const int64_t src = a.rows ? a.rows[r] : r;
    const int W = a.width;
    float ss[1] = {0.0f};
    // (streams and coefficients are read through restrict-qualified pointers: the stores to x_out must not fence the loads)
    const float* __restrict__ hist = a.hist + src * W;
    const float* __restrict__ coef = a.coef;
    float* __restrict__ xo = a.x_out ? a.x_out + (int64_t)r * W : nullptr;
    const int nt = a.n_terms;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float x = nt > 0 ? 0.0f : hist[c];
        for (int j = 0; j < nt; ++j) x += coef[j] * hist[j * a.hist_stride + c];
        row[c] = x;
        if (xo) xo[c] = x;
        ss[0] += x * x;
    }
    block_sum<1>(ss, red);
    const float inv = 1.0f / sqrtf(ss[0] / (float)W + a.eps);
    E* o1 = (E*)a.out1;
    E* o2 = (E*)a.out2;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float x = row[c] * inv;
        if (o1) o1[(int64_t)r * W + c] = from_f32<E>(x * a.gain1[c]);
        if (o2) o2[(int64_t)r * W + c] = from_f32<E>(x * a.gain2[c]);
    }
}

template <typename E>
__global__ __launch_bounds__(1024) void polynorm_kernel(const float* __restrict__ z, const float* __restrict__ coef, E* __restrict__ out,
                                                       float eps, int ff) {
    __shared__ float red[48];
    const int64_t r = blockIdx.x;
    const float* zr = z + r * ff;
    float s[3] = {0.0f, 0.0f, 0.0f};
    for (int c = threadIdx.x; c < ff; c += blockDim.x) {
        const float v = zr[c], v2 = v * v, v3 = v2 * v;
        s[0] += v2;
        s[1] += v2 * v2;
        s[2] += v3 * v3;
    }
    block_sum<3>(s, red);
    const float i1 = coef[0] / sqrtf(s[0] / (float)ff + eps);
    const float i2 = coef[1] / sqrtf(s[1] / (float)ff + eps);
    const float i3 = coef[2] / sqrtf(s[2] / (float)ff + eps);
    const float c3 = coef[3];
    for (int c = threadIdx.x; c < ff; c += blockDim.x) {
        const float v = zr[c], v2 = v * v;
        out[r * ff + c] = from_f32<E>(i1 * v + i2 * v2 + i3 * (v2 * v) + c3);
    }
}

// one wave per row of router logits: sigmoid scores in LDS, `top` rounds of a wave-wide arg-max
__global__ __launch_bounds__(256) void router_topk_kernel(const float* __restrict__ logits, int n_rows, int n_experts, int top,
                                                          int32_t* __restrict__ expert, float* __restrict__ weight) {
    extern __shared__ float sc[];          // [4][n_experts]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = blockIdx.x * 4 + wave;
    if (r >= n_rows) return;
    float* s = sc + wave * n_experts;
    for (int e = lane; e < n_experts; e += 64) s[e] = 1.0f / (1.0f + expf(-logits[(int64_t)r * n_experts + e]));
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int k = 0; k < top; ++k) {
        float best = -1.0f;
        int bi = 0x7fffffff;
        for (int e = lane; e < n_experts; e += 64) {
            const float v = s[e];
            if (v > best) best = v, bi = e;        // ascending e: the first of equal scores stays
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ov > best || (ov == best && oi < bi)) best = ov, bi = oi;
        }
        if (lane == 0) {
            expert[(int64_t)r * top + k] = bi;
            weight[(int64_t)r * top + k] = best;
            s[bi] = -2.0f;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

__global__ __launch_bounds__(1024) void moe_plan_kernel(const int32_t* __restrict__ expert, const float* __restrict__ weight, int n_pairs,
                                                        int top, int n_experts, int32_t* __restrict__ group_off,
                                                        int32_t* __restrict__ row_src, int32_t* __restrict__ row_dst,
                                                        float* __restrict__ row_scale) {
    extern __shared__ int cnt[];           // [n_experts] counts, then [n_experts] cursors
    int* cur = cnt + n_experts;
    for (int e = threadIdx.x; e < n_experts; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += 1024) atomicAdd(&cnt[expert[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int off = 0;
        for (int e = 0; e < n_experts; ++e) {
            group_off[e] = off;
            cur[e] = off;
            off += cnt[e];
        }
        group_off[n_experts] = off;
    }
    __syncthreads();
    // (which row of its bucket a pair lands in does not enter any result: rows of a bucket are independent)
    for (int p = threadIdx.x; p < n_pairs; p += 1024) {
        const int at = atomicAdd(&cur[expert[p]], 1);
        row_src[at] = p / top;
        row_dst[at] = p;
        row_scale[at] = weight[p];
    }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ pair_out, const float* __restrict__ col_scale,
                                                          float* __restrict__ y, int width, int top) {
    const int64_t r = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += 256) {
        float s = 0.0f;
        for (int k = 0; k < top; ++k) s += pair_out[(r * top + k) * width + c];
        y[r * width + c] += col_scale[c] * s;
    }
}

}  // namespace

#define PCB_DTYPE_OK(d) ((d) == PCB_BF16 || (d) == PCB_F32)

PCB_EXPORT int pcb_embed_rows(const void* table, int32_t dtype, const int32_t* ids, float* out, int32_t n_rows, int32_t width,
                              int32_t vocab, void* stream) {
    PCB_REQUIRE(PCB_DTYPE_OK(dtype) && n_rows >= 0 && width > 0 && vocab > 0, PCB_ERR_ARG, "pcb_embed_rows: bad sizes");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(table && ids && out, PCB_ERR_ARG, "pcb_embed_rows: null pointer");
    if (dtype == PCB_BF16)
        hipLaunchKernelGGL(embed_rows_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)table, ids, out,
                           width, vocab, 1.0f);
    else
        hipLaunchKernelGGL(embed_rows_kernel<float>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, (const float*)table, ids, out,
                           width, vocab, 1.0f);
    return pcb_check_launch("embed_rows_kernel");
}

PCB_EXPORT int pcb_embed_scaled_rows(const void* table, int32_t dtype, const int32_t* ids, float scale, float* out, int32_t n_rows,
                                     int32_t width, int32_t vocab, void* stream) {
    PCB_REQUIRE(PCB_DTYPE_OK(dtype) && n_rows >= 0 && width > 0 && vocab > 0, PCB_ERR_ARG, "pcb_embed_scaled_rows: bad sizes");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(table && ids && out, PCB_ERR_ARG, "pcb_embed_scaled_rows: null pointer");
    if (dtype == PCB_BF16)
        hipLaunchKernelGGL(embed_rows_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)table, ids, out,
                           width, vocab, scale);
    else
        hipLaunchKernelGGL(embed_rows_kernel<float>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, (const float*)table, ids, out,
                           width, vocab, scale);
    return pcb_check_launch("embed_rows_kernel");
}

PCB_EXPORT int pcb_mix_norm(const pcb_mix_norm_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_mix_norm_args), PCB_ERR_ARG, "pcb_mix_norm: struct size mismatch");
    PCB_REQUIRE(PCB_DTYPE_OK(a->dtype) && a->n_rows >= 0 && a->width > 0 && a->width <= 16384 && a->n_terms >= 0, PCB_ERR_ARG,
                "pcb_mix_norm: bad sizes (width <= 16384)");
    if (a->n_rows == 0) return PCB_OK;
    PCB_REQUIRE(a->hist && (a->n_terms == 0 || a->coef) && (!a->out1 || a->gain1) && (!a->out2 || a->gain2), PCB_ERR_ARG,
                "pcb_mix_norm: null pointer");
    const size_t lds = (size_t)a->width * sizeof(float);
    // few rows: a row's columns are spread over up to 1024 threads (the loads of a thread's columns are a dependent chain)
    const dim3 threads(a->n_rows <= 512 && a->width > 1024 ? 1024 : 256);
    if (a->dtype == PCB_BF16)
        hipLaunchKernelGGL(mix_norm_kernel<bf16_t>, dim3(a->n_rows), threads, lds, (hipStream_t)stream, *a);
    else
        hipLaunchKernelGGL(mix_norm_kernel<float>, dim3(a->n_rows), threads, lds, (hipStream_t)stream, *a);
    return pcb_check_launch("mix_norm_kernel");
}

PCB_EXPORT int pcb_polynorm(const float* z, const float* coef, void* out, int32_t dtype, float eps, int32_t n_rows, int32_t ff,
                            void* stream) {
    PCB_REQUIRE(PCB_DTYPE_OK(dtype) && n_rows >= 0 && ff > 0, PCB_ERR_ARG, "pcb_polynorm: bad sizes");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(z && coef && out, PCB_ERR_ARG, "pcb_polynorm: null pointer");
    const dim3 threads(n_rows <= 512 && ff > 1024 ? 1024 : 256);
    if (dtype == PCB_BF16)
        hipLaunchKernelGGL(polynorm_kernel<bf16_t>, dim3(n_rows), threads, 0, (hipStream_t)stream, z, coef, (bf16_t*)out, eps, ff);
    else
        hipLaunchKernelGGL(polynorm_kernel<float>, dim3(n_rows), threads, 0, (hipStream_t)stream, z, coef, (float*)out, eps, ff);
    return pcb_check_launch("polynorm_kernel");
}

PCB_EXPORT int pcb_router_topk(const float* logits, int32_t n_rows, int32_t n_experts, int32_t top, int32_t* expert, float* weight,
                               void* stream) {
    PCB_REQUIRE(n_rows >= 0 && n_experts > 0 && n_experts <= 2048 && top > 0 && top <= n_experts, PCB_ERR_ARG,
                "pcb_router_topk: bad sizes (1 <= top <= n_experts <= 2048)");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(logits && expert && weight, PCB_ERR_ARG, "pcb_router_topk: null pointer");
    hipLaunchKernelGGL(router_topk_kernel, dim3(pcb_ceil_div(n_rows, 4)), dim3(256), (size_t)4 * n_experts * sizeof(float),
                       (hipStream_t)stream, logits, n_rows, n_experts, top, expert, weight);
    return pcb_check_launch("router_topk_kernel");
}

PCB_EXPORT int pcb_moe_plan(const int32_t* expert, const float* weight, int32_t n_pairs, int32_t top, int32_t n_experts,
                            int32_t* group_off, int32_t* row_src, int32_t* row_dst, float* row_scale, void* stream) {
    PCB_REQUIRE(n_pairs >= 0 && n_pairs <= (1 << 20) && top > 0 && n_experts > 0 && n_experts <= 2048, PCB_ERR_ARG,
                "pcb_moe_plan: bad sizes");
    PCB_REQUIRE(expert && weight && group_off && row_src && row_dst && row_scale, PCB_ERR_ARG, "pcb_moe_plan: null pointer");
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), (size_t)2 * n_experts * sizeof(int), (hipStream_t)stream, expert, weight,
                       n_pairs, top, n_experts, group_off, row_src, row_dst, row_scale);
    return pcb_check_launch("moe_plan_kernel");
}

PCB_EXPORT int pcb_moe_combine(const float* pair_out, const float* col_scale, float* y, int32_t n_rows, int32_t width, int32_t top,
                               void* stream) {
    PCB_REQUIRE(n_rows >= 0 && width > 0 && top > 0, PCB_ERR_ARG, "pcb_moe_combine: bad sizes");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(pair_out && col_scale && y, PCB_ERR_ARG, "pcb_moe_combine: null pointer");
    hipLaunchKernelGGL(moe_combine_kernel, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, pair_out, col_scale, y, width, top);
    return pcb_check_launch("moe_combine_kernel");
}

// ---- several residual streams: embedding with positions, hyper-connection steps with their norms, gated unit norm ----------------
namespace {
using namespace pcb;

template <typename E>
__global__ __launch_bounds__(256) void embed_pos_rows_kernel(const E* __restrict__ table, const E* __restrict__ pos_table,
                                                             const int32_t* __restrict__ ids, const int32_t* __restrict__ positions,
                                                             float* __restrict__ out, int64_t stream_stride, int n_streams, int width,
                                                             int vocab, int max_positions) {
    const int r = blockIdx.x;
    int id = ids[r];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const E* src = table + (int64_t)id * width;
    const E* ps = nullptr;
    if (pos_table) {
        int p = positions[r];
        p = p < 0 ? 0 : (p >= max_positions ? max_positions - 1 : p);
        ps = pos_table + (int64_t)p * width;
    }
    for (int c = threadIdx.x; c < width; c += 256) {
        const float v = to_f32(src[c]) + (ps ? to_f32(ps[c]) : 0.0f);
        for (int s = 0; s < n_streams; ++s) out[s * stream_stride + (int64_t)r * width + c] = v;
    }
}

constexpr int MAX_STREAMS = 8;

template <typename E>
__global__ __launch_bounds__(1024) void hyper_norm_kernel(pcb_hyper_norm_args a) {
    extern __shared__ float row[];          // RMS only: the row between the sum and the norm
    __shared__ float red[16];
    __shared__ float coef[MAX_STREAMS * MAX_STREAMS + 2 * MAX_STREAMS];
    const int r = blockIdx.x, S = a.n_streams, W = a.width;
    const int64_t src = a.rows ? a.rows[r] : r;
    float* mixw = coef;
    float* outw = coef + MAX_STREAMS * MAX_STREAMS;
    float* inw = outw + MAX_STREAMS;
    if (threadIdx.x < S * S) mixw[threadIdx.x] = a.y ? a.mix[threadIdx.x] : 0.0f;
    if (threadIdx.x < S) {
        outw[threadIdx.x] = a.y ? a.out_w[threadIdx.x] : 0.0f;
        inw[threadIdx.x] = a.in_w ? a.in_w[threadIdx.x] : 1.0f;
    }
    __syncthreads();
    const bool reads = a.out != nullptr || a.x_out != nullptr;
    const float alpha = a.norm == PCB_NORM_DYT ? a.alpha[0] : 0.0f;
    float ss[1] = {0.0f};
    E* o = (E*)a.out;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float x[MAX_STREAMS];
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s) x[s] = s < S ? a.streams[s * a.stream_stride + src * W + c] : 0.0f;
        if (a.y) {
            const float yv = a.y[src * W + c];
            float nx[MAX_STREAMS];
#pragma unroll
            for (int t = 0; t < MAX_STREAMS; ++t) {
                float v = 0.0f;
#pragma unroll
                for (int s = 0; s < MAX_STREAMS; ++s)
                    if (s < S && t < S) v += mixw[s * S + t] * x[s];
                nx[t] = v + (t < S ? outw[t] : 0.0f) * yv;
            }
#pragma unroll
            for (int t = 0; t < MAX_STREAMS; ++t) {
                x[t] = nx[t];
                if (t < S && !a.rows) a.streams[t * a.stream_stride + src * W + c] = nx[t];
            }
        }
        if (!reads) continue;
        float u = 0.0f;
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s)
            if (s < S) u += inw[s] * x[s];
        if (a.x_out) a.x_out[(int64_t)r * W + c] = u;
        if (!o) continue;
        if (a.norm == PCB_NORM_RMS) {
            row[c] = u;
            ss[0] += u * u;
        } else if (a.norm == PCB_NORM_DYT) {
            o[(int64_t)r * W + c] = from_f32<E>(tanhf(alpha * u) * a.gain[c] + (a.bias ? a.bias[c] : 0.0f));
        } else {
            o[(int64_t)r * W + c] = from_f32<E>(u);
        }
    }
    if (o && a.norm == PCB_NORM_RMS) {
        block_sum<1>(ss, red);
        const float inv = 1.0f / sqrtf(ss[0] / (float)W + a.eps);
        for (int c = threadIdx.x; c < W; c += blockDim.x) o[(int64_t)r * W + c] = from_f32<E>(row[c] * inv * a.gain[c]);
    }
}

template <typename E>
__global__ __launch_bounds__(256) void gated_norm_kernel(const float* __restrict__ x, int64_t ldx, const float* __restrict__ gain,
                                                         const E* __restrict__ gate, int64_t ldg, E* __restrict__ out, int64_t ldo,
                                                         float eps, int cols) {
    __shared__ float red[16];
    const int64_t r = blockIdx.x;
    float ss[1] = {0.0f};
    float inv = 1.0f;
    if (gain) {
        for (int c = threadIdx.x; c < cols; c += 256) {
            const float v = x[r * ldx + c];
            ss[0] += v * v;
        }
        block_sum<1>(ss, red);
        inv = 1.0f / sqrtf(ss[0] / (float)cols + eps);
    }
    for (int c = threadIdx.x; c < cols; c += 256) {
        float v = x[r * ldx + c];
        if (gain) v = v * inv * gain[c];
        if (gate) v *= to_f32(gate[r * ldg + c]);
        out[r * ldo + c] = from_f32<E>(v);
    }
}

// the same with a norm per run of `group` columns (a head): one wave per (row, group) pair, four pairs per workgroup -- or, WIDE, a
// whole workgroup per pair (groups of hundreds of columns, where one wave's chain of dependent loads would be the launch's length).
// A skip path (x + skip_w[c / skip_group] * skip) and a gate that comes before the norm are this kernel's alone.
template <typename E, bool WIDE>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ x, int64_t ldx, const float* __restrict__ gain,
                                                               const E* __restrict__ gate, int64_t ldg, E* __restrict__ out, int64_t ldo,
                                                               float eps, int cols, int group, int64_t n_pairs, int gate_first,
                                                               const E* __restrict__ skip, int64_t lds, const float* __restrict__ skip_w,
                                                               int skip_group) {
    __shared__ float red[16];
    constexpr int TPP = WIDE ? 256 : 64;                   // threads per pair
    const int lane = WIDE ? (int)threadIdx.x : (int)(threadIdx.x & 63);
    const int64_t pair = WIDE ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (pair >= n_pairs) return;
    const int per = cols / group;
    const int64_t r = pair / per;
    const int c0 = (int)(pair % per) * group;
    auto value = [&](int c) {                              // what is normed: x (+ the skip path) (* the gate, when it comes first)
        float v = x[r * ldx + c];
        if (skip) v += skip_w[c / skip_group] * to_f32(skip[r * lds + c]);
        if (gate_first && gate) v *= to_f32(gate[r * ldg + c]);
        return v;
    };
    float ss[1] = {0.0f};
    for (int c = lane; c < group; c += TPP) {
        const float v = value(c0 + c);
        ss[0] += v * v;
    }
    if (WIDE)
        block_sum<1>(ss, red);
    else
        ss[0] = wave_sum(ss[0]);
    const float inv = 1.0f / sqrtf(ss[0] / (float)group + eps);
    for (int c = lane; c < group; c += TPP) {
        float v = value(c0 + c) * inv;
        if (gain) v *= gain[c0 + c];
        if (gate && !gate_first) v *= to_f32(gate[r * ldg + c0 + c]);
        out[r * ldo + c0 + c] = from_f32<E>(v);
    }
}

// one workgroup per row; the row waits in LDS between the two sums (width * 4 bytes of dynamic LDS)
template <typename E>
__global__ __launch_bounds__(1024) void post_norm_kernel(pcb_post_norm_args a) {
    extern __shared__ float row[];
    __shared__ float red[16];
    const int r = blockIdx.x, W = a.width;
    const int64_t src = a.rows ? a.rows[r] : r;
    float* __restrict__ x = a.x + src * W;
    float ss[1] = {0.0f};
    if (a.y) {
        const float* __restrict__ y = a.y + src * W;
        const E* __restrict__ g = a.gate ? (const E*)a.gate + src * a.ldg : nullptr;
        for (int c = threadIdx.x; c < W; c += blockDim.x) {
            const float t = y[c] * (g ? to_f32(g[c]) : 1.0f);
            row[c] = t;
            ss[0] += t * t;
        }
        float inv = 1.0f;
        if (a.post_gain) {
            block_sum<1>(ss, red);
            inv = 1.0f / sqrtf(ss[0] / (float)W + a.eps);
        }
        ss[0] = 0.0f;
        const float ys = a.y_scale;
        for (int c = threadIdx.x; c < W; c += blockDim.x) {          // (a thread meets its own columns again: no barrier needed)
            const float v = x[c] + ys * (a.post_gain ? row[c] * inv * a.post_gain[c] : row[c]);
            row[c] = v;
            if (!a.rows) x[c] = v;
            ss[0] += v * v;
        }
    } else {
        for (int c = threadIdx.x; c < W; c += blockDim.x) {
            const float v = x[c];
            row[c] = v;
            ss[0] += v * v;
        }
    }
    if (a.x_out)
        for (int c = threadIdx.x; c < W; c += blockDim.x) a.x_out[(int64_t)r * W + c] = row[c];
    if (!a.out) return;
    E* o = (E*)a.out + (int64_t)r * W;
    if (a.layer_norm) {
        // mean first, then the mean of the squared deviations (the row waits in LDS; a thread meets its own columns again)
        float sm[1] = {0.0f};
        for (int c = threadIdx.x; c < W; c += blockDim.x) sm[0] += row[c];
        block_sum<1>(sm, red);
        const float mean = sm[0] / (float)W;
        float sv[1] = {0.0f};
        for (int c = threadIdx.x; c < W; c += blockDim.x) {
            const float d = row[c] - mean;
            sv[0] += d * d;
        }
        block_sum<1>(sv, red);
        const float inv = 1.0f / sqrtf(sv[0] / (float)W + a.eps);
        for (int c = threadIdx.x; c < W; c += blockDim.x)
            o[c] = from_f32<E>((row[c] - mean) * inv * a.gain[c] + (a.bias ? a.bias[c] : 0.0f));
        return;
    }
    block_sum<1>(ss, red);
    const float inv = 1.0f / sqrtf(ss[0] / (float)W + a.eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x) o[c] = from_f32<E>(row[c] * inv * a.gain[c]);
}

// one wave per row: scores and choice scores in LDS, group maxima by lanes, then rounds of a wave-wide arg-max
__global__ __launch_bounds__(256) void router_select_kernel(const float* __restrict__ logits, int n_rows, int n_out, int top, int score_fn,
                                                            const float* __restrict__ correction, int groups, int keep, int renorm,
                                                            int32_t* __restrict__ expert, float* __restrict__ weight) {
    extern __shared__ float sc[];          // per wave: [n_out] scores, [n_out] choice scores, [64] group scores
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = blockIdx.x * 4 + wave;
    if (r >= n_rows) return;
    float* s = sc + wave * (2 * n_out + 64);
    float* ch = s + n_out;
    float* gs = ch + n_out;
    const float* z = logits + (int64_t)r * n_out;
    const float NEG = -__builtin_inff();
    auto sync = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    if (score_fn == PCB_SCORE_SOFTMAX) {
        float m = NEG;
        for (int e = lane; e < n_out; e += 64) m = fmaxf(m, z[e]);
        m = wave_max(m);
        float sum = 0.0f;
        for (int e = lane; e < n_out; e += 64) {
            const float v = expf(z[e] - m);
            s[e] = v;
            sum += v;
        }
        sum = wave_sum(sum);
        for (int e = lane; e < n_out; e += 64) s[e] = s[e] / sum;
    } else {
        for (int e = lane; e < n_out; e += 64) s[e] = 1.0f / (1.0f + expf(-z[e]));
    }
    for (int e = lane; e < n_out; e += 64) ch[e] = s[e] + (correction ? correction[e] : 0.0f);
    sync();
    if (groups > 1) {
        const int per = n_out / groups;
        if (lane < groups) {
            float b = NEG;
            for (int e = lane * per; e < (lane + 1) * per; ++e) b = fmaxf(b, ch[e]);
            gs[lane] = b;
        }
        sync();
        // the `keep` best groups stay; the others' choice scores become minus infinity
        float mine = lane < groups ? gs[lane] : NEG;
        bool kept = false;
        for (int k = 0; k < keep; ++k) {
            float best = (lane < groups && !kept) ? mine : NEG;
            int bi = (lane < groups && !kept) ? lane : 0x7fffffff;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float ov = __shfl_xor(best, o, 64);
                const int oi = __shfl_xor(bi, o, 64);
                if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) best = ov, bi = oi;
            }
            if (lane == bi) kept = true;
        }
        if (lane < groups && !kept)
            for (int e = lane * per; e < (lane + 1) * per; ++e) ch[e] = NEG;
        sync();
    }
    float wsum = 0.0f;
    for (int k = 0; k < top; ++k) {
        float best = NEG;
        int bi = 0x7fffffff;
        for (int e = lane; e < n_out; e += 64) {
            const float v = ch[e];
            if (v != v) continue;                   // (a taken output is marked with a NaN)
            if (bi == 0x7fffffff || v > best) best = v, bi = e;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) best = ov, bi = oi;
        }
        const float w = s[bi];
        wsum += w;
        if (lane == 0) {
            expert[(int64_t)r * top + k] = bi;
            weight[(int64_t)r * top + k] = w;
            ch[bi] = __builtin_nanf("");
        }
        sync();
    }
    if (renorm && lane < top) weight[(int64_t)r * top + lane] = weight[(int64_t)r * top + lane] / (wsum + 1e-20f);
}

template <typename E>
__global__ __launch_bounds__(256) void moe_mix_kernel(const float* __restrict__ pair_out, const int32_t* __restrict__ expert,
                                                      const float* __restrict__ weight, const E* __restrict__ h, int n_real,
                                                      float* __restrict__ y, int width, int top) {
    const int64_t r = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += 256) {
        float s = 0.0f;
        for (int k = 0; k < top; ++k) {
            const int64_t p = r * top + k;
            const float v = expert[p] >= n_real ? to_f32(h[r * width + c]) : pair_out[p * width + c];
            s += weight[p] * v;
        }
        y[r * width + c] = s;
    }
}

}  // namespace

PCB_EXPORT int pcb_embed_pos_rows(const void* table, const void* pos_table, int32_t dtype, const int32_t* ids, const int32_t* positions,
                                  float* out, int64_t stream_stride, int32_t n_streams, int32_t n_rows, int32_t width, int32_t vocab,
                                  int32_t max_positions, void* stream) {
    PCB_REQUIRE(PCB_DTYPE_OK(dtype) && n_rows >= 0 && width > 0 && vocab > 0 && n_streams >= 1, PCB_ERR_ARG, "pcb_embed_pos_rows: bad sizes");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(table && ids && out && (!pos_table || (positions && max_positions > 0)), PCB_ERR_ARG, "pcb_embed_pos_rows: null pointer");
    PCB_REQUIRE(n_streams == 1 || stream_stride >= (int64_t)n_rows * width, PCB_ERR_ARG, "pcb_embed_pos_rows: streams overlap");
    if (dtype == PCB_BF16)
        hipLaunchKernelGGL(embed_pos_rows_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)table,
                           (const bf16_t*)pos_table, ids, positions, out, stream_stride, n_streams, width, vocab, max_positions);
    else
        hipLaunchKernelGGL(embed_pos_rows_kernel<float>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, (const float*)table,
                           (const float*)pos_table, ids, positions, out, stream_stride, n_streams, width, vocab, max_positions);
    return pcb_check_launch("embed_pos_rows_kernel");
}

PCB_EXPORT int pcb_hyper_norm(const pcb_hyper_norm_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_hyper_norm_args), PCB_ERR_ARG, "pcb_hyper_norm: struct size mismatch");
    PCB_REQUIRE(PCB_DTYPE_OK(a->dtype) && a->n_rows >= 0 && a->width > 0 && a->n_streams >= 1 && a->n_streams <= MAX_STREAMS,
                PCB_ERR_ARG, "pcb_hyper_norm: bad sizes (1 <= streams <= 8)");
    PCB_REQUIRE(a->norm >= PCB_NORM_NONE && a->norm <= PCB_NORM_DYT, PCB_ERR_ARG, "pcb_hyper_norm: unknown norm");
    if (a->n_rows == 0) return PCB_OK;
    PCB_REQUIRE(a->streams && (!a->y || (a->mix && a->out_w)), PCB_ERR_ARG, "pcb_hyper_norm: null pointer");
    PCB_REQUIRE(!a->out || a->norm == PCB_NORM_NONE || (a->gain && (a->norm != PCB_NORM_DYT || a->alpha)), PCB_ERR_ARG,
                "pcb_hyper_norm: the norm needs its gain (and alpha)");
    PCB_REQUIRE(a->norm != PCB_NORM_RMS || a->width <= 16384, PCB_ERR_ARG, "pcb_hyper_norm: width <= 16384 with the RMS norm");
    const size_t lds = a->norm == PCB_NORM_RMS && a->out ? (size_t)a->width * sizeof(float) : 0;
    // few rows: a row's columns are spread over up to 1024 threads (the loads of a thread's columns are a dependent chain)
    const dim3 threads(a->n_rows <= 512 && a->width > 1024 ? 1024 : 256);
    if (a->dtype == PCB_BF16)
        hipLaunchKernelGGL(hyper_norm_kernel<bf16_t>, dim3(a->n_rows), threads, lds, (hipStream_t)stream, *a);
    else
        hipLaunchKernelGGL(hyper_norm_kernel<float>, dim3(a->n_rows), threads, lds, (hipStream_t)stream, *a);
    return pcb_check_launch("hyper_norm_kernel");
}

PCB_EXPORT int pcb_gated_norm(const float* x, int64_t ldx, const float* gain, const void* gate, int64_t ldg, void* out, int64_t ldo,
                              int32_t dtype, float eps, int32_t n_rows, int32_t cols, int32_t group_cols, int32_t gate_first,
                              const void* skip, int64_t lds, const float* skip_w, int32_t skip_group, void* stream) {
    PCB_REQUIRE(PCB_DTYPE_OK(dtype) && n_rows >= 0 && cols > 0 && ldx >= cols && ldo >= cols && (!gate || ldg >= cols), PCB_ERR_ARG,
                "pcb_gated_norm: bad sizes");
    PCB_REQUIRE(group_cols <= 0 || cols % group_cols == 0, PCB_ERR_ARG, "pcb_gated_norm: the groups must divide the columns");
    PCB_REQUIRE(!skip || (skip_w && lds >= cols && skip_group > 0 && cols % skip_group == 0), PCB_ERR_ARG,
                "pcb_gated_norm: a skip path needs its weights and a group size that divides the columns");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(x && out, PCB_ERR_ARG, "pcb_gated_norm: null pointer");
    if (gate_first || skip) group_cols = group_cols > 0 ? group_cols : cols;       // (the per-group kernel knows these two)
    if ((group_cols > 0 && group_cols < cols) || gate_first || skip) {
        const int64_t pairs = (int64_t)n_rows * (cols / group_cols);
        const bool wide = group_cols >= 512;
        const dim3 grid((unsigned)(wide ? pairs : (pairs + 3) / 4));
#define PCB_GGN(E_, WIDE_)                                                                                                                 \
    hipLaunchKernelGGL((gated_group_norm_kernel<E_, WIDE_>), grid, dim3(256), 0, (hipStream_t)stream, x, ldx, gain, (const E_*)gate, ldg, \
                       (E_*)out, ldo, eps, cols, group_cols, pairs, gate_first, (const E_*)skip, lds, skip_w, skip_group)
        if (dtype == PCB_BF16) {
            if (wide) PCB_GGN(bf16_t, true); else PCB_GGN(bf16_t, false);
        } else {
            if (wide) PCB_GGN(float, true); else PCB_GGN(float, false);
        }
#undef PCB_GGN
        return pcb_check_launch("gated_group_norm_kernel");
    }
    if (dtype == PCB_BF16)
        hipLaunchKernelGGL(gated_norm_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, x, ldx, gain, (const bf16_t*)gate,
                           ldg, (bf16_t*)out, ldo, eps, cols);
    else
        hipLaunchKernelGGL(gated_norm_kernel<float>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, x, ldx, gain, (const float*)gate, ldg,
                           (float*)out, ldo, eps, cols);
    return pcb_check_launch("gated_norm_kernel");
}

PCB_EXPORT int pcb_router_select(const float* logits, int32_t n_rows, int32_t n_out, int32_t top, int32_t score_fn,
                                 const float* correction, int32_t groups, int32_t groups_keep, int32_t renorm, int32_t* expert,
                                 float* weight, void* stream) {
    PCB_REQUIRE(n_rows >= 0 && n_out > 0 && n_out <= 2048 && top > 0 && top <= 64 && top <= n_out, PCB_ERR_ARG,
                "pcb_router_select: bad sizes (1 <= top <= 64, top <= n_out <= 2048)");
    PCB_REQUIRE(groups >= 1 && groups <= 64 && n_out % groups == 0 && groups_keep >= 1 && groups_keep <= groups &&
                    top <= n_out / groups * groups_keep,
                PCB_ERR_ARG, "pcb_router_select: bad groups (<= 64 equal groups, top within the kept ones)");
    PCB_REQUIRE(score_fn == PCB_SCORE_SIGMOID || score_fn == PCB_SCORE_SOFTMAX, PCB_ERR_ARG, "pcb_router_select: unknown score function");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(logits && expert && weight, PCB_ERR_ARG, "pcb_router_select: null pointer");
    hipLaunchKernelGGL(router_select_kernel, dim3(pcb_ceil_div(n_rows, 4)), dim3(256), (size_t)4 * (2 * n_out + 64) * sizeof(float),
                       (hipStream_t)stream, logits, n_rows, n_out, top, score_fn, correction, groups, groups_keep, renorm, expert, weight);
    return pcb_check_launch("router_select_kernel");
}

PCB_EXPORT int pcb_moe_mix(const float* pair_out, const int32_t* expert, const float* weight, const void* h, int32_t dtype, int32_t n_real,
                           float* y, int32_t n_rows, int32_t width, int32_t top, void* stream) {
    PCB_REQUIRE(PCB_DTYPE_OK(dtype) && n_rows >= 0 && width > 0 && top > 0 && n_real >= 0, PCB_ERR_ARG, "pcb_moe_mix: bad sizes");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(pair_out && expert && weight && h && y, PCB_ERR_ARG, "pcb_moe_mix: null pointer");
    if (dtype == PCB_BF16)
        hipLaunchKernelGGL(moe_mix_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, pair_out, expert, weight,
                           (const bf16_t*)h, n_real, y, width, top);
    else
        hipLaunchKernelGGL(moe_mix_kernel<float>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, pair_out, expert, weight,
                           (const float*)h, n_real, y, width, top);
    return pcb_check_launch("moe_mix_kernel");
}

PCB_EXPORT int pcb_post_norm(const pcb_post_norm_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_post_norm_args), PCB_ERR_ARG, "pcb_post_norm: struct size mismatch");
    PCB_REQUIRE(PCB_DTYPE_OK(a->dtype) && a->n_rows >= 0 && a->width > 0 && a->width <= 16384, PCB_ERR_ARG,
                "pcb_post_norm: bad sizes (width <= 16384)");
    if (a->n_rows == 0) return PCB_OK;
    PCB_REQUIRE(a->x && (!a->out || a->gain) && (!a->gate || (a->y && a->ldg >= a->width)) && (!a->post_gain || a->y), PCB_ERR_ARG,
                "pcb_post_norm: null pointer (a gate and a norm after the sublayer need its result, a norm its gain)");
    const size_t lds = (size_t)a->width * sizeof(float);
    const dim3 threads(a->n_rows <= 512 && a->width > 1024 ? 1024 : 256);
    if (a->dtype == PCB_BF16)
        hipLaunchKernelGGL(post_norm_kernel<bf16_t>, dim3(a->n_rows), threads, lds, (hipStream_t)stream, *a);
    else
        hipLaunchKernelGGL(post_norm_kernel<float>, dim3(a->n_rows), threads, lds, (hipStream_t)stream, *a);
    return pcb_check_launch("post_norm_kernel");
}
