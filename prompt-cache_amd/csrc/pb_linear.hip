// pcb_linear: Y = A W^T for row-major activations and nn.Linear-layout weights in bf16 or fp32, with what decoder layers fuse
// around a projection: bias, gathered and scaled input rows, per-group weights (experts), a gated-unit epilogue, and the
// layer-scaled accumulation into an fp32 residual stream.
//
// Tiling: workgroup = 4 waves in a 2 x 2 grid, a wave owns TM x TN result tiles of 16 x 16, so the workgroup covers
// (32 TM) x (32 TN) of Y.  Per stage of two 32-element k-steps the A and B panels go global -> registers -> LDS (the next stage's
// loads are in flight while this stage's MFMAs run); waves read their operand fragments from LDS with one 16-byte read per fragment (bf16).
#include "pb_common.h"

namespace {
using namespace pcb;

template <typename E>
struct Tile {
    static constexpr int KS = sizeof(E) == 2 ? 2 : 1;   // 32-element k-steps per LDS stage (fp32 panels are twice as large)
    static constexpr int CE = 16 / sizeof(E);       // elements per 16-byte chunk
    static constexpr int CPR = 32 * KS / CE;         // chunks per staged row
    static constexpr int LD = 32 * KS + CE;          // LDS row stride in elements (16-byte aligned rows, skewed banks)
};

__device__ __forceinline__ u32x4 zero_chunk() { return u32x4{0u, 0u, 0u, 0u}; }

// one 16-byte chunk of row `p` (null: a row outside the matrix) starting at k element k, K elements in the row
template <typename E>
__device__ __forceinline__ u32x4 load_chunk(const E* p, int k, int K, bool vec, float scale, bool scaled) {
    constexpr int CE = Tile<E>::CE;
    u32x4 c = zero_chunk();
    if (p == nullptr || k >= K) return c;
    if (vec) {
        c = *reinterpret_cast<const u32x4*>(p + k);
    } else {
        __attribute__((aligned(16))) E tmp[CE];
#pragma unroll
        for (int e = 0; e < CE; ++e) tmp[e] = k + e < K ? p[k + e] : from_f32<E>(0.0f);
        c = *reinterpret_cast<u32x4*>(tmp);
    }
    if (scaled) {
        __attribute__((aligned(16))) E tmp[CE];
        *reinterpret_cast<u32x4*>(tmp) = c;
#pragma unroll
        for (int e = 0; e < CE; ++e) tmp[e] = from_f32<E>(scale * to_f32(tmp[e]));
        c = *reinterpret_cast<u32x4*>(tmp);
    }
    return c;
}

__device__ __forceinline__ float apply_act(int act, float v, float param) {
    switch (act) {
        case PCB_ACT_SILU: return v / (1.0f + expf(-v));
        case PCB_ACT_SIGMOID: return 1.0f / (1.0f + expf(-v));
        case PCB_ACT_RELU2: return v > 0.0f ? v * v : 0.0f;
        case PCB_ACT_SOFTPLUS: return v > 20.0f ? v : log1pf(expf(v));
        case PCB_ACT_SOFTCAP: return param * tanhf(v / param);
        case PCB_ACT_RELU: return v > 0.0f ? v : 0.0f;
        case PCB_ACT_GELU_TANH: return 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
        case PCB_ACT_LOGSIGMOID: return param * (fminf(v, 0.0f) - log1pf(expf(-fabsf(v))));
        case PCB_ACT_SCALE: return param * v;
        default: return v;
    }
}

// one result element through the epilogue (see pcb_linear_args)
template <typename E, int EPI>
__device__ __forceinline__ void emit(const pcb_linear_args& a, int m, int n, float acc, float acc2, float bv, float cs, float bv2 = 0.0f) {
    float v = acc + bv;
    if (EPI == PCB_EPI_STORE && (a.act | a.act2) && !(a.split_n > 0 && n >= a.split_n) && !(a.split_n3 > 0 && n >= a.split_n3))
        // (the split-off parts are stored as they are)
        v = apply_act((a.act_split > 0 && n >= a.act_split) ? a.act2 : a.act, v, a.act_param);
    if (EPI == PCB_EPI_SILU_MUL) v = apply_act(a.act == PCB_ACT_NONE ? PCB_ACT_SILU : a.act, v, 0.0f) * (acc2 + bv2);
    if (EPI == PCB_EPI_SCALE_ADD) {
        float* y = (float*)a.y + (int64_t)m * a.ldy + n;
        const float b0 = a.base ? a.base[(int64_t)m * a.ldbase + n] : *y;
        *y = b0 + cs * v;
        return;
    }
    if (a.split_n3 > 0 && n >= a.split_n3) {
        ((E*)a.y3)[a.row_off3[m] + (int64_t)(n - a.split_n3) * a.col_stride3] = from_f32<E>(v);
        return;
    }
    if (a.split_n > 0 && n >= a.split_n) {
        const int c = n - a.split_n;
        E* y = (E*)a.y2 + a.row_off2[m] + (int64_t)(c / a.head_dim2) * a.head_stride2 + c % a.head_dim2;
        *y = from_f32<E>(v);
        return;
    }
    const int64_t at = (int64_t)(a.row_dst ? a.row_dst[m] : m) * a.ldy + n;
    if (a.out_f32)
        ((float*)a.y)[at] = v;
    else
        ((E*)a.y)[at] = from_f32<E>(v);
}

template <typename E, int EPI, int TM, int TN>
__global__ __launch_bounds__(256) void linear_kernel(pcb_linear_args a) {
    constexpr bool TWO = EPI == PCB_EPI_SILU_MUL;
    constexpr int BM = 32 * TM, BN = 32 * TN, BROWS = TWO ? 2 * BN : BN;
    constexpr int CE = Tile<E>::CE, CPR = Tile<E>::CPR, LD = Tile<E>::LD, KS = Tile<E>::KS;
    constexpr int A_CH = (BM * CPR + 255) / 256, B_CH = (BROWS * CPR + 255) / 256;
    __shared__ __attribute__((aligned(16))) E As[BM * LD];
    __shared__ __attribute__((aligned(16))) E Bs[BROWS * LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1, group = lane >> 4, l15 = lane & 15;
    const int K = a.K, N = a.N;

    // which rows: a plain launch tiles [0, M); a grouped launch walks the group offsets to find its group and tile
    int g = 0, m_lo, m_hi;
    if (a.n_groups > 0) {
        int t = blockIdx.y;
        m_lo = -1;
        for (g = 0; g < a.n_groups; ++g) {
            const int lo = a.group_off[g], hi = a.group_off[g + 1];
            const int nt = (hi - lo + BM - 1) / BM;
            if (t < nt) {
                m_lo = lo + t * BM;
                m_hi = hi;
                break;
            }
            t -= nt;
        }
        if (m_lo < 0) return;
    } else {
        m_lo = blockIdx.y * BM;
        m_hi = a.M;
        if (m_lo >= m_hi) return;
    }
    const int n_lo = blockIdx.x * BN;
    const E* W = (const E*)a.w + (int64_t)g * a.w_group_stride;
    const E* W2 = TWO ? (const E*)a.w2 + (int64_t)g * a.w_group_stride : nullptr;
    const E* X = (const E*)a.x;
    const bool vec = (K % CE == 0) && (a.ldx % CE == 0) && (a.ldw % CE == 0) && (((uintptr_t)X | (uintptr_t)W | (uintptr_t)W2) % 16 == 0);
    const bool scaled = a.row_scale != nullptr;

    // this thread's chunks of the two panels
    const E* a_row[A_CH];
    float a_scale[A_CH];
    int a_k[A_CH], a_at[A_CH];
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
        const int c = tid + 256 * i, r = c / CPR;
        a_k[i] = (c % CPR) * CE;
        a_at[i] = c < BM * CPR ? r * LD + a_k[i] : -1;
        const int m = m_lo + r;
        a_row[i] = nullptr;
        a_scale[i] = 1.0f;
        if (c < BM * CPR && m < m_hi) {
            a_row[i] = X + (int64_t)(a.row_src ? a.row_src[m] : m) * a.ldx;
            if (scaled) a_scale[i] = a.row_scale[m];
        }
    }
    const E* b_row[B_CH];
    int b_k[B_CH], b_at[B_CH];
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
        const int c = tid + 256 * i, r = c / CPR;
        b_k[i] = (c % CPR) * CE;
        b_at[i] = c < BROWS * CPR ? r * LD + b_k[i] : -1;
        const E* base = (TWO && r >= BN) ? W2 : W;
        const int n = n_lo + (TWO && r >= BN ? r - BN : r);
        b_row[i] = (c < BROWS * CPR && n < N) ? base + (int64_t)n * a.ldw : nullptr;
    }

    f4 acc[TM][TN], acc2[TWO ? TM : 1][TWO ? TN : 1];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};
            if (TWO) acc2[i][j] = f4{0.f, 0.f, 0.f, 0.f};
        }

    u32x4 ra[A_CH], rb[B_CH];
#pragma unroll
    for (int i = 0; i < A_CH; ++i) ra[i] = load_chunk<E>(a_row[i], a_k[i], K, vec, a_scale[i], scaled);
#pragma unroll
    for (int i = 0; i < B_CH; ++i) rb[i] = load_chunk<E>(b_row[i], b_k[i], K, vec, 1.0f, false);

    for (int k0 = 0; k0 < K; k0 += 32 * KS) {
        __syncthreads();                           // the previous stage's fragment reads are done
#pragma unroll
        for (int i = 0; i < A_CH; ++i)
            if (a_at[i] >= 0) *reinterpret_cast<u32x4*>(&As[a_at[i]]) = ra[i];
#pragma unroll
        for (int i = 0; i < B_CH; ++i)
            if (b_at[i] >= 0) *reinterpret_cast<u32x4*>(&Bs[b_at[i]]) = rb[i];
        __syncthreads();
        if (k0 + 32 * KS < K) {
#pragma unroll
            for (int i = 0; i < A_CH; ++i) ra[i] = load_chunk<E>(a_row[i], k0 + 32 * KS + a_k[i], K, vec, a_scale[i], scaled);
#pragma unroll
            for (int i = 0; i < B_CH; ++i) rb[i] = load_chunk<E>(b_row[i], k0 + 32 * KS + b_k[i], K, vec, 1.0f, false);
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            Frag<E> fa[TM];
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[i] = load_frag(&As[((wm * TM + i) * 16 + l15) * LD + 32 * ks], group, 32, true);
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const Frag<E> fb = load_frag(&Bs[((wn * TN + j) * 16 + l15) * LD + 32 * ks], group, 32, true);
#pragma unroll
                for (int i = 0; i < TM; ++i) acc[i][j] = mma(fa[i], fb, acc[i][j]);
                if (TWO) {
                    const Frag<E> fb2 = load_frag(&Bs[(BN + (wn * TN + j) * 16 + l15) * LD + 32 * ks], group, 32, true);
#pragma unroll
                    for (int i = 0; i < TM; ++i) acc2[i][j] = mma(fa[i], fb2, acc2[i][j]);
                }
            }
        }
    }

    const E* bias = (const E*)a.bias;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int n = n_lo + (wn * TN + j) * 16 + l15;
        if (n >= N) continue;
        const float bv = bias ? to_f32(bias[n]) : 0.0f;
        const float bv2 = (TWO && a.bias2) ? to_f32(((const E*)a.bias2)[n]) : 0.0f;
        const float cs = (EPI == PCB_EPI_SCALE_ADD) ? a.col_scale[n] : 0.0f;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m_lo + (wm * TM + i) * 16 + 4 * group + r;
                if (m < m_hi) emit<E, EPI>(a, m, n, acc[i][j][r], TWO ? acc2[i][j][r] : 0.0f, bv, cs, bv2);
            }
    }
}

// ---- few rows: the weights stream once, straight from memory into the matrix cores --------------------------------------------
// Workgroup = 16 result columns x up to 16 rows; its eight waves split the k range (k-step s goes to wave s % 8) and add their
// partial tiles through LDS.  No LDS staging: a lane's B fragment is 16 contiguous bytes of its weight row, its A fragment 16
// bytes of its activation row (a handful of rows that stay in cache).
template <typename E>
__device__ __forceinline__ void scale_frag(Frag<E>& f, float s);
template <>
__device__ __forceinline__ void scale_frag<bf16_t>(Frag<bf16_t>& f, float s) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t w = f.v[e];
        const uint32_t lo = bf16_bits(s * __uint_as_float(w << 16)), hi = bf16_bits(s * __uint_as_float(w & 0xffff0000u));
        f.v[e] = lo | (hi << 16);
    }
}
template <>
__device__ __forceinline__ void scale_frag<float>(Frag<float>& f, float s) {
#pragma unroll
    for (int e = 0; e < 8; ++e) f.v[e] *= s;
}

constexpr int SKW = 8;          // waves of a few-row workgroup

template <typename E, int EPI>
__global__ __launch_bounds__(64 * SKW) void linear_skinny_kernel(pcb_linear_args a) {
    constexpr bool TWO = EPI == PCB_EPI_SILU_MUL;
    constexpr int CE = Tile<E>::CE;
    __shared__ f4 red[TWO ? 2 : 1][SKW][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, group = lane >> 4, l15 = lane & 15;
    const int K = a.K, N = a.N;
    int g = 0, m_lo, m_hi;
    if (a.n_groups > 0) {
        int t = blockIdx.y;
        m_lo = -1;
        for (g = 0; g < a.n_groups; ++g) {
            const int lo = a.group_off[g], hi = a.group_off[g + 1];
            const int nt = (hi - lo + 15) / 16;
            if (t < nt) {
                m_lo = lo + t * 16;
                m_hi = hi;
                break;
            }
            t -= nt;
        }
        if (m_lo < 0) return;
    } else {
        m_lo = blockIdx.y * 16;
        m_hi = a.M;
        if (m_lo >= m_hi) return;
    }
    const int n_lo = blockIdx.x * 16;
    const E* W = (const E*)a.w + (int64_t)g * a.w_group_stride;
    const E* W2 = TWO ? (const E*)a.w2 + (int64_t)g * a.w_group_stride : nullptr;
    const E* X = (const E*)a.x;
    const bool vec = (K % CE == 0) && (a.ldx % CE == 0) && (a.ldw % CE == 0) && (((uintptr_t)X | (uintptr_t)W | (uintptr_t)W2) % 16 == 0);
    const int n_b = n_lo + l15, m_a = m_lo + l15;
    const bool b_ok = n_b < N, a_ok = m_a < m_hi;
    const E* wrow = W + (int64_t)(b_ok ? n_b : 0) * a.ldw;
    const E* wrow2 = TWO ? W2 + (int64_t)(b_ok ? n_b : 0) * a.ldw : nullptr;
    const E* xrow = X + (int64_t)(a_ok ? (a.row_src ? a.row_src[m_a] : m_a) : 0) * a.ldx;
    const bool scaled = a.row_scale != nullptr;
    const float xs = (scaled && a_ok) ? a.row_scale[m_a] : 1.0f;
    f4 acc = f4{0.f, 0.f, 0.f, 0.f}, acc2 = f4{0.f, 0.f, 0.f, 0.f};
    const int nsteps = (K + 31) / 32;
#pragma unroll 8
    for (int st = wave; st < nsteps; st += SKW) {
        const int k0 = 32 * st;
        Frag<E> fa = load_frag(xrow + k0, group, a_ok ? K - k0 : 0, vec);
        if (scaled) scale_frag<E>(fa, xs);
        const Frag<E> fb = load_frag(wrow + k0, group, b_ok ? K - k0 : 0, vec);
        acc = mma(fa, fb, acc);
        if (TWO) {
            const Frag<E> fb2 = load_frag(wrow2 + k0, group, b_ok ? K - k0 : 0, vec);
            acc2 = mma(fa, fb2, acc2);
        }
    }
    red[0][wave][lane] = acc;
    if (TWO) red[1][wave][lane] = acc2;
    __syncthreads();
    if (wave != 0) return;
    acc = red[0][0][lane];
    if (TWO) acc2 = red[1][0][lane];
#pragma unroll
    for (int w = 1; w < SKW; ++w) {
        acc += red[0][w][lane];
        if (TWO) acc2 += red[1][w][lane];
    }
    const int n = n_lo + l15;
    if (n >= N) return;
    const E* bias = (const E*)a.bias;
    const float bv = bias ? to_f32(bias[n]) : 0.0f;
    const float bv2 = (TWO && a.bias2) ? to_f32(((const E*)a.bias2)[n]) : 0.0f;
    const float cs = (EPI == PCB_EPI_SCALE_ADD) ? a.col_scale[n] : 0.0f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int m = m_lo + 4 * group + r;
        if (m < m_hi) emit<E, EPI>(a, m, n, acc[r], acc2[r], bv, cs, bv2);
    }
}

template <typename E, int EPI, int TM, int TN>
int launch(const pcb_linear_args& a, hipStream_t stream) {
    constexpr int BM = 32 * TM, BN = 32 * TN;
    const dim3 grid(pcb_ceil_div(a.N, BN), pcb_ceil_div(a.M, BM) + (a.n_groups > 0 ? a.n_groups : 0));
    hipLaunchKernelGGL((linear_kernel<E, EPI, TM, TN>), grid, dim3(256), 0, stream, a);
    return pcb_check_launch("linear_kernel");
}

template <typename E>
int dispatch(const pcb_linear_args& a, hipStream_t stream) {
    // rows per group decide the row tile: many rows -> 128-row panels, few -> 32-row panels (the weights stream once)
    const int rows = a.n_groups > 0 ? pcb_ceil_div(a.M, a.n_groups) : a.M;
    // (a narrow result -- router logits, step sizes: N <= 64 -- takes the 32-row panels too: 128-row panels would leave M / 128
    // workgroups on the chip, each walking all of K)
    const bool big = rows > 64 && a.N > 64;
    if (rows <= 16) {
        const dim3 grid(pcb_ceil_div(a.N, 16), pcb_ceil_div(a.M, 16) + (a.n_groups > 0 ? a.n_groups : 0));
        switch (a.epilogue) {
            case PCB_EPI_STORE:
                hipLaunchKernelGGL((linear_skinny_kernel<E, PCB_EPI_STORE>), grid, dim3(64 * SKW), 0, stream, a);
                break;
            case PCB_EPI_SILU_MUL:
                hipLaunchKernelGGL((linear_skinny_kernel<E, PCB_EPI_SILU_MUL>), grid, dim3(64 * SKW), 0, stream, a);
                break;
            default:
                hipLaunchKernelGGL((linear_skinny_kernel<E, PCB_EPI_SCALE_ADD>), grid, dim3(64 * SKW), 0, stream, a);
        }
        return pcb_check_launch("linear_skinny_kernel");
    }
    switch (a.epilogue) {
        case PCB_EPI_STORE:
            return big ? launch<E, PCB_EPI_STORE, 4, 4>(a, stream) : launch<E, PCB_EPI_STORE, 1, 2>(a, stream);
        case PCB_EPI_SILU_MUL:
            return big ? launch<E, PCB_EPI_SILU_MUL, 4, 2>(a, stream) : launch<E, PCB_EPI_SILU_MUL, 1, 1>(a, stream);
        default:
            return big ? launch<E, PCB_EPI_SCALE_ADD, 4, 4>(a, stream) : launch<E, PCB_EPI_SCALE_ADD, 1, 2>(a, stream);
    }
}

}  // namespace

PCB_EXPORT int pcb_linear(const pcb_linear_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_linear_args), PCB_ERR_ARG, "pcb_linear: struct size mismatch");
    PCB_REQUIRE(a->dtype == PCB_BF16 || a->dtype == PCB_F32, PCB_ERR_ARG, "pcb_linear: unknown dtype");
    PCB_REQUIRE(a->M >= 0 && a->N > 0 && a->K > 0 && a->ldx >= a->K && a->ldw >= a->K, PCB_ERR_ARG, "pcb_linear: bad sizes");
    PCB_REQUIRE(a->epilogue >= PCB_EPI_STORE && a->epilogue <= PCB_EPI_SCALE_ADD, PCB_ERR_ARG, "pcb_linear: unknown epilogue");
    PCB_REQUIRE(a->act >= PCB_ACT_NONE && a->act <= PCB_ACT_SCALE && a->act2 >= PCB_ACT_NONE && a->act2 <= PCB_ACT_SCALE &&
                    a->act_split >= 0 &&
                    ((a->act | a->act2) == 0 || a->epilogue == PCB_EPI_STORE ||
                     (a->epilogue == PCB_EPI_SILU_MUL && a->act2 == 0 &&
                      (a->act == PCB_ACT_SILU || a->act == PCB_ACT_RELU || a->act == PCB_ACT_GELU_TANH))),
                PCB_ERR_ARG, "pcb_linear: an activation goes with the plain store epilogue (the gated one takes silu, relu or gelu_tanh)");
    PCB_REQUIRE((a->act != PCB_ACT_SOFTCAP && a->act2 != PCB_ACT_SOFTCAP) || a->act_param > 0.0f, PCB_ERR_ARG,
                "pcb_linear: the soft cap must be positive");
    if (a->M == 0) return PCB_OK;
    PCB_REQUIRE(a->x && a->w && a->y, PCB_ERR_ARG, "pcb_linear: null pointer");
    PCB_REQUIRE(a->n_groups >= 0 && (a->n_groups == 0 || a->group_off), PCB_ERR_ARG, "pcb_linear: groups need their offsets");
    PCB_REQUIRE(a->epilogue != PCB_EPI_SILU_MUL || a->w2, PCB_ERR_ARG, "pcb_linear: the gated epilogue takes w2");
    PCB_REQUIRE(a->epilogue == PCB_EPI_SILU_MUL || !a->bias2, PCB_ERR_ARG, "pcb_linear: a second bias goes with the gated epilogue");
    PCB_REQUIRE(a->epilogue != PCB_EPI_SCALE_ADD || (a->col_scale && a->ldy >= a->N && !a->row_dst), PCB_ERR_ARG,
                "pcb_linear: scale-add needs col_scale and a plain fp32 destination");
    PCB_REQUIRE(a->split_n == 0 || (a->epilogue == PCB_EPI_STORE && a->split_n > 0 && a->split_n < a->N && a->y2 && a->row_off2 &&
                                    a->head_dim2 > 0 && a->ldy >= a->split_n),
                PCB_ERR_ARG, "pcb_linear: bad split destination");
    PCB_REQUIRE(a->split_n3 == 0 || (a->epilogue == PCB_EPI_STORE && a->split_n3 > a->split_n && a->split_n3 < a->N && a->y3 && a->row_off3 &&
                                     a->col_stride3 > 0 && (a->split_n > 0 || a->ldy >= a->split_n3)),
                PCB_ERR_ARG, "pcb_linear: bad column-wise destination");
    PCB_REQUIRE(a->split_n > 0 || a->split_n3 > 0 || a->epilogue == PCB_EPI_SCALE_ADD || a->ldy >= a->N, PCB_ERR_ARG, "pcb_linear: ldy < N");
    return a->dtype == PCB_BF16 ? dispatch<pcb::bf16_t>(*a, (hipStream_t)stream) : dispatch<float>(*a, (hipStream_t)stream);
}
