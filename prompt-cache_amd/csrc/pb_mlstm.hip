// pcb_mlstm: the matrix memory of an mLSTM layer, token by token.  Per (slot, head): S [dim][vdim], a normaliser n [dim] and a
// running maximum m of the log gates, all fp32 (see pcb_mlstm_args for the recurrence).
//
// One workgroup = one request x one head x 64 value columns.  Wave p of its four owns the key rows d = p DPT .. (p + 1) DPT - 1 and
// lane j the value column: a thread keeps its DPT entries S[d][j] in registers for the whole request, and the matching entries of
// n as well (every lane of a wave holds the same ones, which spares a broadcast per token).  Tokens arrive in blocks of TB: the
// whole block's q, k, v and gates are requested at once (one memory round trip per block, and the next block's while the current
// one is worked on), staged in LDS -- q scaled, the gates already through cap / logsigmoid --, and the block's tokens then run
// from LDS alone: every thread advances the running maximum by itself, updates its slice, leaves partial sums of S^T q and n . q
// in LDS (two alternating sets, so one barrier per token), and wave 0 adds the four parts and stores the output row.
//
// A long prompt is cut into segments that run side by side (pcb_mlstm_args.from_nothing, pcb_mlstm_chain): with the stabilised
// state (S, n, m) standing for the true sums exp(m) S and exp(m) n, a segment that starts from nothing (S = n = 0, m = -inf) leaves
// its own contribution (S', n', m') and the sum F of its log forget gates, and a state (S, n, m) carried over it becomes
//   m'' = max(F + m, m'),   S'' = exp(F + m - m'') S + exp(m' - m'') S',   n'' likewise
// which is what the token-by-token recurrence gives, since its running maximum unrolls to exactly that maximum.
#include "pb_common.h"

namespace {
using namespace pcb;

__device__ __forceinline__ float soft_cap(float z, float cap) { return cap > 0.0f ? cap * tanhf(z / cap) : z; }
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.0f) - log1pf(expf(-fabsf(z))); }

constexpr int TB = 8;          // tokens per staged block

// OUT false: only the states move (the first pass over segments) -- no products with q, no partial sums, no barrier per token
template <typename E, int DPT, bool OUT>
__global__ __launch_bounds__(256) void mlstm_kernel(pcb_mlstm_args a) {
    constexpr int DM = 4 * DPT;                 // key rows the workgroup can hold (>= dim)
    constexpr int QN = TB * DM / 256;           // q (and k) elements a thread fetches per block
    constexpr int VN = TB * 64 / 256;           // v elements a thread fetches per block
    __shared__ __attribute__((aligned(16))) float qs[2][TB][DM], ks[2][TB][DM];
    __shared__ float vs[2][TB][64], gs[2][TB][2];
    __shared__ float part_o[2][4][64], part_n[2][4];
    const int tid = threadIdx.x, lane = tid & 63, p = tid >> 6;
    const int32_t* rq = a.reqs + 4 * blockIdx.x;
    const int slot = rq[0], pos0 = rq[1], count = rq[2], row0 = rq[3];
    const int h = blockIdx.y, dim = a.dim, vdim = a.vdim;
    const int j0 = blockIdx.z * 64, j = j0 + lane;
    const bool col = j < vdim;
    float* st = a.state + (int64_t)slot * a.slot_stride + (int64_t)h * ((int64_t)dim * vdim + dim + 1);
    float* st_n = st + (int64_t)dim * vdim;
    float S[DPT], nv[DPT];
    float m = a.from_nothing ? -__builtin_inff() : 0.0f, f_sum = 0.0f;
    const bool resume = pos0 > 0 && !a.from_nothing;
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
        const int d = p * DPT + i;
        const bool live = resume && d < dim;
        S[i] = (live && col) ? st[(int64_t)d * vdim + j] : 0.0f;
        nv[i] = live ? st_n[d] : 0.0f;
    }
    if (resume) m = st_n[dim];

    const E* q = (const E*)a.q + (int64_t)row0 * a.ldq + (int64_t)h * dim;
    const E* k = (const E*)a.k + (int64_t)row0 * a.ldk + (int64_t)h * dim;
    const E* v = (const E*)a.v + (int64_t)row0 * a.ldv + (int64_t)h * vdim + j0;
    const E* gi = (const E*)a.gi + (int64_t)row0 * a.ldgi + h;
    const E* gf = (const E*)a.gf + (int64_t)row0 * a.ldgf + h;
    // a block in flight: this thread's share of its q, k, v and (threads 0 .. TB-1) one token's gates
    float rq_[QN], rk_[QN], rv_[VN], rgi = 0.0f, rgf = 0.0f;
    auto fetch = [&](int blk) {
        const int t0 = blk * TB;
#pragma unroll
        for (int i = 0; i < QN; ++i) {
            const int e = tid + 256 * i, tt = e / DM, d = e % DM;
            const bool ok = d < dim && t0 + tt < count;
            rq_[i] = (OUT && ok) ? to_f32(q[(int64_t)(t0 + tt) * a.ldq + d]) * a.q_scale : 0.0f;
            rk_[i] = ok ? to_f32(k[(int64_t)(t0 + tt) * a.ldk + d]) : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < VN; ++i) {
            const int e = tid + 256 * i, tt = e >> 6, jj = e & 63;
            rv_[i] = (j0 + jj < vdim && t0 + tt < count) ? to_f32(v[(int64_t)(t0 + tt) * a.ldv + jj]) : 0.0f;
        }
        if (tid < TB && t0 + tid < count) {
            rgi = to_f32(gi[(int64_t)(t0 + tid) * a.ldgi]);
            rgf = to_f32(gf[(int64_t)(t0 + tid) * a.ldgf]);
        }
    };
    auto stage = [&](int b) {
#pragma unroll
        for (int i = 0; i < QN; ++i) {
            const int e = tid + 256 * i;
            if (OUT) qs[b][e / DM][e % DM] = rq_[i];
            ks[b][e / DM][e % DM] = rk_[i];
        }
#pragma unroll
        for (int i = 0; i < VN; ++i) {
            const int e = tid + 256 * i;
            vs[b][e >> 6][e & 63] = rv_[i];
        }
        if (tid < TB) {
            gs[b][tid][0] = soft_cap(rgi, a.gate_cap);
            gs[b][tid][1] = log_sigmoid(soft_cap(rgf, a.gate_cap));
        }
    };
    const int n_blk = (count + TB - 1) / TB;
    if (n_blk > 0) fetch(0);
    for (int blk = 0; blk < n_blk; ++blk) {
        const int b = blk & 1;
        stage(b);                                          // (buffer b was last read a whole block of barriers ago)
        if (blk + 1 < n_blk) fetch(blk + 1);
        __syncthreads();
        const int n_tok = count - blk * TB < TB ? count - blk * TB : TB;
        for (int tt = 0; tt < n_tok; ++tt) {
            const int t = blk * TB + tt, pb = t & 1;
            const float li = gs[b][tt][0], lf = gs[b][tt][1];
            const float m_new = fmaxf(lf + m, li);
            const float keep = expf(lf + m - m_new), take = expf(li - m_new);      // (m = -inf: keep = 0)
            m = m_new;
            f_sum += lf;
            float acc = 0.0f, accn = 0.0f;
            const float tv = take * vs[b][tt][lane];
            const float4* k4 = reinterpret_cast<const float4*>(&ks[b][tt][p * DPT]);     // (rows past dim were staged as zeros)
            const float4* q4 = reinterpret_cast<const float4*>(&qs[b][tt][p * DPT]);
#pragma unroll
            for (int i4 = 0; i4 < DPT / 4; ++i4) {
                const float4 kk = k4[i4], qq = OUT ? q4[i4] : float4{0.f, 0.f, 0.f, 0.f};
                const float kd[4] = {kk.x, kk.y, kk.z, kk.w}, qd[4] = {qq.x, qq.y, qq.z, qq.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = 4 * i4 + e;
                    S[i] = keep * S[i] + kd[e] * tv;
                    nv[i] = keep * nv[i] + take * kd[e];
                    if (OUT) {
                        acc += S[i] * qd[e];
                        accn += nv[i] * qd[e];
                    }
                }
            }
            if (!OUT) continue;
            part_o[pb][p][lane] = acc;
            if (lane == 0) part_n[pb][p] = accn;
            __syncthreads();
            if (p == 0 && col) {
                const float num = (part_o[pb][0][lane] + part_o[pb][1][lane]) + (part_o[pb][2][lane] + part_o[pb][3][lane]);
                const float nq_dot = (part_n[pb][0] + part_n[pb][1]) + (part_n[pb][2] + part_n[pb][3]);
                const float den = fmaxf(fabsf(nq_dot), expf(-m_new)) + 1e-6f;
                a.out[(int64_t)(row0 + t) * a.ldo + (int64_t)h * vdim + j] = num / den;
            }
        }
    }
    // where the request's last state goes: its own record, or (the last segment of a prompt) the slot it belongs to
    if (a.end_slots && a.end_slots[blockIdx.x] >= 0) {
        st = a.end_state + (int64_t)a.end_slots[blockIdx.x] * a.end_slot_stride + (int64_t)h * ((int64_t)dim * vdim + dim + 1);
        st_n = st + (int64_t)dim * vdim;
    }
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
        const int d = p * DPT + i;
        if (d < dim) {
            if (col) st[(int64_t)d * vdim + j] = S[i];
            if (blockIdx.z == 0 && lane == 0) st_n[d] = nv[i];
        }
    }
    if (blockIdx.z == 0 && tid == 0) {
        st_n[dim] = m;
        if (a.log_f_sum) a.log_f_sum[(int64_t)blockIdx.x * a.H + h] = f_sum;
    }
}

// one workgroup per (chain, head, 1024 state elements): walks the chain's segments, handing each its start state and folding its
// contribution in.  Nothing is updated in place: the state after the last segment is what the second pass leaves.
__global__ __launch_bounds__(256) void mlstm_chain_kernel(const float* __restrict__ local, const float* __restrict__ f_sum,
                                                          float* __restrict__ start, const float* __restrict__ state, int64_t slot_stride,
                                                          const int32_t* __restrict__ chains, int H, int64_t rec) {
    const int32_t* ch = chains + 4 * blockIdx.x;
    const int slot = ch[0], pos0 = ch[1], seg0 = ch[2], n_seg = ch[3], h = blockIdx.y;
    const int64_t elems = rec - 1;                     // S and n; the record's last float is m
    const float* st = state + (int64_t)slot * slot_stride + (int64_t)h * rec;
    float mm = pos0 > 0 ? st[elems] : 0.0f;
    const int64_t e0 = (int64_t)blockIdx.z * 1024 + threadIdx.x;
    float v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = (pos0 > 0 && e0 + 256 * u < elems) ? st[e0 + 256 * u] : 0.0f;
    for (int g = seg0; g < seg0 + n_seg; ++g) {
        const float* lc = local + ((int64_t)g * H + h) * rec;
        float* sg = start + ((int64_t)g * H + h) * rec;
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (e0 + 256 * u < elems) sg[e0 + 256 * u] = v[u];
        if (blockIdx.z == 0 && threadIdx.x == 0) sg[elems] = mm;
        if (g + 1 == seg0 + n_seg) break;
        const float F = f_sum[(int64_t)g * H + h], ml = lc[elems];
        const float m_new = fmaxf(F + mm, ml);
        const float keep = expf(F + mm - m_new), take = expf(ml - m_new);
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (e0 + 256 * u < elems) v[u] = keep * v[u] + take * lc[e0 + 256 * u];
        mm = m_new;
    }
}

template <typename E>
int dispatch(const pcb_mlstm_args& a, hipStream_t stream) {
    const dim3 grid(a.n_reqs, a.H, pcb_ceil_div(a.vdim, 64)), block(256);
    if (a.out) {
        if (a.dim <= 64)
            hipLaunchKernelGGL((mlstm_kernel<E, 16, true>), grid, block, 0, stream, a);
        else if (a.dim <= 128)
            hipLaunchKernelGGL((mlstm_kernel<E, 32, true>), grid, block, 0, stream, a);
        else
            hipLaunchKernelGGL((mlstm_kernel<E, 64, true>), grid, block, 0, stream, a);
    } else {
        if (a.dim <= 64)
            hipLaunchKernelGGL((mlstm_kernel<E, 16, false>), grid, block, 0, stream, a);
        else if (a.dim <= 128)
            hipLaunchKernelGGL((mlstm_kernel<E, 32, false>), grid, block, 0, stream, a);
        else
            hipLaunchKernelGGL((mlstm_kernel<E, 64, false>), grid, block, 0, stream, a);
    }
    return pcb_check_launch("mlstm_kernel");
}

}  // namespace

PCB_EXPORT int pcb_mlstm(const pcb_mlstm_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_mlstm_args), PCB_ERR_ARG, "pcb_mlstm: struct size mismatch");
    PCB_REQUIRE(a->dtype == PCB_BF16 || a->dtype == PCB_F32, PCB_ERR_ARG, "pcb_mlstm: unknown dtype");
    PCB_REQUIRE(a->n_reqs >= 0 && a->H > 0 && a->dim > 0 && a->dim <= 256 && a->vdim > 0 && a->ldq >= (int64_t)a->H * a->dim &&
                    a->ldk >= (int64_t)a->H * a->dim && a->ldv >= (int64_t)a->H * a->vdim && a->ldgi >= a->H && a->ldgf >= a->H &&
                    a->slot_stride >= (int64_t)a->H * ((int64_t)a->dim * a->vdim + a->dim + 1) && (!a->out || a->ldo >= (int64_t)a->H * a->vdim),
                PCB_ERR_ARG, "pcb_mlstm: bad sizes (up to 256 key columns per head)");
    if (a->n_reqs == 0) return PCB_OK;
    PCB_REQUIRE(a->q && a->k && a->v && a->gi && a->gf && a->reqs && a->state, PCB_ERR_ARG, "pcb_mlstm: null pointer");
    PCB_REQUIRE(!a->end_slots || (a->end_state && a->end_slot_stride >= (int64_t)a->H * ((int64_t)a->dim * a->vdim + a->dim + 1)), PCB_ERR_ARG,
                "pcb_mlstm: end slots need the states they point into");
    return a->dtype == PCB_BF16 ? dispatch<pcb::bf16_t>(*a, (hipStream_t)stream) : dispatch<float>(*a, (hipStream_t)stream);
}

PCB_EXPORT int pcb_mlstm_chain(const float* local, const float* log_f_sum, float* start, const float* state, int64_t slot_stride,
                               const int32_t* chains, int32_t n_chains, int32_t H, int32_t dim, int32_t vdim, void* stream) {
    PCB_REQUIRE(n_chains >= 0 && H > 0 && dim > 0 && vdim > 0 && slot_stride >= (int64_t)H * ((int64_t)dim * vdim + dim + 1), PCB_ERR_ARG,
                "pcb_mlstm_chain: bad sizes");
    if (n_chains == 0) return PCB_OK;
    PCB_REQUIRE(local && log_f_sum && start && state && chains, PCB_ERR_ARG, "pcb_mlstm_chain: null pointer");
    const int64_t rec = (int64_t)dim * vdim + dim + 1;
    hipLaunchKernelGGL(mlstm_chain_kernel, dim3(n_chains, H, (unsigned)((rec - 1 + 1023) / 1024)), dim3(256), 0, (hipStream_t)stream, local,
                       log_f_sum, start, state, slot_stride, chains, H, rec);
    return pcb_check_launch("mlstm_chain_kernel");
}
