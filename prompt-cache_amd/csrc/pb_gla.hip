// pcb_gla: linear attention whose decay changes from token to token -- one decay per key channel (gated linear attention) or one
// per head (the state-space-duality form of a selective scan: k = B, q = C, v = dt * x) -- token by token, with the matrix state
// S [dim][vdim] of every (slot, head) in fp32 (see pcb_gla_args for the recurrence).
//
// One workgroup = one request x one head x 64 value columns.  Wave p of its four owns the key rows d = p DPT .. (p + 1) DPT - 1 and
// lane j the value column: a thread keeps its DPT entries S[d][j] in registers for the whole request.  Tokens arrive in blocks of
// TB: the whole block's q, k, v and log decays are requested at once (one memory round trip per block, and the next block's while
// the current one is worked on) and staged in LDS -- q scaled, v times its step size, the decays already through their one
// exponential per (token, channel), which the 64 value columns share --, and the block's tokens then run from LDS alone.  Every
// wave leaves its part of S^T q for each token of the block in LDS; after ONE barrier per block all threads add the four parts
// and store the block's output rows.
//
// A long prompt is cut into segments that run side by side: a first pass runs every segment from a zero state and leaves its
// contribution and the sum of its log decays (ld_sum), pcb_state_chain hands every segment its start state
// (S <- exp(ld_sum) S + contribution, row by row), and a second pass runs every segment from there and writes the outputs.
#include "pb_common.h"

namespace {
using namespace pcb;

constexpr int TB = 8;          // tokens per staged block

// OUT false: only the states move (the first pass over segments) -- no products with q, no partial sums
template <typename E, int DPT, bool OUT>
__global__ __launch_bounds__(256) void gla_kernel(pcb_gla_args a) {
    constexpr int DM = 4 * DPT;                 // key rows the workgroup can hold (>= dim)
    constexpr int QN = TB * DM / 256;           // q (k, decay) elements a thread fetches per block
    constexpr int VN = TB * 64 / 256;           // v elements a thread fetches per block
    __shared__ __attribute__((aligned(16))) float qs[2][TB][DM], ks[2][TB][DM], as[2][TB][DM];
    __shared__ float vs[2][TB][64];
    __shared__ float part_o[TB][4][64];
    __shared__ float lsum_s[256];
    const int tid = threadIdx.x, lane = tid & 63, p = tid >> 6;
    const int32_t* rq = a.reqs + 4 * blockIdx.x;
    const int slot = rq[0], pos0 = rq[1], count = rq[2], row0 = rq[3];
    const int h = blockIdx.y, hk = h / (a.H / a.Hk), dim = a.dim, vdim = a.vdim;
    const int j0 = blockIdx.z * 64, j = j0 + lane;
    const bool col = j < vdim;
    float* st = a.state + (int64_t)slot * a.slot_stride + (int64_t)h * dim * vdim;
    float S[DPT];
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
        const int d = p * DPT + i;
        S[i] = (pos0 > 0 && d < dim && col) ? st[(int64_t)d * vdim + j] : 0.0f;
    }
    const E* q = (const E*)a.q + (int64_t)row0 * a.ldq + (int64_t)hk * dim;
    const E* k = (const E*)a.k + (int64_t)row0 * a.ldk + (int64_t)hk * dim;
    const E* v = (const E*)a.v + (int64_t)row0 * a.ldv + (int64_t)h * vdim + j0;
    const float* ld = a.ld + (int64_t)row0 * a.ldld + (int64_t)h * a.dcols;
    const float* vsc = a.v_scale ? a.v_scale + (int64_t)row0 * a.ldvs + h : nullptr;
    const float coef = a.ld_coef ? a.ld_coef[h] : 1.0f;
    const bool per_channel = a.dcols > 1;
    // a block in flight: this thread's share of its q, k, log decays and v.  (256 is a multiple of DM: a thread meets the same key
    // channel in every block, so its sum of log decays is that channel's over the thread's tokens.)
    float rq_[QN], rk_[QN], rl_[QN], rv_[VN], l_sum = 0.0f;
    auto fetch = [&](int blk) {
        const int t0 = blk * TB;
#pragma unroll
        for (int i = 0; i < QN; ++i) {
            const int e = tid + 256 * i, tt = e / DM, d = e % DM;
            const bool ok = d < dim && t0 + tt < count;
            rq_[i] = (OUT && ok) ? to_f32(q[(int64_t)(t0 + tt) * a.ldq + d]) * a.q_scale : 0.0f;
            rk_[i] = ok ? to_f32(k[(int64_t)(t0 + tt) * a.ldk + d]) : 0.0f;
            rl_[i] = ok ? coef * ld[(int64_t)(t0 + tt) * a.ldld + (per_channel ? d : 0)] : 0.0f;
            l_sum += rl_[i];
        }
#pragma unroll
        for (int i = 0; i < VN; ++i) {
            const int e = tid + 256 * i, tt = e >> 6, jj = e & 63;
            const bool ok = j0 + jj < vdim && t0 + tt < count;
            rv_[i] = ok ? to_f32(v[(int64_t)(t0 + tt) * a.ldv + jj]) * (vsc ? vsc[(int64_t)(t0 + tt) * a.ldvs] : 1.0f) : 0.0f;
        }
    };
    auto stage = [&](int b) {
#pragma unroll
        for (int i = 0; i < QN; ++i) {
            const int e = tid + 256 * i;
            if (OUT) qs[b][e / DM][e % DM] = rq_[i];
            ks[b][e / DM][e % DM] = rk_[i];
            as[b][e / DM][e % DM] = expf(rl_[i]);           // (log decays are <= 0; rows past dim and tokens past the end: exp(0) on zeros)
        }
#pragma unroll
        for (int i = 0; i < VN; ++i) {
            const int e = tid + 256 * i;
            vs[b][e >> 6][e & 63] = rv_[i];
        }
    };
    const int n_blk = (count + TB - 1) / TB;
    if (n_blk > 0) fetch(0);
    for (int blk = 0; blk < n_blk; ++blk) {
        const int b = blk & 1;
        stage(b);                                          // (buffer b was last read two barriers ago)
        if (blk + 1 < n_blk) fetch(blk + 1);
        __syncthreads();
        const int n_tok = count - blk * TB < TB ? count - blk * TB : TB;
        for (int tt = 0; tt < n_tok; ++tt) {
            float acc = 0.0f;
            const float tv = vs[b][tt][lane];
            const float4* k4 = reinterpret_cast<const float4*>(&ks[b][tt][p * DPT]);     // (rows past dim were staged as zeros)
            const float4* q4 = reinterpret_cast<const float4*>(&qs[b][tt][p * DPT]);
            const float4* a4 = reinterpret_cast<const float4*>(&as[b][tt][p * DPT]);
#pragma unroll
            for (int i4 = 0; i4 < DPT / 4; ++i4) {
                const float4 kk = k4[i4], aa = a4[i4], qq = OUT ? q4[i4] : float4{0.f, 0.f, 0.f, 0.f};
                const float kd[4] = {kk.x, kk.y, kk.z, kk.w}, ad[4] = {aa.x, aa.y, aa.z, aa.w}, qd[4] = {qq.x, qq.y, qq.z, qq.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = 4 * i4 + e;
                    S[i] = ad[e] * S[i] + kd[e] * tv;
                    if (OUT) acc += S[i] * qd[e];
                }
            }
            if (OUT) part_o[tt][p][lane] = acc;
        }
        if (!OUT) continue;
        __syncthreads();
        for (int e = tid; e < n_tok * 64; e += 256) {
            const int tt = e >> 6, jj = e & 63;
            if (j0 + jj < vdim)
                a.out[(int64_t)(row0 + blk * TB + tt) * a.ldo + (int64_t)h * vdim + j0 + jj] =
                    (part_o[tt][0][jj] + part_o[tt][1][jj]) + (part_o[tt][2][jj] + part_o[tt][3][jj]);
        }
    }
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
        const int d = p * DPT + i;
        if (d < dim && col) st[(int64_t)d * vdim + j] = S[i];
    }
    if (a.ld_sum && blockIdx.z == 0) {
        // the request's sum of log decays per channel (or per head): the threads that met channel d add their parts
        lsum_s[tid] = l_sum;
        __syncthreads();
        if (tid < DM && tid < (per_channel ? dim : 1)) {
            float s = 0.0f;
            for (int u = tid; u < 256; u += DM) s += lsum_s[u];
            a.ld_sum[(int64_t)blockIdx.x * a.H * a.dcols + (int64_t)h * a.dcols + tid] = s;
        }
    }
}

template <typename E, bool OUT>
void dispatch_dim(const pcb_gla_args& a, hipStream_t stream) {
    const dim3 grid(a.n_reqs, a.H, pcb_ceil_div(a.vdim, 64)), block(256);
    if (a.dim <= 32)
        hipLaunchKernelGGL((gla_kernel<E, 8, OUT>), grid, block, 0, stream, a);
    else if (a.dim <= 64)
        hipLaunchKernelGGL((gla_kernel<E, 16, OUT>), grid, block, 0, stream, a);
    else if (a.dim <= 128)
        hipLaunchKernelGGL((gla_kernel<E, 32, OUT>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((gla_kernel<E, 64, OUT>), grid, block, 0, stream, a);
}

template <typename E>
int dispatch(const pcb_gla_args& a, hipStream_t stream) {
    if (a.out)
        dispatch_dim<E, true>(a, stream);
    else
        dispatch_dim<E, false>(a, stream);
    return pcb_check_launch("gla_kernel");
}

}  // namespace

PCB_EXPORT int pcb_gla(const pcb_gla_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_gla_args), PCB_ERR_ARG, "pcb_gla: struct size mismatch");
    PCB_REQUIRE(a->dtype == PCB_BF16 || a->dtype == PCB_F32, PCB_ERR_ARG, "pcb_gla: unknown dtype");
    PCB_REQUIRE(a->n_reqs >= 0 && a->H > 0 && a->H <= 65535 && a->Hk > 0 && a->H % a->Hk == 0 && a->dim > 0 && a->dim <= 256 && a->vdim > 0 &&
                    a->ldq >= (int64_t)a->Hk * a->dim && a->ldk >= (int64_t)a->Hk * a->dim && a->ldv >= (int64_t)a->H * a->vdim &&
                    (a->dcols == 1 || a->dcols == a->dim) && a->ldld >= (int64_t)a->H * a->dcols && (!a->v_scale || a->ldvs >= a->H) &&
                    a->slot_stride >= (int64_t)a->H * a->dim * a->vdim && (!a->out || a->ldo >= (int64_t)a->H * a->vdim),
                PCB_ERR_ARG, "pcb_gla: bad sizes (up to 256 key columns per head; a decay per key column or one per head)");
    if (a->n_reqs == 0) return PCB_OK;
    PCB_REQUIRE(a->q && a->k && a->v && a->ld && a->reqs && a->state, PCB_ERR_ARG, "pcb_gla: null pointer");
    return a->dtype == PCB_BF16 ? dispatch<pcb::bf16_t>(*a, (hipStream_t)stream) : dispatch<float>(*a, (hipStream_t)stream);
}
