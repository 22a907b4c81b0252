// pcb_mlstm: the matrix memory of an mLSTM layer, token by token.  Per (slot, head): S [dim][vdim], a normaliser n [dim] and a
// running maximum m of the log gates, all fp32 (see pcb_mlstm_args for the recurrence).
//
// One workgroup = one request x one head x 64 value columns.  Wave p of its four owns the key rows d = p, p + 4, p + 8, ... and
// lane j the value column: a thread keeps its DPT entries S[d][j] in registers for the whole request, and the matching entries of
// n as well (every lane of a wave holds the same ones, which spares a broadcast per token).  Per token the workgroup stages q and
// k in LDS (read back as broadcasts), every thread takes the two gates through cap / logsigmoid / the running maximum by itself,
// updates its slice and leaves partial sums of S^T q and n . q in LDS; wave 0 adds the four parts and stores the output row.
// The next token's q, k, v and gates are requested before the current token's arithmetic.
#include "pb_common.h"

namespace {
using namespace pcb;

__device__ __forceinline__ float soft_cap(float z, float cap) { return cap > 0.0f ? cap * tanhf(z / cap) : z; }
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.0f) - log1pf(expf(-fabsf(z))); }

template <typename E, int DPT>
__global__ __launch_bounds__(256) void mlstm_kernel(pcb_mlstm_args a) {
    __shared__ float qs[2][4 * DPT], ks[2][4 * DPT];
    __shared__ float part_o[4][64], part_n[4];
    const int tid = threadIdx.x, lane = tid & 63, p = tid >> 6;
    const int32_t* rq = a.reqs + 4 * blockIdx.x;
    const int slot = rq[0], pos0 = rq[1], count = rq[2], row0 = rq[3];
    const int h = blockIdx.y, dim = a.dim, vdim = a.vdim;
    const int j = blockIdx.z * 64 + lane;
    const bool col = j < vdim;
    float* st = a.state + (int64_t)slot * a.slot_stride + (int64_t)h * ((int64_t)dim * vdim + dim + 1);
    float* st_n = st + (int64_t)dim * vdim;
    float S[DPT], nv[DPT];
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
        const int d = p + 4 * i;
        const bool live = pos0 > 0 && d < dim;
        S[i] = (live && col) ? st[(int64_t)d * vdim + j] : 0.0f;
        nv[i] = live ? st_n[d] : 0.0f;
    }
    if (pos0 > 0) m = st_n[dim];

    const E* q = (const E*)a.q + (int64_t)row0 * a.ldq + (int64_t)h * dim;
    const E* k = (const E*)a.k + (int64_t)row0 * a.ldk + (int64_t)h * dim;
    const E* v = (const E*)a.v + (int64_t)row0 * a.ldv + (int64_t)h * vdim;
    const E* gi = (const E*)a.gi + (int64_t)row0 * a.ldgi + h;
    const E* gf = (const E*)a.gf + (int64_t)row0 * a.ldgf + h;
    // what the next token brings: the thread's share of q / k for the staging (tid < dim), its value, both gates
    float nq = 0.0f, nk = 0.0f, nval = 0.0f, ngi = 0.0f, ngf = 0.0f;
    auto fetch = [&](int t) {
        if (tid < dim) {
            nq = to_f32(q[(int64_t)t * a.ldq + tid]) * a.q_scale;
            nk = to_f32(k[(int64_t)t * a.ldk + tid]);
        }
        nval = col ? to_f32(v[(int64_t)t * a.ldv + j]) : 0.0f;
        ngi = to_f32(gi[(int64_t)t * a.ldgi]);
        ngf = to_f32(gf[(int64_t)t * a.ldgf]);
    };
    if (count > 0) fetch(0);
    for (int t = 0; t < count; ++t) {
        const int b = t & 1;
        if (tid < dim) {
            qs[b][tid] = nq;
            ks[b][tid] = nk;
        }
        const float val = nval;
        const float li = soft_cap(ngi, a.gate_cap), lf = log_sigmoid(soft_cap(ngf, a.gate_cap));
        if (t + 1 < count) fetch(t + 1);
        __syncthreads();                                   // q and k of this token are staged (and part_* of the last one were read)
        const float m_new = fmaxf(lf + m, li);
        const float keep = expf(lf + m - m_new), take = expf(li - m_new);
        m = m_new;
        float acc = 0.0f, accn = 0.0f;
        const float tv = take * val;
#pragma unroll
        for (int i = 0; i < DPT; ++i) {
            const int d = p + 4 * i;                       // (rows past dim hold zeros in S and n and read staged values that are never used)
            const float kd = d < dim ? ks[b][d] : 0.0f, qd = d < dim ? qs[b][d] : 0.0f;
            S[i] = keep * S[i] + kd * tv;
            nv[i] = keep * nv[i] + take * kd;
            acc += S[i] * qd;
            accn += nv[i] * qd;
        }
        part_o[p][lane] = acc;
        if (lane == 0) part_n[p] = accn;
        __syncthreads();
        if (p == 0 && col) {
            const float num = (part_o[0][lane] + part_o[1][lane]) + (part_o[2][lane] + part_o[3][lane]);
            const float nq_dot = (part_n[0] + part_n[1]) + (part_n[2] + part_n[3]);
            const float den = fmaxf(fabsf(nq_dot), expf(-m_new)) + 1e-6f;
            if (a.out) a.out[(int64_t)(row0 + t) * a.ldo + (int64_t)h * vdim + j] = num / den;
        }
    }
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
        const int d = p + 4 * i;
        if (d < dim) {
            if (col) st[(int64_t)d * vdim + j] = S[i];
            if (blockIdx.z == 0 && lane == 0) st_n[d] = nv[i];
        }
    }
    if (blockIdx.z == 0 && tid == 0) st_n[dim] = m;
}

template <typename E>
int dispatch(const pcb_mlstm_args& a, hipStream_t stream) {
    const dim3 grid(a.n_reqs, a.H, pcb_ceil_div(a.vdim, 64)), block(256);
    if (a.dim <= 64)
        hipLaunchKernelGGL((mlstm_kernel<E, 16>), grid, block, 0, stream, a);
    else if (a.dim <= 128)
        hipLaunchKernelGGL((mlstm_kernel<E, 32>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((mlstm_kernel<E, 64>), grid, block, 0, stream, a);
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
    return a->dtype == PCB_BF16 ? dispatch<pcb::bf16_t>(*a, (hipStream_t)stream) : dispatch<float>(*a, (hipStream_t)stream);
}
