// pcb_head_prep: what happens to projected rows between the projection and the attention -- a unit-RMS norm per head (with or
// without a gain), a blend with another layer's values, rotary positions on neighbouring column pairs, and the store into a row
// matrix or a slot's cache (row by row or column by column).  Up to four segments (queries, keys, values, ...) per launch.
//
// One workgroup per (row, segment).  The turn of every column pair depends on the row's position only, so the workgroup first
// fills a cos / sin table in LDS -- the angle is the float64 product position x frequency, reduced by float64 sincos, so a
// position in the thousands costs no bits of the angle -- and its waves then take the heads in turn: one pass for the sum of
// squares, one that norms, blends, turns and stores.  A lane owns neighbouring column pairs, so a rotation never crosses lanes.
#include "pb_common.h"

namespace {
using namespace pcb;

constexpr int MAX_PAIRS = 512;   // rotated column pairs per head

template <typename E>
__global__ __launch_bounds__(256) void head_prep_kernel(pcb_head_prep_args a) {
    __shared__ float cs[MAX_PAIRS], sn[MAX_PAIRS];
    const pcb_head_prep_seg& s = a.seg[blockIdx.y];
    const int64_t row = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int D = s.head_dim, np = s.rot_dims / 2;
    if (np > 0) {
        const double p = (double)a.pos[row];
        for (int i = threadIdx.x; i < np; i += blockDim.x) {
            double sv, cv;
            sincos(p * a.freqs[i], &sv, &cv);
            cs[i] = (float)cv * a.rot_mag;
            sn[i] = (float)sv * a.rot_mag;
        }
        __syncthreads();
    }
    const float lam = s.blend ? s.blend[0] : 0.0f;
    for (int h = wave; h < s.heads; h += waves) {
        const E* __restrict__ x = (const E*)s.src + row * s.ld_src + (int64_t)h * s.src_head_stride;
        float inv = 1.0f;
        if (s.norm) {
            float ss = 0.0f;
            for (int c = lane; c < D; c += 64) {
                const float v = to_f32(x[c]);
                ss += v * v;
            }
            ss = wave_sum(ss);
            inv = 1.0f / sqrtf(ss / (float)D + a.eps);
        }
        const float* __restrict__ other = s.blend ? s.other + row * s.ld_other + (int64_t)h * D : nullptr;
        float* __restrict__ keep = s.keep ? s.keep + row * s.ld_keep + (int64_t)h * D : nullptr;
        E* dst = (E*)s.dst + (s.row_off ? s.row_off[row] : row * s.ld_dst) + (int64_t)h * s.head_stride;
        for (int c0 = 2 * lane; c0 < D; c0 += 128) {
            float v[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int c = c0 + e;
                float t = 0.0f;
                if (c < D) {
                    t = to_f32(x[c]) * inv;
                    if (s.gain) t *= s.gain[c];
                    if (other) t = (1.0f - lam) * t + lam * other[c];
                    if (keep) keep[c] = t;
                }
                v[e] = t;
            }
            const int i = (c0 - s.rot_off) >> 1;
            if (c0 >= s.rot_off && i < np) {             // (rot_off is even: a pair never straddles the rotated range's edge)
                const float u = v[0], w = v[1];
                v[0] = u * cs[i] - w * sn[i];
                v[1] = w * cs[i] + u * sn[i];
            }
#pragma unroll
            for (int e = 0; e < 2; ++e)
                if (c0 + e < D) dst[(int64_t)(c0 + e) * s.col_stride] = from_f32<E>(v[e]);
        }
    }
}

}  // namespace

PCB_EXPORT int pcb_head_prep(const pcb_head_prep_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_head_prep_args), PCB_ERR_ARG, "pcb_head_prep: struct size mismatch");
    PCB_REQUIRE(a->dtype == PCB_BF16 || a->dtype == PCB_F32, PCB_ERR_ARG, "pcb_head_prep: unknown dtype");
    PCB_REQUIRE(a->n_rows >= 0 && a->n_segs >= 1 && a->n_segs <= 4, PCB_ERR_ARG, "pcb_head_prep: one to four segments");
    int rot = 0;
    for (int i = 0; i < a->n_segs; ++i) {
        const pcb_head_prep_seg& s = a->seg[i];
        PCB_REQUIRE(s.heads > 0 && s.head_dim > 0 && s.head_dim <= 1024 && s.src_head_stride >= 0 && s.ld_src >= (int64_t)(s.heads - 1) * s.src_head_stride + s.head_dim && s.col_stride > 0,
                    PCB_ERR_ARG, "pcb_head_prep: bad segment sizes (heads of up to 1024 columns)");
        PCB_REQUIRE(s.rot_dims >= 0 && s.rot_dims % 2 == 0 && s.rot_off >= 0 && s.rot_off % 2 == 0 && s.rot_off + s.rot_dims <= s.head_dim &&
                        s.rot_dims <= 2 * MAX_PAIRS && (s.rot_dims == 0 || rot == 0 || rot == s.rot_dims),
                    PCB_ERR_ARG, "pcb_head_prep: rotated columns come in pairs inside the head, the same number in every segment that rotates");
        if (s.rot_dims) rot = s.rot_dims;
        PCB_REQUIRE(!s.blend || (s.other && s.ld_other >= (int64_t)s.heads * s.head_dim), PCB_ERR_ARG, "pcb_head_prep: a blend needs the other rows");
        PCB_REQUIRE(!s.keep || s.ld_keep >= (int64_t)s.heads * s.head_dim, PCB_ERR_ARG, "pcb_head_prep: keep rows too short");
        PCB_REQUIRE(a->n_rows == 0 || (s.src && s.dst), PCB_ERR_ARG, "pcb_head_prep: null pointer");
    }
    if (a->n_rows == 0) return PCB_OK;
    PCB_REQUIRE(rot == 0 || (a->pos && a->freqs), PCB_ERR_ARG, "pcb_head_prep: a rotation needs positions and frequencies");
    const dim3 grid(a->n_rows, a->n_segs);
    if (a->dtype == PCB_BF16)
        hipLaunchKernelGGL(head_prep_kernel<pcb::bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, *a);
    else
        hipLaunchKernelGGL(head_prep_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, *a);
    return pcb_check_launch("head_prep_kernel");
}
