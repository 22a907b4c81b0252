// pcb_attn_softmax: causal softmax attention over a slot-addressed cache with separate keys and values (grouped key/value
// heads, value size independent of the key size, optional sliding window or blocks of positions that see only themselves, per-row
// score factor, optional learned sink in the denominator, optional output gate per element or per head).
//
// One workgroup = one tile of up to 16 queries x one query head; its four waves take every fourth block of 32 keys and keep a
// running maximum / denominator per query (online softmax), then merge through LDS.  Both products are "swapped" so that no
// operand is transposed between them:
//   S^T = K Q^T   a wave's result tile has the query in the lane's column (l & 15) and keys 4 (l >> 4) + r in its rows,
//   O^T = V^T P^T the weights P of a query are exactly what its lanes hold; the k index of this product runs over the 32 keys of
//                 the block in the order (l >> 4, e) -> key 4 (l >> 4) + e (e < 4), 16 + 4 (l >> 4) + e - 4 (e >= 4), the same for
//                 both operands, so the permutation cancels.
// With one key head and tiles of one row each (decoding over a shared latent), head_rows makes the 16 rows of a tile 16 HEADS of that
// one token instead: the heads read the same keys and values, so one pass over them serves sixteen heads.
// Scores, maxima, weights and sums are fp32.  bf16: the weights enter the second product as a hi + lo pair of bf16 values (two
// MFMAs), so they are not rounded to 8 bits; fp32: the fp32 matrix cores take them as they are.
#include "pb_common.h"

namespace {
using namespace pcb;

constexpr int AW = 4;          // waves of a workgroup

template <typename E>
struct PFrag;
template <>
struct PFrag<bf16_t> {
    Frag<bf16_t> hi, lo;
};
template <>
struct PFrag<float> {
    Frag<float> hi;
};

__device__ __forceinline__ void make_p(PFrag<bf16_t>& f, const float (&p)[8]) {
    // hi = the upper 16 bits of p as they stand, lo = the rest, cut to 16 bits: hi + lo carries 16 bits of p's mantissa (p is a
    // finite non-negative weight, so no rounding carry or NaN needs care)
    uint32_t h[8], l[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t u = __float_as_uint(p[e]);
        h[e] = u >> 16;
        l[e] = __float_as_uint(p[e] - __uint_as_float(u & 0xffff0000u)) >> 16;
    }
    f.hi.v = u32x4{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
    f.lo.v = u32x4{l[0] | (l[1] << 16), l[2] | (l[3] << 16), l[4] | (l[5] << 16), l[6] | (l[7] << 16)};
}
__device__ __forceinline__ void make_p(PFrag<float>& f, const float (&p)[8]) {
#pragma unroll
    for (int e = 0; e < 8; ++e) f.hi.v[e] = p[e];
}

// the value operand of one 16-column block: element e of lane (column c, group g) is V[key(g, e)][c]
__device__ __forceinline__ Frag<bf16_t> load_v(const bf16_t* const (&rows)[8], int c, bool ok) {
    Frag<bf16_t> f;
    uint32_t w[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) w[e] = ok ? rows[e][c].bits : 0u;
    f.v = u32x4{w[0] | (w[1] << 16), w[2] | (w[3] << 16), w[4] | (w[5] << 16), w[6] | (w[7] << 16)};
    return f;
}
__device__ __forceinline__ Frag<float> load_v(const float* const (&rows)[8], int c, bool ok) {
    Frag<float> f;
#pragma unroll
    for (int e = 0; e < 8; ++e) f.v[e] = ok ? rows[e][c] : 0.0f;
    return f;
}

// the same operand from a cache kept column by column: `col` points at key 32 kb of the lane's value column; the lane's eight keys
// are the two runs 4 g .. 4 g + 3 and 16 + 4 g .. 16 + 4 g + 3, one wide load each.  Keys past `valid` (counted from key 32 kb)
// are replaced by zeros: what lies there need not be numbers.
__device__ __forceinline__ Frag<bf16_t> load_v_cols(const bf16_t* col, int g, bool ok, int valid) {
    Frag<bf16_t> f;
    uint2 lo = uint2{0u, 0u}, hi = uint2{0u, 0u};
    if (ok) {
        lo = *reinterpret_cast<const uint2*>(col + 4 * g);
        hi = *reinterpret_cast<const uint2*>(col + 16 + 4 * g);
    }
    if (valid < 32) {
        const int a = valid - 4 * g, b = valid - 16 - 4 * g;      // how many of each run exist
        lo.x &= a >= 2 ? 0xffffffffu : (a == 1 ? 0x0000ffffu : 0u);
        lo.y &= a >= 4 ? 0xffffffffu : (a == 3 ? 0x0000ffffu : 0u);
        hi.x &= b >= 2 ? 0xffffffffu : (b == 1 ? 0x0000ffffu : 0u);
        hi.y &= b >= 4 ? 0xffffffffu : (b == 3 ? 0x0000ffffu : 0u);
    }
    f.v = u32x4{lo.x, lo.y, hi.x, hi.y};
    return f;
}
__device__ __forceinline__ Frag<float> load_v_cols(const float* col, int g, bool ok, int valid) {
    Frag<float> f;
    float4 lo = float4{0.f, 0.f, 0.f, 0.f}, hi = lo;
    if (ok) {
        lo = *reinterpret_cast<const float4*>(col + 4 * g);
        hi = *reinterpret_cast<const float4*>(col + 16 + 4 * g);
    }
    const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) f.v[e] = ((e < 4 ? 4 * g + e : 16 + 4 * g + e - 4) < valid) ? v[e] : 0.0f;
    return f;
}

__device__ __forceinline__ f4 mma_p(const Frag<bf16_t>& v, const PFrag<bf16_t>& p, f4 c) {
    c = mma(v, p.hi, c);
    return mma(v, p.lo, c);
}
__device__ __forceinline__ f4 mma_p(const Frag<float>& v, const PFrag<float>& p, f4 c) { return mma(v, p.hi, c); }

// KSQ: 32-element k-steps of the key size; VB: 16-column blocks of the value size
template <typename E, int KSQ, int VB>
__global__ __launch_bounds__(64 * AW) void attn_softmax_kernel(pcb_attn_softmax_args a) {
    __shared__ float red_o[AW - 1][VB * 256];
    __shared__ float red_ml[AW - 1][2][16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, c = lane & 15;
    // (the launch walks the tiles from the last to the first: within a request later tiles see more keys, and the long ones should
    // not be the ones that start last)
    const int32_t* tile = a.tiles + 4 * (gridDim.x - 1 - blockIdx.x);
    const int slot = tile[0], pos0 = tile[1], rows = tile[2], row0 = tile[3];
    const int dim = a.dim, vdim = a.vdim;
    // what the 16 lanes-columns of the tile stand for: its rows (one head, blockIdx.y), or -- head_rows -- 16 heads of its one row
    const int n_q = a.head_rows ? (a.H - 16 * (int)blockIdx.y < 16 ? a.H - 16 * (int)blockIdx.y : 16) : rows;
    const int last = pos0 + (a.head_rows ? 0 : rows - 1);   // the newest key any query of the tile sees
    const int qi = c < n_q ? c : n_q - 1;                   // (lanes past the tile repeat its last query; nothing of theirs is stored)
    const int h = a.head_rows ? 16 * (int)blockIdx.y + qi : (int)blockIdx.y;
    const int hk = a.head_rows ? 0 : h / (a.H / a.Hkv);
    const int qpos = a.head_rows ? pos0 : pos0 + qi;
    const int64_t qrow = a.head_rows ? row0 : row0 + qi;
    const E* K = (const E*)a.kcache + (int64_t)slot * a.slot_stride + (int64_t)hk * a.head_stride;
    const E* V = (const E*)a.vcache + (int64_t)slot * a.v_slot_stride + (int64_t)hk * a.v_head_stride;
    const E* qp = (const E*)a.q + qrow * a.ldq + (int64_t)h * dim;
    constexpr int CE = 16 / sizeof(E);
    const bool qvec = ((uintptr_t)a.q % 16 == 0) && (a.ldq % CE == 0) && (dim % CE == 0);
    const bool kvec = ((uintptr_t)a.kcache % 16 == 0) && (a.slot_stride % CE == 0) && (a.head_stride % CE == 0) && (a.row_stride % CE == 0);
    Frag<E> qf[KSQ];
#pragma unroll
    for (int ks = 0; ks < KSQ; ++ks) qf[ks] = load_frag(qp + 32 * ks, g, dim - 32 * ks, qvec);
    // scores are kept in units of ln 2 (the factor log2(e) rides on the scale), so that every exponential is one v_exp_f32
    const float sc = a.scale * (a.q_scale ? a.q_scale[qrow] : 1.0f) * 1.44269504088896f;
    const float NEG = -__builtin_inff();
    // the oldest key this lane's query sees: the window's and the block's edges, whichever is later
    // (keys before the window's edge stay visible when they are among the sequence's kept first ones; the block's edge hides all)
    const int key_lo = a.window > 0 ? qpos - a.window + 1 : 0;
    const int blk_lo = a.block > 0 ? qpos / a.block * a.block : 0;
    const int kept = a.window > 0 ? a.keep_first : 0;

    float m = NEG, l = 0.0f;
    f4 o[VB];
#pragma unroll
    for (int vb = 0; vb < VB; ++vb) o[vb] = f4{0.f, 0.f, 0.f, 0.f};

    int kb_lo = a.window > 0 ? (pos0 - a.window + 1 > 0 ? (pos0 - a.window + 1) / 32 : 0) : 0;
    if (a.block > 0) kb_lo = max(kb_lo, pos0 / a.block * a.block / 32);      // (the tile's first query has the oldest block)
    int kb_hi = last / 32;
    // kept first keys: the blocks that hold them and lie before the window's first block are walked too.  The walk runs over
    // indices v in [kb_lo - n_first, kb_hi]: v >= kb_win stands for key block v itself, v < kb_win for block v - (kb_win - n_first).
    const int kb_win = kb_lo;
    const int n_first = (a.keep_first > 0 && a.window > 0) ? (kb_win < (a.keep_first + 31) / 32 ? kb_win : (a.keep_first + 31) / 32) : 0;
    const int v_shift = kb_win - n_first;
    kb_lo -= n_first;
    auto block_of = [&](int v) { return v < kb_win ? v - v_shift : v; };
    if (a.n_splits > 1) {                                   // this workgroup's run of the key blocks (it may be empty)
        const int per = (kb_hi - kb_lo + a.n_splits) / a.n_splits;
        kb_lo += (int)blockIdx.z * per;
        kb_hi = kb_lo + per - 1 < kb_hi ? kb_lo + per - 1 : kb_hi;
    }
    // the key operands of a block are requested one block ahead (where the registers allow it), so that their latency hides behind
    // the block in work
    constexpr bool PREK = sizeof(E) == 2 ? KSQ <= 4 : KSQ <= 2;
    Frag<E> kn[PREK ? 2 : 1][PREK ? KSQ : 1];
    auto fetch_k = [&](int kv) {
        const int kb = block_of(kv);
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            int j = kb * 32 + kt * 16 + c;                  // this lane's key row of the K operand
            j = j > last ? last : j;
            const E* kp = K + (int64_t)j * a.row_stride;
#pragma unroll
            for (int ks = 0; ks < KSQ; ++ks) kn[PREK ? kt : 0][PREK ? ks : 0] = load_frag(kp + 32 * ks, g, dim - 32 * ks, kvec);
        }
    };
    if (PREK && kb_lo + wave <= kb_hi) fetch_k(kb_lo + wave);
    for (int kv = kb_lo + wave; kv <= kb_hi; kv += AW) {
        const int kb = block_of(kv);
        float s[8];
        Frag<E> kc[PREK ? 2 : 1][PREK ? KSQ : 1];
        if (PREK) {
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int ks = 0; ks < KSQ; ++ks) kc[PREK ? kt : 0][PREK ? ks : 0] = kn[PREK ? kt : 0][PREK ? ks : 0];
            if (kv + AW <= kb_hi) fetch_k(kv + AW);
        }
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            int j = kb * 32 + kt * 16 + c;
            j = j > last ? last : j;
            const E* kp = K + (int64_t)j * a.row_stride;
            f4 acc = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KSQ; ++ks)
                acc = mma(PREK ? kc[PREK ? kt : 0][PREK ? ks : 0] : load_frag(kp + 32 * ks, g, dim - 32 * ks, kvec), qf[ks], acc);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = kb * 32 + kt * 16 + 4 * g + r;
                const bool seen = key <= qpos && key >= blk_lo && (key >= key_lo || key < kept);
                s[kt * 4 + r] = seen ? acc[r] * sc : NEG;
            }
        }
        // the value operands are requested before the softmax arithmetic (column-wise cache: two wide loads per 16 columns)
        const int v_valid = last + 1 - kb * 32;             // keys of this block that exist
        Frag<E> vfs[VB];
        if (a.v_cols) {
#pragma unroll
            for (int vb = 0; vb < VB; ++vb) {
                const int col = vb * 16 + c;
                if (vb * 16 < vdim) vfs[vb] = load_v_cols(V + (int64_t)(col < vdim ? col : 0) * a.v_stride + kb * 32, g, col < vdim, v_valid);
            }
        }
        float bm = s[0];
#pragma unroll
        for (int e = 1; e < 8; ++e) bm = fmaxf(bm, s[e]);
        bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
        bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
        const float m_new = fmaxf(m, bm);
        const float m_use = m_new == NEG ? 0.0f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m - m_use);      // (m = -inf: 0)
        float p[8], psum = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            p[e] = __builtin_amdgcn_exp2f(s[e] - m_use);
            psum += p[e];
        }
        l = l * alpha + psum;
        m = m_new;
        PFrag<E> pf;
        make_p(pf, p);
        const E* vrows[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            int key = kb * 32 + (e < 4 ? 4 * g + e : 16 + 4 * g + e - 4);
            key = key > last ? last : key;
            vrows[e] = V + (int64_t)key * a.v_stride;
        }
#pragma unroll
        for (int vb = 0; vb < VB; ++vb) {
            if (vb * 16 >= vdim) break;
            const int col = vb * 16 + c;
            const Frag<E> vf = a.v_cols ? vfs[vb] : load_v(vrows, col, col < vdim);
            f4 t = o[vb];
#pragma unroll
            for (int r = 0; r < 4; ++r) t[r] *= alpha;
            o[vb] = mma_p(vf, pf, t);
        }
    }
    // the denominator's parts of the four lane groups
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);

    // merge the waves: wave 0 collects
    if (wave > 0) {
#pragma unroll
        for (int vb = 0; vb < VB; ++vb)
#pragma unroll
            for (int r = 0; r < 4; ++r) red_o[wave - 1][(vb * 4 + r) * 64 + lane] = o[vb][r];
        if (g == 0) {
            red_ml[wave - 1][0][c] = m;
            red_ml[wave - 1][1][c] = l;
        }
    }
    __syncthreads();
    if (wave > 0) return;
    float mm = m;
#pragma unroll
    for (int w = 0; w < AW - 1; ++w) mm = fmaxf(mm, red_ml[w][0][c]);
    const float m_use = mm == NEG ? 0.0f : mm;
    float f0 = __builtin_amdgcn_exp2f(m - m_use);
    float lt = l * f0;
#pragma unroll
    for (int vb = 0; vb < VB; ++vb)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[vb][r] *= f0;
#pragma unroll
    for (int w = 0; w < AW - 1; ++w) {
        const float fw = __builtin_amdgcn_exp2f(red_ml[w][0][c] - m_use);
        lt += red_ml[w][1][c] * fw;
#pragma unroll
        for (int vb = 0; vb < VB; ++vb)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[vb][r] += fw * red_o[w][(vb * 4 + r) * 64 + lane];
    }
    if (c >= n_q) return;
    if (a.n_splits > 1) {
        float* pp = a.part + ((qrow * a.H + h) * a.n_splits + blockIdx.z) * (int64_t)(vdim + 2);
        if (g == 0) pp[vdim] = mm, pp[vdim + 1] = lt;
#pragma unroll
        for (int vb = 0; vb < VB; ++vb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int col = vb * 16 + 4 * g + r;
                if (col < vdim) pp[col] = o[vb][r];
            }
        return;
    }
    float keep = 1.0f;
    if (a.sink) {
        // one more term exp(sink) without a value: the sum moves to the larger of the two maxima (a query always sees itself, so
        // m_use is a number)
        const float sk = a.sink[h] * 1.44269504088896f;
        const float top = fmaxf(m_use, sk);
        keep = __builtin_amdgcn_exp2f(m_use - top);
        lt = lt * keep + __builtin_amdgcn_exp2f(sk - top);
    }
    const float inv = keep / lt;
    E* op = (E*)a.out + qrow * a.ldo + (int64_t)h * vdim;
    const E* gp = a.gate ? (const E*)a.gate + qrow * a.ldg + (a.gate_per_head ? 0 : (int64_t)h * vdim) : nullptr;
    const float gh = (gp && a.gate_per_head) ? to_f32(gp[h]) : 1.0f;
#pragma unroll
    for (int vb = 0; vb < VB; ++vb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int col = vb * 16 + 4 * g + r;
            if (col < vdim) {
                float v = o[vb][r] * inv * gh;
                if (gp && !a.gate_per_head) v *= to_f32(gp[col]);
                op[col] = from_f32<E>(v);
            }
        }
}

// one workgroup per (tile, head): the runs' partial results of each query are rescaled to their common maximum and summed
template <typename E>
__global__ __launch_bounds__(256) void attn_merge_kernel(pcb_attn_softmax_args a) {
    const int32_t* tile = a.tiles + 4 * blockIdx.x;
    const int rows = tile[2], row0 = tile[3], h = blockIdx.y, vdim = a.vdim, Z = a.n_splits;
    const float NEG = -__builtin_inff();
    for (int i = threadIdx.x; i < rows * vdim; i += 256) {
        const int64_t qrow = row0 + i / vdim;
        const int col = i % vdim;
        const float* pp = a.part + (qrow * a.H + h) * Z * (int64_t)(vdim + 2);
        float mm = NEG;
        for (int z = 0; z < Z; ++z) mm = fmaxf(mm, pp[z * (vdim + 2) + vdim]);
        const float m_use = mm == NEG ? 0.0f : mm;
        float l = 0.0f, o = 0.0f;
        for (int z = 0; z < Z; ++z) {
            const float f = __builtin_amdgcn_exp2f(pp[z * (vdim + 2) + vdim] - m_use);      // (maxima are in units of ln 2)
            l += f * pp[z * (vdim + 2) + vdim + 1];
            o += f * pp[z * (vdim + 2) + col];
        }
        if (a.sink) {
            const float sk = a.sink[h] * 1.44269504088896f;
            const float top = fmaxf(m_use, sk);
            const float keep = __builtin_amdgcn_exp2f(m_use - top);
            l = l * keep + __builtin_amdgcn_exp2f(sk - top);
            o *= keep;
        }
        float v = o / l;
        if (a.gate) v *= to_f32(((const E*)a.gate)[qrow * a.ldg + (a.gate_per_head ? (int64_t)h : (int64_t)h * vdim + col)]);
        ((E*)a.out)[qrow * a.ldo + (int64_t)h * vdim + col] = from_f32<E>(v);
    }
}

template <typename E>
int dispatch(const pcb_attn_softmax_args& a, hipStream_t stream) {
    const dim3 grid(a.n_tiles, a.head_rows ? (a.H + 15) / 16 : a.H, a.n_splits > 1 ? a.n_splits : 1), block(64 * AW);
    const int big = a.dim > a.vdim ? a.dim : a.vdim;
    if (big <= 64)
        hipLaunchKernelGGL((attn_softmax_kernel<E, 2, 4>), grid, block, 0, stream, a);
    else if (big <= 128)
        hipLaunchKernelGGL((attn_softmax_kernel<E, 4, 8>), grid, block, 0, stream, a);
    else if (a.dim <= 256)
        hipLaunchKernelGGL((attn_softmax_kernel<E, 8, 16>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((attn_softmax_kernel<E, 12, 16>), grid, block, 0, stream, a);
    if (a.n_splits > 1) hipLaunchKernelGGL(attn_merge_kernel<E>, dim3(a.n_tiles, a.H), dim3(256), 0, stream, a);
    return pcb_check_launch("attn_softmax_kernel");
}

}  // namespace

PCB_EXPORT int pcb_attn_softmax(const pcb_attn_softmax_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_attn_softmax_args), PCB_ERR_ARG, "pcb_attn_softmax: struct size mismatch");
    PCB_REQUIRE(a->dtype == PCB_BF16 || a->dtype == PCB_F32, PCB_ERR_ARG, "pcb_attn_softmax: unknown dtype");
    PCB_REQUIRE(a->n_tiles >= 0 && a->H > 0 && a->Hkv > 0 && a->H % a->Hkv == 0 && a->dim > 0 && a->dim <= 384 && a->vdim > 0 &&
                    a->vdim <= 256 && a->ldq >= (int64_t)a->H * a->dim && a->ldo >= (int64_t)a->H * a->vdim &&
                    a->row_stride >= a->dim && (a->v_cols ? (a->v_stride % 8 == 0 && a->v_stride > 0 && (uintptr_t)a->vcache % 16 == 0 &&
                                                             a->v_head_stride % 8 == 0 && a->v_slot_stride % 8 == 0)
                                                          : a->v_stride >= a->vdim),
                PCB_ERR_ARG, "pcb_attn_softmax: bad sizes (key size up to 384, value size up to 256; a column-wise value cache in multiples of 8)");
    if (a->n_tiles == 0) return PCB_OK;
    PCB_REQUIRE(a->q && a->tiles && a->kcache && a->vcache && a->out &&
                    (!a->gate || a->ldg >= (a->gate_per_head ? (int64_t)a->H : (int64_t)a->H * a->vdim)),
                PCB_ERR_ARG, "pcb_attn_softmax: null pointer");
    PCB_REQUIRE(!a->head_rows || a->Hkv == 1, PCB_ERR_ARG, "pcb_attn_softmax: heads as rows need one key head (and tiles of one row)");
    PCB_REQUIRE(a->n_splits <= 1 || (a->part && a->n_splits <= 64), PCB_ERR_ARG, "pcb_attn_softmax: up to 64 runs, with their scratch");
    return a->dtype == PCB_BF16 ? dispatch<pcb::bf16_t>(*a, (hipStream_t)stream) : dispatch<float>(*a, (hipStream_t)stream);
}
