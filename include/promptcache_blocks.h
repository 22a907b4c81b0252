/* C-ABI of libpromptcache_blocks.so: building-block kernels (gfx950) for decoder designs that keep plain row-major bf16 or fp32
 * tensors and an fp32 residual stream.  Built from prompt-cache_amd/csrc/pb_*.hip; bound by promptcache_amd/_blocks.py.
 *
 * Conventions: every entry point returns PCB_OK or a negative code (pcb_last_error_string() says why), validates its arguments
 * on the host before it launches anything, launches on `stream` (a hipStream_t) without synchronising, and takes device
 * pointers unless a parameter says otherwise.  `dtype` selects the element type E of weights, activations and cached keys:
 * PCB_BF16 (products on the bf16 matrix cores, fp32 accumulation) or PCB_F32 (fp32 matrix cores: true 32-bit products).
 * Residual streams, norms, scores, softmax weights, router logits and reductions are fp32 in both.
 */
#ifndef PROMPTCACHE_BLOCKS_H
#define PROMPTCACHE_BLOCKS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PCB_ABI_VERSION 4
#define PCB_OK 0
#define PCB_ERR_ARG (-2001)
#define PCB_ERR_HIP_BASE (-3000)

#define PCB_BF16 0
#define PCB_F32 1

int pcb_version(void);
const char* pcb_last_error_string(void);

/* out[r][:] = fp32(table[ids[r]][:]) : the embedding rows as the first residual stream. */
int pcb_embed_rows(const void* table, int32_t dtype, const int32_t* ids, float* out, int32_t n_rows, int32_t width, int32_t vocab,
                   void* stream);

/* out[r][:] = scale * fp32(table[ids[r]][:]) : embedding rows times a constant (the product is taken in fp32). */
int pcb_embed_scaled_rows(const void* table, int32_t dtype, const int32_t* ids, float scale, float* out, int32_t n_rows, int32_t width,
                          int32_t vocab, void* stream);

/* Weighted sum of residual streams + up to two RMS norms of the result, one workgroup per row:
 *   x[r]    = n_terms > 0 ? sum_j coef[j] * hist[j][src(r)] : hist[0][src(r)]       src(r) = rows ? rows[r] : r
 *   out1[r] = x[r] / sqrt(mean(x[r]^2) + eps) * gain1                               (E; likewise out2 with gain2 when given)
 * x_out (fp32 [n_rows][width]) receives x when given. */
typedef struct pcb_mix_norm_args {
    uint32_t struct_bytes;
    int32_t dtype;
    const float* hist;
    int64_t hist_stride; /* elements between stream j and stream j + 1 */
    const float* coef;
    int32_t n_terms;
    float* x_out;
    const int32_t* rows;
    const float* gain1;
    void* out1;
    const float* gain2;
    void* out2;
    float eps;
    int32_t n_rows;
    int32_t width;
} pcb_mix_norm_args;
int pcb_mix_norm(const pcb_mix_norm_args* a, void* stream);

/* Y = A W^T (+ bias), A = gathered / scaled rows of X.  W is [N][K] row-major (nn.Linear layout).
 *
 * rows      A row r = row_scale[r] * X[row_src ? row_src[r] : r]   (the scaled row is rounded to E)
 * groups    n_groups > 0: rows [group_off[g], group_off[g+1]) use W + g * w_group_stride (and W2 likewise); M is then an upper
 *           bound of group_off[n_groups] (the launch covers it; the kernel reads the offsets)
 * epilogue  PCB_EPI_STORE      v = acc + bias[n]
 *           PCB_EPI_SILU_MUL   v = f(acc + bias[n]) * (acc2 + bias2[n]), acc2 = A W2^T   (gated unit; f = SiLU, or `act` when it is
 *                              PCB_ACT_RELU / PCB_ACT_GELU_TANH / PCB_ACT_SILU; both biases optional)
 *           PCB_EPI_SCALE_ADD  v = (base ? base[m][n] : y32[m][n]) + col_scale[n] * (acc + bias[n]), stored fp32 (ldy)
 * output    STORE / SILU_MUL: element type E, or fp32 when out_f32; row m goes to y + (row_dst ? row_dst[m] : m) * ldy.
 *           split_n > 0 (STORE only): columns n >= split_n go to y2 instead: row m at y2 + row_off2[m], column c = n - split_n at
 *           (c / head_dim2) * head_stride2 + c % head_dim2  (a projection that appends its second part to a key cache). */
#define PCB_EPI_STORE 0
#define PCB_EPI_SILU_MUL 1
#define PCB_EPI_SCALE_ADD 2
/* element-wise function of a STORE epilogue: z, z sigmoid(z), sigmoid(z), max(z, 0)^2, ln(1 + e^z), cap tanh(z / cap), ... */
#define PCB_ACT_NONE 0
#define PCB_ACT_SILU 1
#define PCB_ACT_SIGMOID 2
#define PCB_ACT_RELU2 3
#define PCB_ACT_SOFTPLUS 4
#define PCB_ACT_SOFTCAP 5
#define PCB_ACT_RELU 6      /* max(z, 0) */
#define PCB_ACT_GELU_TANH 7 /* 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))) */
#define PCB_ACT_LOGSIGMOID 8 /* act_param * ln(sigmoid(z)): the logarithm of a decay sigmoid(z)^act_param */
#define PCB_ACT_SCALE 9      /* act_param * z */
typedef struct pcb_linear_args {
    uint32_t struct_bytes;
    int32_t dtype;
    int32_t epilogue;
    const void* x;
    int64_t ldx;
    const int32_t* row_src;
    const float* row_scale;
    const void* w;
    const void* w2;
    int64_t ldw;
    const void* bias; /* [N] E, may be null */
    int32_t M, N, K;
    const int32_t* group_off;
    int32_t n_groups;
    int64_t w_group_stride;
    void* y;
    int64_t ldy;
    int32_t out_f32;
    const int32_t* row_dst;
    const float* base;
    int64_t ldbase;
    const float* col_scale; /* [N] fp32 */
    int32_t split_n;
    void* y2;
    const int64_t* row_off2;
    int32_t head_dim2;
    int64_t head_stride2;
    int32_t split_n3;  /* > 0 (STORE only): columns n >= split_n3 go to y3 instead, one element per (row, column) with the ROW index
                          running fastest in memory: row m, column c = n - split_n3 at y3 + row_off3[m] + c * col_stride3 (a projection
                          that appends its last part to a cache kept column by column) */
    void* y3;
    const int64_t* row_off3;
    int64_t col_stride3;
    int32_t act;       /* PCB_ACT_*: STORE only, applied to acc + bias before the store (not to the columns split off to y2 / y3) */
    int32_t act_split; /* > 0: columns n >= act_split take act2 instead of act */
    int32_t act2;
    float act_param;   /* PCB_ACT_SOFTCAP: the cap; PCB_ACT_LOGSIGMOID, PCB_ACT_SCALE: the factor (it serves act and act2 alike) */
    const void* bias2; /* [N] E, may be null: the second product's bias of the gated epilogue */
} pcb_linear_args;
int pcb_linear(const pcb_linear_args* a, void* stream);

/* out[r][f] = c0 * z/rms(z) + c1 * z^2/rms(z^2) + c2 * z^3/rms(z^3) + c3 over row r of z (fp32 [n_rows][ff]), rms with eps inside the
 * root; coef = {c0, c1, c2, c3} fp32 on the device; out is E. */
int pcb_polynorm(const float* z, const float* coef, void* out, int32_t dtype, float eps, int32_t n_rows, int32_t ff, void* stream);

/* Top-k choice of a sigmoid router: logits fp32 [n_rows][n_experts] (the router projection, e.g. pcb_linear with an fp32
 * destination), score = sigmoid(logit), the `top` largest scores win (ties: the lower index).  pair p = r * top + k: expert[p],
 * weight[p] = the score itself (not renormalised). */
int pcb_router_topk(const float* logits, int32_t n_rows, int32_t n_experts, int32_t top, int32_t* expert, float* weight, void* stream);

/* Bucket the pairs by expert: group_off[n_experts + 1], and per bucketed row its token (row_src), its pair (row_dst) and its
 * weight (row_scale).  One workgroup; n_pairs <= 1 << 20. */
int pcb_moe_plan(const int32_t* expert, const float* weight, int32_t n_pairs, int32_t top, int32_t n_experts, int32_t* group_off,
                 int32_t* row_src, int32_t* row_dst, float* row_scale, void* stream);

/* y[r][n] += col_scale[n] * sum_k pair_out[r * top + k][n]  (fixed order over k). */
int pcb_moe_combine(const float* pair_out, const float* col_scale, float* y, int32_t n_rows, int32_t width, int32_t top, void* stream);

/* Causal attention over a slot-addressed key cache whose values ARE the keys (one plane), with optional
 *   - linear distance bias: score_h -= slopes[h] * (i - j)
 *   - cross-head mixing of the biased scores before the softmax: score_h <- sum_g talk[h][g] * score_g
 *   - sliding window: key j is seen by query i iff 0 <= i - j < window (window <= 0: all earlier keys)
 *   - sink: one more term exp(0) in the softmax denominator that carries no value
 * Queries are flat rows; tile t = {slot, first query position, query rows (<= 16), first flat row} (int32 x 4, device).  The
 * cache holds key j of kv head g of slot s at cache + s * slot_stride + g * head_stride + j * head_dim and must already contain
 * the queries' own keys.  Query head h reads kv head h / (H / Hkv).  scratch: fp32 [n_tiles * 16][H][band] with
 * band = pcb_attn_talk_band(window, max_kv_len) (the distances a row can see, padded); out is E [rows][ldo], head h at column
 * h * head_dim. */
typedef struct pcb_attn_talk_args {
    uint32_t struct_bytes;
    int32_t dtype;
    const void* q;
    int64_t ldq;
    const int32_t* tiles;
    int32_t n_tiles;
    const void* cache;
    int64_t slot_stride;
    int64_t head_stride;
    int32_t H, Hkv, head_dim;
    float scale;
    int32_t window;
    int32_t max_kv_len; /* no tile reaches a key position >= this */
    const float* slopes; /* [H] or null */
    const float* talk;   /* [H][H] or null */
    int32_t sink;
    float* scratch;
    int64_t scratch_floats;
    void* out;
    int64_t ldo;
    const int32_t* tiles64; /* optional: the same rows cut into tiles of up to 64 queries (same record) for the value pass */
    int32_t n_tiles64;
    int32_t max_tile_rows; /* an upper bound of the tiles' query rows when the host knows one (0: unknown); <= 4 selects the
                              value pass written for decoding */
} pcb_attn_talk_args;
int32_t pcb_attn_talk_band(int32_t window, int32_t max_kv_len);
int pcb_attn_talk(const pcb_attn_talk_args* a, void* stream);

/* ---- residual streams, norms, routers of designs with several residual streams --------------------------------------------- */

/* out[s][r][:] = fp32(table[ids[r]]) + fp32(pos_table[positions[r]]) for every stream s < n_streams (pos_table null: no
 * position term).  out is fp32 [n_streams][.. stream_stride ..]. */
int pcb_embed_pos_rows(const void* table, const void* pos_table, int32_t dtype, const int32_t* ids, const int32_t* positions,
                       float* out, int64_t stream_stride, int32_t n_streams, int32_t n_rows, int32_t width, int32_t vocab,
                       int32_t max_positions, void* stream);

/* Hyper-connection step around a sublayer, one workgroup per row, in two optional halves:
 *   write (y given):   x_t <- sum_s mix[s][t] x_s + out_w[t] * y[src]        all streams t at once from the old ones, in place
 *                      (with `rows` the new streams are used but not written back)
 *   read (out given):  u = sum_s in_w[s] x_s  (in_w null: the plain sum),  out[r] = norm(u) as E,  x_out[r] = u (fp32) if given
 * norm: PCB_NORM_NONE u; PCB_NORM_RMS u / sqrt(mean(u^2) + eps) * gain; PCB_NORM_DYT tanh(alpha[0] * u) * gain + bias.
 * src = rows ? rows[r] : r.  n_streams <= 8. */
#define PCB_NORM_NONE 0
#define PCB_NORM_RMS 1
#define PCB_NORM_DYT 2
typedef struct pcb_hyper_norm_args {
    uint32_t struct_bytes;
    int32_t dtype;
    float* streams;
    int64_t stream_stride;
    int32_t n_streams;
    const float* y; /* fp32 [rows][width] */
    const float* mix;   /* [S][S], indexed [from][to] */
    const float* out_w; /* [S] */
    const float* in_w;  /* [S] or null */
    int32_t norm;
    const float* gain;
    const float* bias;
    const float* alpha; /* one float on the device */
    float eps;
    void* out;
    float* x_out;
    const int32_t* rows;
    int32_t n_rows;
    int32_t width;
} pcb_hyper_norm_args;
int pcb_hyper_norm(const pcb_hyper_norm_args* a, void* stream);

/* out[r][c] = E( (gain ? x[r][c] / sqrt(mean x[r]^2 + eps) * gain[c] : x[r][c]) * (gate ? gate[r][c] : 1) ), x fp32 [n_rows][ldx],
 * gate E [n_rows][ldg], out E [n_rows][ldo]: a unit norm with an element-wise gate.  The mean runs over all `cols` columns
 * (group_cols <= 0: one norm over all heads' outputs) or over each run of group_cols columns by itself (a norm per head;
 * group_cols divides cols; then the norm is taken with or without a gain).
 * skip (E [n_rows][lds], optional): x[r][c] + skip_w[c / skip_group] * skip[r][c] stands for x[r][c] (a skip path with one weight per
 * head).  gate_first: the gate is applied BEFORE the norm, out = norm(x * gate) * gain. */
int pcb_gated_norm(const float* x, int64_t ldx, const float* gain, const void* gate, int64_t ldg, void* out, int64_t ldo,
                   int32_t dtype, float eps, int32_t n_rows, int32_t cols, int32_t group_cols, int32_t gate_first, const void* skip,
                   int64_t lds, const float* skip_w, int32_t skip_group, void* stream);

/* Router choice over n_out outputs per row (logits fp32 [n_rows][n_out]):
 *   score s = score_fn == PCB_SCORE_SOFTMAX ? softmax(logits) : sigmoid(logits);  choice score = s + correction (if given)
 *   groups > 1: outputs form `groups` equal runs of neighbours; a group's score is its largest choice score; only outputs of
 *   the groups_keep best groups can be chosen
 *   the `top` largest choice scores win (ties: the lower index); weight = s (without the correction), divided by the sum of
 *   the chosen weights + 1e-20 when renorm.  pair p = r * top + k: expert[p], weight[p].  n_out <= 2048, groups <= 64. */
#define PCB_SCORE_SIGMOID 0
#define PCB_SCORE_SOFTMAX 1
int pcb_router_select(const float* logits, int32_t n_rows, int32_t n_out, int32_t top, int32_t score_fn, const float* correction,
                      int32_t groups, int32_t groups_keep, int32_t renorm, int32_t* expert, float* weight, void* stream);

/* y[r][:] = sum_k weight[p] * (expert[p] >= n_real ? h[r][:] : pair_out[p][:]),  p = r * top + k  (fixed order over k):
 * the weighted sum of a token's experts' results, identity experts (index >= n_real) standing for the token's own input h
 * (E [n_rows][width]).  y fp32 [n_rows][width] is overwritten. */
int pcb_moe_mix(const float* pair_out, const int32_t* expert, const float* weight, const void* h, int32_t dtype, int32_t n_real,
                float* y, int32_t n_rows, int32_t width, int32_t top, void* stream);

/* ---- mixers ------------------------------------------------------------------------------------------------------------------- */

/* Causal softmax attention over a slot-addressed cache with separate keys and values.
 * Queries are flat rows; tile t = {slot, first query position, query rows (<= 16), first flat row} (int32 x 4, device).
 * Key j of kv head g of slot s: kcache + s * slot_stride + g * head_stride + j * row_stride (dim elements).  Its value: row by row
 * like the keys (v_cols = 0: vcache + s * v_slot_stride + g * v_head_stride + j * v_stride, vdim elements -- keys and values may
 * interleave in one plane), or column by column (v_cols = 1: column c of key j at vcache + s * v_slot_stride + g * v_head_stride +
 * c * v_stride + j; every column must be readable up to the next multiple of 32 keys, and v_stride a multiple of 8), which lets
 * the value operand of the matrix cores be read with wide loads.  The cache already holds the queries' own keys and values.  score = q_scale[row] * scale * q.k (q_scale null: 1); key j is seen by the query at position i iff j <= i and
 * (window <= 0 or i - j < window or j < keep_first) and (block <= 0 or floor(i / block) == floor(j / block): blocks of positions counted from 0, a
 * key is seen inside the query's own block only).  sink (fp32 [H], optional): the softmax denominator of head h also holds
 * exp(sink[h]) -- a term without key or value, not scaled.  The result (E [rows][ldo], head h at column h * vdim) is multiplied by
 * a gate when given (E, row stride ldg): element-wise gate[row][h * vdim + c], or one number per head gate[row][h] when
 * gate_per_head.  dim <= 384, vdim <= 256. */
typedef struct pcb_attn_softmax_args {
    uint32_t struct_bytes;
    int32_t dtype;
    const void* q;
    int64_t ldq;
    const float* q_scale;
    const int32_t* tiles;
    int32_t n_tiles;
    const void* kcache;
    const void* vcache;
    int64_t slot_stride, head_stride, row_stride;
    int64_t v_slot_stride, v_head_stride, v_stride;
    int32_t v_cols;
    int32_t H, Hkv, dim, vdim;
    float scale;
    int32_t window;
    const void* gate;
    int64_t ldg;
    void* out;
    int64_t ldo;
    int32_t n_splits; /* > 1: every (tile, head) is cut into n_splits runs of key blocks that run as workgroups of their own and
                         leave (maximum, denominator, weighted values) in `part`; a second launch merges them.  For steps of few
                         rows over long caches. */
    float* part;      /* fp32 [rows][H][n_splits][vdim + 2], rows = the flat rows the tiles cover (row index = flat row) */
    int32_t block;
    const float* sink;
    int32_t gate_per_head;
    int32_t head_rows; /* 1: every tile has ONE row and there is one key head (Hkv = 1): a workgroup takes 16 heads of that row at once
                          (the heads read the same keys and values) -- for decoding over a shared latent */
    int32_t keep_first; /* > 0 (with a window): keys at positions < keep_first stay visible to every later query, at their true
                           positions (the sequence's first tokens are kept behind the sliding window) */
} pcb_attn_softmax_args;
int pcb_attn_softmax(const pcb_attn_softmax_args* a, void* stream);

/* Linear attention with one scalar decay per head and a matrix state per (slot, head):
 *   S_t = decay[h] * S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t        (S: [dim][vdim], fp32, zero before position 0)
 * q, k: E rows with head h at column h * dim; v: head h at column h * vdim; out fp32 [rows][ldo].  request r = {slot, first
 * position, tokens, first flat row} (int32 x 4, device): its tokens are consecutive rows; a request that starts at position 0
 * starts from a zero state whatever the slot held.  state: fp32 [slots][H][dim][vdim] (slot_stride floats per slot), read at the
 * start and written at the end of each request.  All products run on the fp32 matrix cores.  dim <= 256.
 * out null: only the states move (the first pass of a segmented prefill, see pcb_state_chain). */
typedef struct pcb_decay_attn_args {
    uint32_t struct_bytes;
    int32_t dtype;
    const void* q;
    const void* k;
    const void* v;
    int64_t ldq, ldk, ldv;
    const int32_t* reqs;
    int32_t n_reqs;
    float* state;
    int64_t slot_stride;
    const float* decay;
    int32_t H, dim, vdim;
    float* out;
    int64_t ldo;
} pcb_decay_attn_args;
int pcb_decay_attn(const pcb_decay_attn_args* a, void* stream);

/* Causal per-channel convolution of `taps` taps (the last tap is the current token's) with bias and optional SiLU:
 *   out[r][c] = act( bias[c] + sum_j w[c][j] * in(pos(r) - (taps - 1) + j)[c] ),  in(p) = 0 for p < 0
 * row_meta[r] = {slot, position, index of the row among its request's rows of this step, 0}: inputs older than the step come from
 * state (E [slots][taps - 1][C]: the last taps - 1 inputs of the slot).  pcb_conv_state_update then moves the state behind the
 * step's rows (reqs as in pcb_decay_attn); it must run after pcb_causal_conv of the same step.  taps <= 16. */
int pcb_causal_conv(const void* x, int64_t ldx, const void* w, const void* bias, int32_t dtype, int32_t silu, const int32_t* row_meta,
                    const void* state, int64_t slot_stride, void* out, int64_t ldo, int32_t n_rows, int32_t C, int32_t taps,
                    void* stream);
int pcb_conv_state_update(const void* x, int64_t ldx, int32_t dtype, const int32_t* reqs, int32_t n_reqs, void* state,
                          int64_t slot_stride, int32_t C, int32_t taps, void* stream);

/* Selective scan (one state vector of N floats per channel):
 *   S[c][n] <- exp(dt[c] * A[c][n]) * S[c][n] + dt[c] * x[c] * B[n],   y[c] = sum_n S[c][n] * Cm[n] + D[c] * x[c],
 *   out[c] = y[c] * silu(z[c])   (z null: out = y)
 * per token, in order, for each request {slot, first position, tokens, first flat row}.  x, z: E rows; dt, B, Cm: fp32 rows;
 * A fp32 [C][N], D fp32 [C]; state fp32 [slots][C][N] (zero before position 0); out E.  N <= 256.
 * out null: only the states move; dt_sum (fp32 [n_reqs][C], optional) receives each request's sum of dt per channel. */
typedef struct pcb_selective_scan_args {
    uint32_t struct_bytes;
    int32_t dtype;
    const void* x;
    int64_t ldx;
    const float* dt;
    int64_t lddt;
    const float* B;
    const float* Cm;
    int64_t ldbc;
    const void* z;
    int64_t ldz;
    const float* A;
    const float* D;
    const int32_t* reqs;
    int32_t n_reqs;
    float* state;
    int64_t slot_stride;
    int32_t C, N;
    void* out;
    int64_t ldo;
    float* dt_sum;
} pcb_selective_scan_args;
int pcb_selective_scan(const pcb_selective_scan_args* a, void* stream);

/* Segmented prefill of a linear recurrence S <- f S + (input term), f = exp(coef * x): a long sequence is cut into segments, a
 * first pass runs every segment from a ZERO state (local[g] = its own contribution), this call chains them, and a second pass runs
 * every segment from its true start state.  For chain c = {slot, first position, first segment, segments} (int32 x 4), element-wise
 * over `elems` floats e:
 *   s = first position > 0 ? state[slot][e] : 0
 *   for g = first segment ..:   start[g][e] = s;   s = exp(coef[e] * x[g][e / group]) * s + local[g][e]
 *   state[slot][e] = s
 * local, start: fp32 [segments][elems]; coef fp32 [elems]; x fp32 [segments][elems / group]. */
int pcb_state_chain(const float* local, float* start, float* state, int64_t slot_stride, const int32_t* chains, int32_t n_chains,
                    const float* coef, const float* x, int32_t elems, int32_t group, void* stream);

/* ---- sublayers between two norms, per-head preparation of queries / keys / values, matrix memories ------------------------------ */

/* A residual step with a norm after the sublayer and the norm before the next one, one workgroup per row, in two optional halves:
 *   write (y given):  t = y[src] * (gate ? gate[src] : 1);  x[src] += post_gain ? t / sqrt(mean(t^2) + eps) * post_gain : t
 *                     (with `rows` the sum is used but not written back)
 *   read (out given): out[r] = x[src] / sqrt(mean(x[src]^2) + eps) * gain as E;  x_out[r] = x[src] (fp32) if given
 *                     layer_norm: out[r] = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * gain + bias instead
 * y_scale: the sublayer's result enters as y_scale * y (after gate and post norm; 1 = as it is).
 * src = rows ? rows[r] : r.  y fp32 [..][width]; gate E rows of stride ldg; x fp32 [..][width].  width <= 16384. */
typedef struct pcb_post_norm_args {
    uint32_t struct_bytes;
    int32_t dtype;
    float* x;
    const float* y;
    const void* gate;
    int64_t ldg;
    const float* post_gain;
    const float* gain;
    void* out;
    float* x_out;
    const int32_t* rows;
    float eps;
    int32_t n_rows;
    int32_t width;
    float y_scale;
    int32_t layer_norm;
    const float* bias; /* [width] fp32, layer_norm only (null: none) */
} pcb_post_norm_args;
int pcb_post_norm(const pcb_post_norm_args* a, void* stream);

/* Per-head preparation of projected rows: up to four segments (queries, keys, values, ...) of one launch, each `heads` heads of
 * head_dim columns read from E rows (src + row * ld_src + h * src_head_stride).  Per head, in this order, all in fp32:
 *   norm:   x <- x / sqrt(mean(x^2) + eps)  (norm != 0), times gain[c] when given
 *   blend:  x <- (1 - blend[0]) x + blend[0] * other[row][h * head_dim + c]      (other fp32, blend one float on the device)
 *   keep:   keep[row][h * head_dim + c] = x                                       (fp32: what a later launch blends with)
 *   rotate: columns rot_off + 2i, rot_off + 2i + 1 (i < rot_dims / 2) turn by the angle pos[row] * freqs[i]:
 *           (u, v) <- rot_mag * (u cos - v sin, v cos + u sin); the angle is a float64 product, other columns pass unchanged
 *   store:  E at dst + (row_off ? row_off[row] : row * ld_dst) + h * head_stride + c * col_stride  (rows of a matrix, a cache kept
 *           row by row, or one kept column by column)
 * freqs: float64 [rot_dims / 2] on the device, shared by the segments that rotate (they have the same rot_dims).  head_dim <= 1024. */
typedef struct pcb_head_prep_seg {
    const void* src;
    int64_t ld_src;
    int64_t src_head_stride;
    int32_t heads, head_dim;
    int32_t norm;
    const float* gain;
    const float* blend;
    const float* other;
    int64_t ld_other;
    float* keep;
    int64_t ld_keep;
    int32_t rot_off, rot_dims;
    void* dst;
    int64_t ld_dst;
    const int64_t* row_off;
    int64_t head_stride, col_stride;
} pcb_head_prep_seg;
typedef struct pcb_head_prep_args {
    uint32_t struct_bytes;
    int32_t dtype;
    int32_t n_rows;
    int32_t n_segs;
    const int32_t* pos;
    const double* freqs;
    float rot_mag;
    float eps;
    pcb_head_prep_seg seg[4];
} pcb_head_prep_args;
int pcb_head_prep(const pcb_head_prep_args* a, void* stream);

/* Matrix memory with exponential gating (mLSTM): per (slot, head) a state S [dim][vdim], a normaliser n [dim] and a running
 * maximum m, all fp32, zero before position 0.  Per token, with the head's log input gate li and log forget gate lf:
 *   li = cap(gi),  lf = logsigmoid(cap(gf)),  cap(z) = gate_cap > 0 ? gate_cap tanh(z / gate_cap) : z
 *   m' = max(lf + m, li);  S' = exp(lf + m - m') S + exp(li - m') k v^T;  n' = exp(lf + m - m') n + exp(li - m') k
 *   o = S'^T (q_scale q) / (max(|n' . q_scale q|, exp(-m')) + 1e-6)
 * q, k: E rows, head h at column h * dim; v: head h at column h * vdim; gi, gf: E rows, one column per head (the gates'
 * pre-activations, bias included); out fp32 [rows][ldo].  request r = {slot, first position, tokens, first flat row} as in
 * pcb_decay_attn.  state: fp32 per slot [H][dim * vdim + dim + 1] (S, then n, then m), slot_stride floats apart.
 * out null: only the states move.  from_nothing: every request starts from S = n = 0 and m = -infinity whatever its position
 * says (a segment's own contribution, see pcb_mlstm_chain); log_f_sum (fp32 [n_reqs][H], optional) receives each request's sum
 * of log forget gates.  end_slots (int32 [n_reqs], optional): request r with end_slots[r] >= 0 leaves its last state in
 * end_state + end_slots[r] * end_slot_stride instead of its own record (the last segment of a prompt writes the slot's state). */
typedef struct pcb_mlstm_args {
    uint32_t struct_bytes;
    int32_t dtype;
    const void* q;
    const void* k;
    const void* v;
    const void* gi;
    const void* gf;
    int64_t ldq, ldk, ldv, ldgi, ldgf;
    const int32_t* reqs;
    int32_t n_reqs;
    float* state;
    int64_t slot_stride;
    int32_t H, dim, vdim;
    float q_scale;
    float gate_cap;
    float* out;
    int64_t ldo;
    int32_t from_nothing;
    float* log_f_sum;
    const int32_t* end_slots;
    float* end_state;
    int64_t end_slot_stride;
} pcb_mlstm_args;
int pcb_mlstm(const pcb_mlstm_args* a, void* stream);

/* Segmented prefill of the matrix memory: a first pcb_mlstm pass runs every segment from nothing (local[g] = its contribution,
 * log_f_sum[g] = its sum of log forget gates, both per head), this call chains them, and a second pass runs every segment from its
 * true start state.  For chain c = {slot, first position, first segment, segments} (int32 x 4) and every head, with records
 * (S, n, m) of dim * vdim + dim + 1 floats:
 *   (S, n, m) = first position > 0 ? state[slot] : (0, 0, 0)
 *   for g = first segment ..:  start[g] = (S, n, m);  m' = max(F_g + m, m_g);
 *                              S <- exp(F_g + m - m') S + exp(m_g - m') S_g;  n likewise;  m <- m'
 * local, start: fp32 [segments][H][record]; state is only read. */
int pcb_mlstm_chain(const float* local, const float* log_f_sum, float* start, const float* state, int64_t slot_stride, const int32_t* chains,
                    int32_t n_chains, int32_t H, int32_t dim, int32_t vdim, void* stream);

/* Linear attention whose decay changes from token to token, with a matrix state per (slot, head):
 *   S_t = diag(exp(l_t)) S_(t-1) + k_t (s_t v_t)^T,   o_t = S_t^T (q_scale q_t)        (S: [dim][vdim], fp32, zero before position 0)
 * l_t = ld_coef[h] * ld[row][h * dcols + (dcols == 1 ? 0 : d)] is the log decay of key row d (ld_coef null: 1): dcols = dim gives every
 * key channel its own decay (gated linear attention), dcols = 1 one decay per head and token (the matrix form of a selective
 * scan with scalar decays: k = B, q = C, v = x, s = the step size, l = -rate * step size).  s_t = v_scale[row][h] (null: 1).
 * q, k: E rows with head h / (H / Hk) at column (h / (H / Hk)) * dim (Hk heads of queries and keys serve H heads of values);
 * v: head h at column h * vdim; ld, v_scale: fp32 rows; out fp32 [rows][ldo].  request r = {slot, first position, tokens, first
 * flat row} as in pcb_decay_attn; state fp32 [slots][H][dim][vdim].  Decays, step sizes and every product that feeds a state are
 * fp32.  dim <= 256.
 * out null: only the states move (the first pass of a segmented prefill); ld_sum (fp32 [n_reqs][H * dcols], optional) receives each
 * request's sum of log decays, which is what pcb_state_chain needs (coef = 1, group = vdim or dim * vdim). */
typedef struct pcb_gla_args {
    uint32_t struct_bytes;
    int32_t dtype;
    const void* q;
    const void* k;
    const void* v;
    int64_t ldq, ldk, ldv;
    const float* ld;
    int64_t ldld;
    int32_t dcols;
    const float* ld_coef;
    const float* v_scale;
    int64_t ldvs;
    const int32_t* reqs;
    int32_t n_reqs;
    float* state;
    int64_t slot_stride;
    int32_t H, Hk, dim, vdim;
    float q_scale;
    float* out;
    int64_t ldo;
    float* ld_sum;
} pcb_gla_args;
int pcb_gla(const pcb_gla_args* a, void* stream);

#ifdef __cplusplus
}
#endif
#endif
