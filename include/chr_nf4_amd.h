/* C ABI of the MI355X (gfx950) NF4 packed-linear library, libchr_nf4_amd.so.
 *
 * Every entry point below replaces the reference entry point of the same name;
 * the citation after each one is the reference declaration (gpu/include/chr_gpu.h)
 * and definition it stands in for.  Struct layouts are the reference's, field for
 * field, so a binding written against chr_gpu.h binds this library unchanged.
 *
 * Conventions shared by all calls
 *   - plain pointers and sizes only; every buffer is caller-owned device memory;
 *     nothing here allocates, frees or synchronises
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream)
 *   - activations are bfloat16 bits, scales are IEEE binary16 bits
 *   - return 0 on success, else
 *       -1 null pointer            -5 packed or x not 16-byte aligned
 *       -2 N out of range             (scale not 2-byte aligned)
 *       -3 bad dims / null blobs   -6 launch failure
 *       -4 K_pad != 64*ceil(K/64)  -7 split-K workspace too small
 *       -8 a sum-of-squares hand-over (chr_dv2_*_sumsq) this launch cannot serve
 *     (chr_gpu.h:30-33; gpu/nf4/nf4_gemm.cu:1621-1644, 1683-1698)
 *
 * Naming follows the reference: M = out features, K = in features,
 * N = token columns; y[M,N] = dequant(W[M,K]) @ x[K,N].
 */
#pragma once

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Weight descriptor (chr_gpu.h:11-17).  packed is [M, K_pad/2] row-major, low
 * nibble = even column; scale is [M, K_pad/64] binary16 bits. */
typedef struct {
  int32_t M;
  int32_t K;
  int32_t K_pad;
  const uint8_t *packed;
  const uint16_t *scale;
} chr_nf4_dev_t;

/* Launch plan (chr_gpu.h:48-60).  Same fields and meaning; the numbers describe
 * this library's gfx950 tiles, not the reference's sm_86 ones.
 * path: 1 = N==1 row-streaming GEMV tile, 2 = MFMA tile for N<=16,
 *       3 = MFMA tile for N<=32, 4 = MFMA tile for N<=64 (plan only). */
typedef struct {
  int32_t path;
  int32_t grid_x;          /* ceil(M / bm) */
  int32_t grid_y;          /* split_k */
  int32_t block;           /* threads per workgroup */
  int32_t bm;              /* rows of M per workgroup */
  int32_t bk;              /* K per staged tile */
  int32_t n_ktiles;        /* ceil(K_pad / bk) */
  int32_t tiles_per_split; /* K tiles one workgroup walks */
  int32_t ctas;            /* grid_x * grid_y */
  int32_t smem_bytes;      /* LDS bytes per workgroup */
  int64_t ws_floats;       /* FP32 partials; 0 when grid_y == 1 */
} chr_nf4_plan_t;

/* y[M,N] = dequant(W) @ x[K,N]; x and y are bf16 row-major (token index
 * fastest).  N in [1, 32].  No workspace, so split_k == 1.
 * Replaces chr_nf4_gemm (chr_gpu.h:34-35; nf4_gemm.cu:1779-1785). */
int chr_nf4_gemm(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                 void *stream);

/* Pure launch math; only M/K/K_pad are read.  N in [1, 64].
 * Chunks of 8, 16, 24, 32 or exactly 64 columns with K_pad a multiple of 256 can run the tile
 * whose workgroups finish their rows themselves (block 1024; bm 32 or 64 rows a workgroup;
 * grid_y workgroups share a row block's K in 512-wide chunks, at most 12 each -- 256-wide and
 * at most 20 at 64 columns, where tiles_per_split counts those -- and the last of them
 * to finish adds their fp32 partials up in split order: ws_floats = grid_y * M * N when
 * grid_y > 1, no reduce launch).  The planner takes it where its cost model prefers it to
 * the split tiles (at 14B shapes: all of them); chr_nf4_gemm_stream_policy and
 * CHR_NF4_GEMM_STREAM (0 never, 2 wherever it fits) change that, a forced split
 * (chr_nf4_set_tuning) or a scale blob that is not 8-byte aligned keep a launch on the split
 * tiles.  It multiplies bf16(level) and applies the fp16 scale to each 64-wide group's sum,
 * where the other tiles multiply bf16(level * scale) as the reference's kernel does.
 * Replaces chr_nf4_gemm_plan (chr_gpu.h:64-65; nf4_gemm.cu:1656-1667). */
int chr_nf4_gemm_plan(const chr_nf4_dev_t *w, int32_t N, int32_t have_ws,
                      chr_nf4_plan_t *out);

/* As chr_nf4_gemm with a caller-owned FP32 workspace of at least
 * plan.ws_floats floats (ws == NULL means "no split-K").  N in [1, 32].
 * Replaces chr_nf4_gemm_ws (chr_gpu.h:70-71; nf4_gemm.cu:1773-1777). */
int chr_nf4_gemm_ws(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                    float *ws, int64_t ws_floats, void *stream);

/* Same launch with the column ceiling given by the caller: max_n is clamped to
 * [1, 64] and N > max_n is refused with -2.  Chunks of 33..64 columns run the
 * 64-column tile (the reference plans that width but never launches it).
 * Replaces chr_nf4_gemm_ws_max (chr_gpu.h:75-76; nf4_gemm.cu:1669-1771). */
int chr_nf4_gemm_ws_max(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                        float *ws, int64_t ws_floats, void *stream, int32_t max_n);

/* chr_nf4_gemm_ws without a workspace argument and without any allocation: the
 * split-K partials go to a device array owned by the library (16 MiB of fp32 on
 * every GPU it runs on, held until the process ends).  N in [1, 32].  Returns
 * what chr_nf4_gemm_ws returns for a workspace of
 * chr_nf4_gemm_noalloc_max_floats() floats, bit for bit; a launch whose
 * partials need more comes back as -7 and nothing runs.  All calls on one GPU
 * share the array: calls that overlap on that GPU (two streams, two threads)
 * race.  The first call on a device looks the array's address up and must not
 * be made under graph capture; later ones can.
 * No counterpart in the reference: for callers that cannot allocate (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). */
int chr_nf4_gemm_noalloc(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                         void *stream);
int64_t chr_nf4_gemm_noalloc_max_floats(void);

/* Process-wide planner override: path 0 auto; split_k 0 auto, >0 forced;
 * one_wave = compute units the split-K target is expressed in, 0 = this GPU's.
 * Initial values come from CHR_NF4_PATH / CHR_NF4_SPLIT_K / CHR_NF4_ONE_WAVE.
 * Replaces chr_nf4_set_tuning (chr_gpu.h:84; nf4_gemm.cu:1648-1654). */
void chr_nf4_set_tuning(int32_t path, int32_t split_k, int32_t one_wave);

/* Which prefill launches run the tile whose workgroups finish their rows themselves:
 * 0 where the planner's cost model prefers it (the default), > 0 wherever it fits, < 0 never.
 * Process-wide, like chr_nf4_set_tuning.  Launches of that tile that split K count their
 * arrivals in a table the library owns: one row per stream for eager launches, one row per
 * capture and stream for launches recorded into a graph (so a graph may be replayed on any
 * stream, beside eager launches on the stream it was captured from and beside other graphs),
 * none for the per-thread default stream; when the 512 rows are taken, and on that stream,
 * the splits meet in a reduce launch instead (same bits).  What the caller must not do is
 * replay one executable graph concurrently with itself, which the HIP runtime orders anyway.
 * No counterpart in the reference. */
void chr_nf4_gemm_stream_policy(int32_t policy);

/* N=1 GEMV.  x bf16 [K], y bf16 [M].  add: optional bf16 [M] residual, may
 * alias y.  rms_w: optional bf16 [K]; when set, RMSNorm(x, rms_w, rms_eps),
 * rounded to bf16, is what the dots consume.
 * Arithmetic: fp32 accumulation, one bf16 rounding of y.  Launches of fewer than 16M codes
 * multiply fp32 levels (as nf4_gemv.cu:70-101); launches from 16M codes up, and every
 * launch with rms_w or K != K_pad, stage x in LDS (K_pad * 2.25 <= 85 KB; -6 when rms_w or a
 * ragged K require it and it does not fit) and multiply the levels in the form
 * CHR_NF4_GEMV_TERMS names: 3 or unset, levels rounded to binary16 (2^-12 relative) against x
 * held as binary16, every 16 consecutive activations times a power of two of their own (exact
 * for every bf16 element within 2^-29 of the largest of its 16); 2, levels as two bf16 terms
 * (below 2^-17); 1, levels rounded to bf16 (2^-9, the
 * precision of the reference's tensor-core path, nf4_gemm.cu:322).  CHR_NF4_GEMV_STAGED=0|1
 * in the environment forces either kernel family where both are possible.
 * Replaces chr_nf4_gemv (chr_gpu.h:92-93; nf4_gemv.cu:790-834). */
int chr_nf4_gemv(const chr_nf4_dev_t *w, const void *x, void *y, void *stream,
                 const void *add, const void *rms_w, float rms_eps);

/* One launch over q.M + k.M + v.M rows sharing x; optional bf16 biases are
 * added in fp32 before the single bf16 rounding.
 * Replaces chr_nf4_gemv_qkv (chr_gpu.h:99-103; nf4_gemv.cu:836-874). */
int chr_nf4_gemv_qkv(const chr_nf4_dev_t *q, const chr_nf4_dev_t *k,
                     const chr_nf4_dev_t *v, const void *x, void *yq, void *yk,
                     void *yv, const void *bq, const void *bk, const void *bv,
                     void *stream, const void *rms_w, float rms_eps);

/* y[r] = bf16( silu(gate_r . x) * (up_r . x) ), both dots kept in fp32.
 * Replaces chr_nf4_gemv_swiglu (chr_gpu.h:108-110; nf4_gemv.cu:876-924). */
int chr_nf4_gemv_swiglu(const chr_nf4_dev_t *gate, const chr_nf4_dev_t *up,
                        const void *x, void *y, void *stream, const void *rms_w,
                        float rms_eps);

/* In-place rotate-half RoPE on q [n_q,hd] and k [n_kv,hd] (rounded to bf16),
 * then k and v are written to the caches [max_seq,n_kv,hd] at *position (int64).
 * Replaces chr_nf4_rope_kv (chr_gpu.h:115-118; nf4_gemv.cu:926-950). */
int chr_nf4_rope_kv(void *q, void *k, const void *v, void *k_cache, void *v_cache,
                    const void *cos, const void *sin, const void *position,
                    int32_t n_q, int32_t n_kv, int32_t hd, int32_t max_seq,
                    void *stream);

/* GQA decode attention over t < *valid_len (int32 on device).  With
 * k_act/v_act/cos/sin/position it also rotates q and the current k in fp32,
 * writes bf16(k_rot) and v into the caches at *position, and serves that slot
 * from registers.  ws: n_q*n_split*(hd+2) floats.  hd <= 256, n_split <= 64.
 * Replaces chr_nf4_attn (chr_gpu.h:124-128; nf4_gemv.cu:952-994). */
int chr_nf4_attn(const void *q, const void *k, const void *v, void *out,
                 const void *valid_len, float *ws, int32_t n_q, int32_t n_kv,
                 int32_t hd, int32_t n_split, float scale, void *stream,
                 const void *k_act, const void *v_act, const void *cos,
                 const void *sin, const void *position, int32_t max_seq);

/* y[i] = bf16( (w[i]*x[i]) * rsqrt(mean(x^2) + eps) ); x, w, y bf16 [n].
 * Replaces chr_nf4_rms (chr_gpu.h:131-132; nf4_gemv.cu:996-1011). */
int chr_nf4_rms(const void *x, const void *w, void *y, int32_t n, float eps,
                void *stream);

/* ---- entry points whose reference counterpart is not a C function ---------- */

/* out[M,K] fp32 = LUT[code] * f32(scale), one binary32 multiply per weight,
 * padding columns dropped.  Device twin of the CPU codec's Decode
 * (internal/nf4/nf4.go:85-121), used to prove bit-exact unpacking. */
int chr_nf4_dequant(const chr_nf4_dev_t *w, float *out, void *stream);

/* Decode rows ids[0..n) of a packed table to bf16 [n, K]:
 * bf16( LUT[code] * f32(scale) ).  ids are int64 on device.
 * Replaces dequant_nf4_rows (gpu/host/embedding.py:74-107), the embedding
 * gather of the decode step. */
int chr_nf4_embed_rows(const chr_nf4_dev_t *table, const void *ids, int32_t n,
                       void *out, void *stream);

/* Quantise src[M,K] fp32 (device) into dst->packed / dst->scale (device,
 * writable despite the const in the struct).  Device twin of the CPU codec's
 * Encode (internal/nf4/nf4.go:46-82,129-185), bit for bit, used to make
 * synthetic weights at model scale.  *status (int32 on device, may be NULL)
 * is OR-ed with 1 when a non-finite weight was met (its group is skipped). */
int chr_nf4_quantize(const float *src, const chr_nf4_dev_t *dst, int32_t *status,
                     void *stream);

/* valid_len (int32 on device) = *position (int64 on device) + 1.
 * Replaces GraphSafeKV.mark_written (gpu/decodev2/kv.py:118-120), three tensor
 * ops in the reference, one launch here. */
int chr_dv2_mark_written(const void *position, void *valid_len, void *stream);

/* *next_token = argmax over logits[0..n) (bf16; the lowest index wins a tie; a
 * NaN logit wins outright).  With commit != 0 it also feeds the id back:
 * *token = next, *position += 1, *finished |= (next == *eos_id); all scalars
 * live on the device (int64, int64, int64, uint8, int64).
 * Replaces the argmax of forward_decode plus DecodeState.commit_step
 * (gpu/decodev2/step.py:182, gpu/decodev2/state.py:98-103). */
int chr_dv2_argmax_commit(const void *logits, int32_t n, void *next_token, void *token,
                          void *position, void *finished, const void *eos_id, int32_t commit,
                          void *stream);

/* ---- decode step: fewer launches than the reference's call sequence.  These entry
 * points have no single counterpart in the reference; each computes what the cited
 * sequence of reference calls computes. */

/* valid_len = *position + 1; x = packed embedding row *token as bf16; and, when norm_w
 * is not NULL, h = RMSNorm(x, norm_w, eps).  One launch for GraphSafeKV.mark_written +
 * gather_embed (+ the first nf4_rms) of forward_decode (gpu/decodev2/step.py:165-172,
 * kv.py:118-120, gpu/host/embedding.py:74-107). */
int chr_dv2_begin_step(const chr_nf4_dev_t *table, const void *token, const void *position,
                       void *valid_len, void *x, const void *norm_w, float eps, void *h,
                       void *stream);

/* chr_nf4_attn as one launch: one workgroup of n_waves (1..16) wavefronts per query head,
 * each wavefront takes every n_waves-th cache row, the partial softmax states meet in
 * LDS and the workgroup writes the merged head.  No workspace.  Replaces the
 * attn_flash + attn_merge pair (gpu/nf4/nf4_gemv.cu:952-994) for contexts short enough
 * that n_q workgroups can stream the cache (a few thousand rows). */
int chr_dv2_attn(const void *q, const void *k, const void *v, void *out, const void *valid_len,
                 int32_t n_q, int32_t n_kv, int32_t hd, int32_t n_waves, float scale,
                 void *stream, const void *k_act, const void *v_act, const void *cos,
                 const void *sin, const void *position, int32_t max_seq);

/* Attention whose merge is left to the o projection: n_parts workgroups of n_waves (<= 16)
 * wavefronts per query head each leave an unnormalised softmax state {m, l, 0, 0, o[hd]} in
 * `state` (chr_dv2_attn_state_floats(n_q, hd, n_parts) floats, 16-byte aligned); RoPE and the
 * cache write are fused as in chr_nf4_attn.  chr_dv2_gemv_attn then computes
 * y = W @ merge(state) (+ add), merging while it stages its activations: hd % 8 == 0,
 * W.K == n_q*hd == W.K_pad.  Together they replace attn_flash + attn_merge + the o GEMV
 * (gpu/nf4/nf4_gemv.cu:952-994, gpu/decodev2/step.py:119-137) with two launches that spread
 * a head over several compute units.  No reference counterpart. */
int64_t chr_dv2_attn_state_floats(int32_t n_q, int32_t hd, int32_t n_parts);
int chr_dv2_attn_parts(const void *q, const void *k, const void *v, const void *valid_len,
                       float *state, int32_t n_q, int32_t n_kv, int32_t hd, int32_t n_parts,
                       int32_t n_waves, float scale, void *stream, const void *k_act,
                       const void *v_act, const void *cos, const void *sin,
                       const void *position, int32_t max_seq);
int chr_dv2_gemv_attn(const chr_nf4_dev_t *w, const float *state, int32_t n_q, int32_t hd,
                      int32_t n_parts, void *y, const void *add, void *stream);

/* The sum of squares of a vector handed from the launch that writes it to the launch that
 * normalises it, for a decode step that folds every RMSNorm into the GEMV that consumes it
 * (the rms_w argument of chr_nf4_gemv, gpu/nf4/nf4_gemv.cu:264-289): with rms_w alone the
 * consuming launch sums x^2 over its workgroup, two barriers between x arriving and the first
 * product (0.7 us of a 7 us launch); here the writer, which has every element in hand as it
 * stores it, leaves the sum in chr_dv2_sumsq_parts() floats (its workgroups' sums over the bf16
 * values they stored, in a fixed order, zeros behind them: a 16-byte aligned buffer of that
 * many floats, the caller's), and the reader's wavefronts add the parts up themselves.  No
 * reference counterpart.
 *   sumsq_out (chr_dv2_gemv_sumsq, chr_dv2_gemv_attn_sumsq, chr_dv2_begin_step_sumsq): this
 *     launch writes the parts for its y (after `add`).  Only the GEMV kernels that stage x in LDS
 *     do (launches of 16 M codes and more, and every launch that merges attention states):
 *     chr_dv2_sumsq_ok(M, K, K_pad, merges_attention) says whether a matrix of that shape runs
 *     on one (it reads the same environment switches a launch reads); else -8.
 *   sumsq_in (chr_dv2_gemv_sumsq, chr_dv2_gemv_qkv_sumsq, chr_dv2_gemv_swiglu_sumsq): with
 *     rms_w, mean(x^2) comes from the parts that the writer of x left.  Needs K % 8 == 0 and
 *     x, rms_w and the parts 16-byte aligned; else -8.  The parts must be those of this x:
 *     nothing checks it.
 * Either pointer NULL: the entry behaves as the one it extends.  The values differ from the
 * reader's own sum by the order of the additions only. */
int32_t chr_dv2_sumsq_parts(void);
int32_t chr_dv2_sumsq_ok(int32_t M, int32_t K, int32_t K_pad, int32_t merges_attention);
int chr_dv2_gemv_sumsq(const chr_nf4_dev_t *w, const void *x, void *y, void *stream,
                       const void *add, const void *rms_w, float rms_eps, const float *sumsq_in,
                       float *sumsq_out);
int chr_dv2_gemv_qkv_sumsq(const chr_nf4_dev_t *q, const chr_nf4_dev_t *k, const chr_nf4_dev_t *v,
                           const void *x, void *yq, void *yk, void *yv, const void *bq,
                           const void *bk, const void *bv, void *stream, const void *rms_w,
                           float rms_eps, const float *sumsq_in);
int chr_dv2_gemv_swiglu_sumsq(const chr_nf4_dev_t *gate, const chr_nf4_dev_t *up, const void *x,
                              void *y, void *stream, const void *rms_w, float rms_eps,
                              const float *sumsq_in);
int chr_dv2_gemv_attn_sumsq(const chr_nf4_dev_t *w, const float *state, int32_t n_q, int32_t hd,
                            int32_t n_parts, void *y, const void *add, void *stream,
                            float *sumsq_out);
/* chr_dv2_begin_step without its RMSNorm, leaving the parts for the first layer's q/k/v. */
int chr_dv2_begin_step_sumsq(const chr_nf4_dev_t *table, const void *token, const void *position,
                             void *valid_len, void *x, void *stream, float *sumsq_out);

/* ---- Chunked prefill glue on the GEMM's own layout -----------------------------------------
 * The reference's prefill (gpu/decodev2/prefill.py:58-133) runs everything but its linears as
 * stock torch ops on token-major [N, features] tensors and transposes around every GEMM
 * (gpu/decodev2/linear.py:96-113).  These entries do the same arithmetic directly on the
 * feature-major [features, N] bf16 tiles chr_nf4_gemm reads and writes (N <= 64 tokens of one
 * chunk, token index fastest), so a prefill layer is a straight sequence of launches that can
 * be captured in a graph.  None has a counterpart in the reference's C-ABI. */

/* y[k][n] = (w[k] * x[k][n]) * rsqrt(mean_k x[k][n]^2 + eps) per column n
 * (gpu/decodev2/ops.py:18-20).  -2 when N is outside 1..64. */
int chr_dv2_rms_cols(const void *x, const void *w, void *y, int32_t rows, int32_t N, float eps,
                     void *stream);

/* chr_dv2_rms_cols with the column sums of squares supplied (what chr_dv2_gemm_add_sq left for
 * this x: sq[sq_blocks * N]) instead of read from the tile.  N must divide 1024.
 * No reference counterpart. */
int chr_dv2_rms_cols_sq(const void *x, const void *w, void *y, int32_t rows, int32_t N, float eps,
                        const float *sq, int32_t sq_blocks, void *stream);

/* Rotate-half RoPE of q [n_q*hd, N] and k [n_kv*hd, N] at positions *start + n
 * (start: device int64), writing rotated q token-major to q_out [N, n_q*hd] and rotated k
 * and v to cache rows *start + n of [max_seq, n_kv, hd] (gpu/decodev2/prefill.py:100-108).
 * Tokens whose row would fall outside the cache are skipped. */
int chr_dv2_rope_kv_cols(const void *q, const void *k, const void *v, void *q_out,
                         void *k_cache, void *v_cache, const void *cos, const void *sin,
                         const void *start, int32_t N, int32_t n_q, int32_t n_kv, int32_t hd,
                         int32_t max_seq, void *stream);

/* Causal attention of a chunk (gpu/decodev2/ops.py:31-44): token t of q [n_tok, n_q*hd]
 * attends to cache rows 0 .. *first_len + t - 1 (first_len: device int32, the prefix length
 * token 0 sees, itself included), one workgroup of n_waves (<= 16) wavefronts per
 * (head, token).  out[t*out_tok_stride + (head*hd + d)*out_dim_stride]: strides (n_q*hd, 1)
 * give token-major output, (1, N) feature-major. */
int chr_dv2_attn_chunk(const void *q, const void *k, const void *v, void *out,
                       const void *first_len, int32_t n_tok, int32_t n_q, int32_t n_kv,
                       int32_t hd, int32_t n_waves, float scale, void *stream, int32_t max_seq,
                       int32_t out_tok_stride, int32_t out_dim_stride);

/* y = silu(gate) * up over `count` bf16 elements, the activation rounded to bf16 before the
 * product as torch's two ops round (gpu/decodev2/ops.py:23-24). */
int chr_dv2_swiglu_elems(const void *gate, const void *up, void *y, int64_t count, void *stream);

/* Feature-major residual/bias: with a, y = y + (a [+ bias[row]]); with a NULL, y += bias[row];
 * every sum rounded to bf16 (gpu/decodev2/linear.py:114-116, prefill.py:113,133). */
int chr_dv2_add_cols(void *y, const void *a, const void *bias, int32_t rows, int32_t N,
                     void *stream);

/* chr_nf4_gemm_ws with the epilogue of the reference's linear + residual
 * (gpu/decodev2/linear.py:114-116, prefill.py:113,133) folded into the split-K reduction:
 * y = residual + (bf16(W x) + bias[row]), each step rounded to bf16 as the separate torch
 * adds round; bias (bf16 [M]) and residual (bf16 [M, N]) may each be NULL, residual may alias
 * y.  N = 2..64 (-2 for N = 1: the GEMV has its own residual argument).  Beyond the 32
 * columns of the reference's live entries this one also launches the 33..64-column tile that
 * chr_nf4_gemm_plan describes: two 32-column blocks per dequantised weight fragment, so a
 * 64-token chunk costs one pass over the weights, not two.  Workspace as the plan says.
 * No reference counterpart. */
int chr_dv2_gemm_add(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N, float *ws,
                     int64_t ws_floats, const void *bias, const void *residual, void *stream);

/* chr_dv2_gemm_add that also leaves, for the RMSNorm that reads y next, the column sums of
 * squares of the values it stored: with R = chr_dv2_sq_rows(N) = 1024 / N rows per block,
 * colsq[b * N + n] = sum over rows R b .. R b + R - 1 of y[row][n]^2 (fp32,
 * ceil(M / R) * N elements, no NULL).  The sums are taken where the stored values are made: in
 * the tile that finishes its rows itself (32 and 64 columns) or in the split-K reduction, so
 * they exist only when the launch runs one of the two and N divides 256: returns 0 when colsq
 * was written, 1 when the product was computed but colsq was not (the caller then normalises
 * with chr_dv2_rms_cols), a negative code as chr_dv2_gemm_add.  The two places add a block's
 * squares in different orders (the tile by wavefront and lane, the reduction by row), each
 * fixed: a launch repeats its bits, but which place a launch takes follows its plan (shape,
 * chr_nf4_gemm_stream_policy, whether a row of arrival counts was left for its stream), so
 * colsq, and through it single elements of the next RMSNorm's bf16 output, are reproducible
 * for one plan and not across plans.  chr_dv2_sq_rows gives 0 for an N that does not divide
 * 1024.  No reference counterpart (the reference's prefill normalises with a torch op,
 * gpu/decodev2/prefill.py:58-133). */
int chr_dv2_gemm_add_sq(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N, float *ws,
                        int64_t ws_floats, const void *bias, const void *residual, float *colsq,
                        void *stream);
int32_t chr_dv2_sq_rows(int32_t N);

/* q, k and v of one layer in one launch (the prefill twin of chr_nf4_gemv_qkv,
 * gpu/decodev2/ops.py:27-35 calls three GEMMs): the three matrices share x [K, N] and K; y is
 * [Mq + Mk + Mv, N] with q's rows first, bias (bf16 [Mq + Mk + Mv], or NULL) is added per row
 * as chr_dv2_gemm_add adds it.  N = 2..64.  chr_dv2_gemm_qkv_ws gives the fp32 workspace
 * elements the launch needs (0: none; -1: bad arguments).  No reference counterpart. */
int64_t chr_dv2_gemm_qkv_ws(const chr_nf4_dev_t *q, const chr_nf4_dev_t *k,
                            const chr_nf4_dev_t *v, int32_t N);
int chr_dv2_gemm_qkv(const chr_nf4_dev_t *q, const chr_nf4_dev_t *k, const chr_nf4_dev_t *v,
                     const void *x, void *y, int32_t N, float *ws, int64_t ws_floats,
                     const void *bias, void *stream);

/* Gate and up of a layer in one launch with the SwiGLU in the split-K reduce (the prefill twin
 * of chr_nf4_gemv_swiglu; gpu/decodev2/prefill.py:133 runs two GEMMs, F.silu and a product):
 * y [M, N] = silu(gate x) * (up x), gate and up rounded to bf16 first and the activation
 * rounded to bf16 before the product, as those separate bf16 ops round.  Both matrices are
 * M x K.  N = 2..64.  The launch goes through fp32 partials and a reduce that applies the
 * activation -- chr_dv2_gemm_swiglu_ws gives the workspace elements it needs (-1: bad
 * arguments) -- or, at 64 columns where the planner takes the unsplit tile that finishes its
 * rows itself, pairs 32 gate rows with their up rows in a workgroup, which stores the
 * activation: then chr_dv2_gemm_swiglu_ws gives 0 and ws may be NULL.  No reference
 * counterpart. */
int64_t chr_dv2_gemm_swiglu_ws(const chr_nf4_dev_t *gate, const chr_nf4_dev_t *up, int32_t N);
int chr_dv2_gemm_swiglu(const chr_nf4_dev_t *gate, const chr_nf4_dev_t *up, const void *x,
                        void *y, int32_t N, float *ws, int64_t ws_floats, void *stream);

/* chr_dv2_argmax_commit as two launches for a large vocabulary: 128 workgroups leave the best
 * (value, index) of a slice each in ws, a small launch picks among them and commits; same
 * tie and NaN rules.  ws: chr_dv2_argmax_ws_bytes() bytes of device memory, 8-byte aligned;
 * with ws NULL or too small, or n < 16384, this is chr_dv2_argmax_commit.
 * No reference counterpart. */
int64_t chr_dv2_argmax_ws_bytes(void);
int chr_dv2_argmax_commit_ws(const void *logits, int32_t n, void *next_token, void *token,
                             void *position, void *finished, const void *eos_id, int32_t commit,
                             void *ws, int64_t ws_bytes, void *stream);

/* Library version, for the loader's sanity check. */
int chr_nf4_abi_version(void);

#ifdef __cplusplus
}
#endif
