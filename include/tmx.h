/* tmx: MI355X (gfx950) decode-step kernels for an int4 group-quantised QLoRA
 * policy behind tunix's Sampler -- C ABI.
 *
 * The reference (bigdatamark/tunix) has no FFI for this path: its decode step is
 * XLA-compiled JAX.  Each entry point below names the reference arithmetic it
 * replaces (path:line relative to the reference tree).  The same functions are
 * what an XLA custom-call handler registered through jax.ffi would forward to.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *   - `stream` is a hipStream_t passed as void*; entry points only enqueue work
 *     on it: they never allocate, free or synchronise.  Four calls wait for the
 *     stream and say so where they are declared: tmx_handover_status,
 *     tmx_decode_status, tmx_decode_steps_graph (which also creates and destroys
 *     a stream, an event and a graph) and tmx_decode_steps_profiled (events);
 *     some kernels set their dynamic LDS limit with hipFuncSetAttribute on their
 *     first launch in the process;
 *   - bf16 tensors are raw 16-bit patterns, row-major, innermost index last;
 *   - return value: TMX_OK or a negative TMX_ERR_* code, nothing is launched
 *     when an argument check fails.
 *
 * Packed int4 tile format ("q4t") of a logical weight W[K, N] (K % 64 == 0,
 * N % 32 == 0), nibble u = q + 8 with q in [-8, 7]:
 *   tile (nb, kb) = rows [64 kb, 64 kb + 64) x columns [32 nb, 32 nb + 32) is the
 *   1024 bytes at byte offset (nb * (K / 64) + kb) * 1024; inside it lane
 *   l = 32 h + (n % 32) owns the 16 bytes at l * 16 = four little-endian 32-bit
 *   words t = 0..3; nibble i (bits 4i..4i+3) of word t is the element
 *   k = 64 kb + 16 t + 8 h + 2 (i % 4) + (i / 4).
 *   Scales: bf16 [N / 32][K / G][32], G % 64 == 0.
 */
#ifndef TMX_H_
#define TMX_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TMX_OK 0
#define TMX_ERR_ARG (-1)         /* null pointer / inconsistent optional arguments */
#define TMX_ERR_SHAPE (-2)       /* a dimension violates the kernel's tiling rules */
#define TMX_ERR_LAUNCH (-3)      /* the HIP runtime refused the launch */
#define TMX_ERR_UNSUPPORTED (-4) /* valid request outside what is implemented */
#define TMX_ERR_SCRATCH (-5)     /* the request needs more scratch memory than the library's static buffer holds */
#define TMX_ERR_DEVICE_WAIT (-6) /* a bounded wait inside a kernel ran out (reported by tmx_decode_status) */

#define TMX_FAMILY_LLAMA3 0
#define TMX_FAMILY_QWEN3 1

#define TMX_MAX_RPAD 128   /* widest padded LoRA projection (sum of fused ranks, rounded up to 32) */
#define TMX_MAX_SPLITS 16  /* most K-slices a projection is split into */
#define TMX_MAX_LORA_SPLITS 32 /* most K-slices of the LoRA projection x . A */
#define TMX_MAX_MOE_PAIRS 8192 /* most routed (token, expert) pairs of one pass: rows x experts_per_tok */
#define TMX_MAX_FILL_ROWS 4096 /* most rows (sequences x tokens per sequence) of one pass of tmx_decode_steps */

#define TMX_SAMPLE_GREEDY 0
#define TMX_SAMPLE_TOP_P 1
#define TMX_SAMPLE_SCORE 2 /* teacher forcing: no token is chosen; logprobs[m, *step + 1] =
                              z[token_buffer[m, *step + 1]] - logsumexp(z), z = logits / temperature
                              with NaN -> -1e9 and the rest clipped to [-1e9, 1e9], so the result is
                              always finite (tunix/rl/common.py:426-606 compute_per_token_logps,
                              :207-226 selective_log_softmax) */

const char* tmx_status_string(int status);
/* Bumped whenever a struct of this header grows or an entry point changes: 7 = tmx_model_desc.head_tiles and the
 * tmx_decode_state.share_* fields are present.  A caller that fills the structs checks it once after loading. */
#define TMX_ABI_VERSION 7
int tmx_abi_version(void);

/* w_out[K, N] bf16 = bf16(q) * scale evaluated in bf16, bit-exact.
 * Replaces qwix's dequantise step behind tunix/cli/utils/model.py:31-77
 * (weight_qtype / tile_size of the LoraProvider). */
int tmx_int4_dequant(void* stream, const void* qweight, const void* scales, void* w_out, int K, int N,
                     int G);

/* y[M, N] = bf16(x[M, K] . dequant(qweight)) (+ LoRA delta) (+ residual).  Up to 128 rows run
 * the decode kernels (K % 64 == 0); more rows run in 256-row blocks and need K % 128 == 0.
 * Replaces the qwix-wrapped Einsum / nnx.Linear call: tunix/models/llama3/model.py:216-218,
 * :489-496; tunix/models/qwen3/model.py:389-393, :1199-1208.
 *   lora_a_t : A in MFMA fragment order, bf16 [K/64][r_pad/32][4][64][8], r_pad % 32 == 0,
 *              columns >= r zero (NULL: no LoRA): element A[64 kb + 16 t + 8 h + j][32 ct + c]
 *              at ((((kb * (r_pad/32) + ct) * 4 + t) * 64 + 32 h + c) * 8 + j)
 *   lora_b   : bf16 [r, N]
 *   residual : bf16 [M, N] or NULL; added after the LoRA delta, in bf16
 *   workspace: tmx_qlora_linear_workspace_bytes(M, K, N) bytes (f32 K-slice planes) */
size_t tmx_qlora_linear_workspace_bytes(int M, int K, int N);
int tmx_qlora_linear(void* stream, const void* x, const void* qweight, const void* scales,
                     const void* lora_a_t, const void* lora_b, const void* residual, void* y,
                     void* workspace, int M, int K, int N, int G, int r, int r_pad, float lora_scale);

/* tmx_qlora_linear without a workspace argument and without any allocation.  No counterpart in
 * the reference: it exists for callers that cannot allocate device memory around the call (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The K-slice and
 * LoRA planes live in a static device array of TMX_STATIC_SCRATCH_BYTES that each GPU the library
 * runs on holds until the process ends; a request whose tmx_qlora_linear_workspace_bytes(M, K, N)
 * exceeds it returns TMX_ERR_SCRATCH and launches nothing (every decode shape of the 8B models
 * up to 128 rows fits).  All calls on one GPU share that GPU's array: calls that overlap on one
 * GPU (two streams, two threads) race; calls on one stream are ordered and safe.  Same results
 * as tmx_qlora_linear, bit for bit. */
#define TMX_STATIC_SCRATCH_BYTES (32u << 20)
size_t tmx_qlora_linear_noalloc_max_bytes(void);
int tmx_qlora_linear_noalloc(void* stream, const void* x, const void* qweight, const void* scales,
                             const void* lora_a_t, const void* lora_b, const void* residual, void* y,
                             int M, int K, int N, int G, int r, int r_pad, float lora_scale);

/* The matrix product alone, for callers that fuse their own consumer: writes `nsplit` f32
 * K-slice planes y_part[nsplit][M][N] (their sum is x . dequant(W)) and, with LoRA,
 * t_part[tmx_qlora_linear_num_lora_splits(K, N)][M][TMX_MAX_RPAD] (their sum is x . A).
 * nsplit in [1, TMX_MAX_SPLITS] and such that no K-slice is empty;
 * tmx_qlora_linear_num_splits() returns the count the library itself would pick. */
int tmx_qlora_linear_num_splits(int M, int K, int N);
int tmx_qlora_linear_num_lora_splits(int K, int N);
int tmx_qlora_linear_planes(void* stream, const void* x, const void* qweight, const void* scales,
                            const void* lora_a_t, float* y_part, float* t_part, int M, int K, int N,
                            int G, int r_pad, int nsplit);

/* tmx_qlora_linear_planes whose launch also finishes the LoRA product: once every slice of x . A is
 * there, the LoRA workgroups of the launch add the planes in slice order, round to bf16 and write
 * delta[M, N] = bf16(bf16(t . B) * lora_scale) (bf16), the term the consumer adds to the rounded sum of the
 * y planes (column n below seg_end0 uses t columns 0..r-1, below seg_end1 r..2r-1, else 2r..3r-1: the
 * fused q | k | v layout; pass N, N for a single matrix).  This is what the decode step does for
 * projections whose K-slices are long enough to hide it (slices of at least 2048 rows of W, at most two
 * 32-column tiles per LoRA wave): tmx_qlora_linear_delta_workspace_bytes returns 0 for every other shape
 * and the call TMX_ERR_UNSUPPORTED.  workspace: that many bytes (cleared by the call: one small launch).
 * Up to 128 rows, r <= 64.  The LoRA workgroups wait for one another a bounded number of polls; if that
 * wait ever runs out they take t as zero and set a word inside `workspace` that tmx_handover_status
 * reports.  No counterpart in the reference beyond the LoRA arithmetic itself. */
size_t tmx_qlora_linear_delta_workspace_bytes(int M, int K, int N, int r, int r_pad, int nsplit);
int tmx_qlora_linear_planes_delta(void* stream, const void* x, const void* qweight, const void* scales,
                                  const void* lora_a_t, const void* lora_b, float* y_part, float* t_part,
                                  void* delta, void* workspace, int M, int K, int N, int G, int r, int r_pad,
                                  float lora_scale, int seg_end0, int seg_end1, int nsplit);

/* WAITS for `stream`, then reports and clears the "a bounded wait ran out" word of a hand-over workspace
 * (the `workspace` of tmx_qlora_linear_planes_delta or tmx_qlora_gate_up_swiglu_handover): TMX_OK, or
 * TMX_ERR_DEVICE_WAIT when the last call on that workspace dropped its LoRA term.  No counterpart in
 * the reference (XLA has no such failure mode). */
int tmx_handover_status(void* stream, void* workspace);

/* One projection of the single-sequence regime (1..4 rows) in ONE launch: optional RMSNorm of
 * x in the prologue (norm_w != NULL; family as tmx_rmsnorm), the int4 product, the LoRA delta
 * computed inside (t = x . A by every workgroup), then either nothing, the residual add
 * y = bf16(y + residual), or SwiGLU (swiglu != 0: N = 2 F stacked gate | up columns, y is
 * [M, F] = bf16(silu(gate) * up), r_pad == 32 with 2 r <= 32).  Same rounding chain as
 * tmx_rmsnorm + tmx_qlora_linear (+ tmx_swiglu).  M <= 4, M K <= 16384 with the norm (32768
 * without), r <= 32, r_pad <= 64; the norm and the residual do not combine.
 * tunix/models/llama3/model.py:290-297, :216-218, :489-496, :546-564. */
int tmx_small_linear(void* stream, const void* x, const void* norm_w, float eps, int family,
                     const void* qweight, const void* scales, const void* lora_a_t, const void* lora_b,
                     const void* residual, void* y, int M, int K, int N, int G, int r, int r_pad,
                     float lora_scale, int swiglu);

/* ---- row-wise kernels between the matrix products ------------------------- */

/* y[M, D] = RMSNorm(x) * w.  TMX_FAMILY_LLAMA3: bf16(bf16(w * x) / rms)
 * (tunix/models/llama3/model.py:290-297); TMX_FAMILY_QWEN3: bf16(w * (x / rms))
 * in f32 (tunix/models/qwen3/model.py:478-484). */
int tmx_rmsnorm(void* stream, const void* x, const void* w, void* y, int M, int D, float eps, int family);

/* The three consumers below take the output of a projection either as a bf16 tensor
 * (*_bf16) or as `nsplit` f32 K-slice planes [nsplit][M][N] (*_part) that they sum and round
 * to bf16 first, and apply the LoRA-B half:
 *   delta[m, n] = bf16(bf16(sum_r t[m, r] lora_b[r, n]) * lora_scale),
 *   t[m, r] = bf16(sum_s t_part[s][m][r]), t_part f32 [t_nsplit][M][ldt] (NULL: no LoRA). */

/* h = bf16(bf16(y + delta) + residual) -> x_out;  xn_out = RMSNorm(h) * norm_w.
 * residual, x_out, norm_w may be NULL.  Residual wiring of
 * tunix/models/llama3/model.py:546-564, tunix/models/qwen3/model.py:1268-1289. */
int tmx_lora_residual_rmsnorm(void* stream, const void* y_bf16, const float* y_part, int nsplit,
                              const float* t_part, int t_nsplit, int ldt, const void* lora_b, int r,
                              float lora_scale,
                              const void* residual, void* x_out, const void* norm_w, void* xn_out, int M,
                              int D, float eps, int family);

/* qkv[B, (N + 2 Kh) H] (+ deltas, t columns x.A_q | x.A_k | x.A_v) -> optional per-head
 * RMSNorm (Qwen3 q_norm / k_norm), RoPE at positions[b, *step], q_out[B, N H] and the
 * K / V rows of cache slot *step % C.  tunix/models/llama3/model.py:249-270, :348-377;
 * tunix/models/qwen3/model.py:432-453, :559-597. */
int tmx_rope_kv_write(void* stream, const void* qkv_bf16, const float* qkv_part, int nsplit,
                      const float* t_part, int t_nsplit, int ldt, const void* lora_b, int r,
                      float lora_scale,
                      const void* q_norm_w, const void* k_norm_w, const int32_t* positions,
                      const int32_t* step, int buf_len, void* q_out, void* kcache, void* vcache, int B,
                      int N, int Kh, int H, int C, float theta, float eps, int family);

/* act[M, F] = bf16(silu(gate) * up), gate_up[M, 2F] = gate columns then up columns
 * (+ deltas, t columns x.A_gate | x.A_up).  tunix/models/llama3/model.py:489-496. */
int tmx_swiglu(void* stream, const void* gate_up_bf16, const float* gate_up_part, int nsplit,
               const float* t_part, int t_nsplit, int ldt, const void* lora_b, int r, float lora_scale,
               void* act, int M, int F);

/* act[M, F] = bf16(silu(g) * u) with g | u = x . dequant(Wq, s) (+ LoRA deltas) for the stacked
 * gate | up matrix [K, 2F], in one launch: projection, LoRA and SwiGLU fused.  Needs
 * K % 256 == 0, K < 8192, F % 64 == 0; with LoRA lora_a_t = [A_gate | A_up] in fragment order
 * with r_pad == 32 (2 r <= 32) and lora_b [r][2F].  tunix/models/llama3/model.py:489-496 with
 * the qwix-wrapped projections of :461-487. */
int tmx_qlora_gate_up_swiglu(void* stream, const void* x, const void* qweight, const void* scales,
                             const void* lora_a_t, const void* lora_b, void* act, int M, int K, int F,
                             int G, int r, float lora_scale);

/* The same launch in the form the decode step runs at up to 64 rows with LoRA: t = x . [A_gate | A_up] is
 * computed once, by K / 256 extra workgroups of the launch, and handed to the others through `workspace`
 * (tmx_qlora_gate_up_swiglu_handover_bytes(M, K, F, r) bytes, whose state block the call clears with one
 * small launch) instead of being recomputed by every workgroup; same results up to the summation order of
 * t's K-slices.  The size query returns 0, and the call TMX_ERR_UNSUPPORTED, for shapes that do not take
 * this form on the current device (more than 64 rows, K % 512 != 0, 2 r > 32, or more workgroups than
 * compute units).  The receiving workgroups wait a bounded number of polls: see tmx_handover_status. */
size_t tmx_qlora_gate_up_swiglu_handover_bytes(int M, int K, int F, int r);
int tmx_qlora_gate_up_swiglu_handover(void* stream, const void* x, const void* qweight, const void* scales,
                                      const void* lora_a_t, const void* lora_b, void* act, void* workspace,
                                      int M, int K, int F, int G, int r, float lora_scale);

/* ---- GQA decode attention -------------------------------------------------- */

/* out[B, N H] = softmax(q . K^T / sqrt(H) over positions j <= *step with
 * input_mask[b, j]) . V, caches bf16 [B, C, Kh, H].  tunix/models/llama3/model.py:379-396,
 * tunix/models/qwen3/model.py:776-793 with the mask of tunix/generate/utils.py:35-59.
 * workspace: tmx_gqa_decode_workspace_bytes() bytes (may be 0 -> NULL allowed). */
size_t tmx_gqa_decode_workspace_bytes(int B, int N, int Kh, int H, int C);
int tmx_gqa_decode_attention(void* stream, const void* q, const void* kcache, const void* vcache,
                             const uint8_t* input_mask, const int32_t* step, int buf_len, void* out,
                             void* workspace, int B, int N, int Kh, int H, int C);

/* tmx_gqa_decode_attention for a batch made of consecutive groups of `share_group` sequences whose cache
 * slots [0, share_len) hold identical K / V rows and identical input_mask entries: the G samples of one
 * prompt that a GRPO rollout decodes side by side (tunix/rl/rl_learner.py:432-435 repeats every prompt
 * num_generations times, in consecutive rows).  Those slots are read once per group, from the group's
 * first sequence, for all of the group's queries; every sequence reads only its own slots from share_len
 * on.  The softmax runs over the same positions as in tmx_gqa_decode_attention (the results differ in
 * the order of the f32 sums only).  The caller vouches for the sharing; nothing checks that the rows
 * really are equal.  B <= 128, B % share_group == 0, 32 <= share_len <= C, H in {64, 128}, N / Kh in
 * {1, 2, 4, 8}, else TMX_ERR_UNSUPPORTED.  workspace: tmx_gqa_decode_shared_workspace_bytes() bytes. */
size_t tmx_gqa_decode_shared_workspace_bytes(int B, int N, int Kh, int H, int C);
int tmx_gqa_decode_attention_shared(void* stream, const void* q, const void* kcache, const void* vcache,
                                    const uint8_t* input_mask, const int32_t* step, int buf_len, void* out,
                                    void* workspace, int B, int N, int Kh, int H, int C, int share_group,
                                    int share_len);

/* The same for T consecutive query tokens of every sequence (cache fill and scoring passes):
 * q and out are [n_seq * T, N H], row s * T + t is the token at slot *step + t of sequence s and
 * attends to the slots j <= *step + t with input_mask[s, j] (the causal mask of
 * tunix/generate/utils.py:2116-2229 restricted to the rows of the pass); K and V of the pass's
 * own tokens must already be in the caches.  From 4 tokens per sequence on, a workgroup walks the
 * cache once for a block of tokens (MFMA kernel, head_dim 64 or 128); below, every row runs the
 * decode kernel.  workspace: tmx_gqa_decode_workspace_bytes(n_seq * T, N, Kh, H, C) bytes. */
int tmx_gqa_attention_rows(void* stream, const void* q, const void* kcache, const void* vcache,
                           const uint8_t* input_mask, const int32_t* step, int buf_len, void* out,
                           void* workspace, int n_seq, int T, int N, int Kh, int H, int C);

/* ---- final projection + log-softmax + token selection ---------------------- */

/* logits = bf16(x[M, D] . head_w[V, D]^T) as f32; forbidden ids -> -inf; mode
 * TMX_SAMPLE_GREEDY: token = argmax (first index on ties), logprob =
 * log_softmax(logits)[token]; TMX_SAMPLE_TOP_P (top_p >= 1, no top_k): z = logits /
 * temperature, token = argmax(z + gumbel(threefry(fold_in(seed, *step)))), logprob =
 * log_softmax(z)[token].  Writes token_buffer[m, *step + 1], logprobs[m, *step + 1]
 * (if not NULL), done[m] |= token in eos.  tunix/generate/sampler.py:112-168, :520-599;
 * tunix/models/llama3/model.py:688-697.  logits_out: optional f32 [M, V]. */
size_t tmx_head_sample_workspace_bytes(int M, int V);
int tmx_head_sample(void* stream, const void* x, const void* head_w, int M, int D, int V, int mode,
                    float temperature, uint32_t seed_hi, uint32_t seed_lo, const int32_t* step,
                    const int32_t* forbidden, int n_forbidden, const int32_t* eos, int n_eos,
                    int32_t* token_buffer, float* logprobs, uint8_t* done, int buf_len,
                    float* logits_out, void* workspace);

/* The same from a copy of the head matrix laid out for streaming: tmx_head_tiles_pack writes head_tiles
 * (V * D bf16 elements, like head_w) from head_w[V, D]; 32 rows x 64 columns form a tile of 4 KiB, the tiles of
 * 32 rows follow each other along D, and inside a tile the 16 bytes head_w[32 vt + n][64 kt + 32 h + 8 t .. + 7]
 * sit at byte (t * 64 + 32 h + n) * 16.  V % 32 == 0, D % 64 == 0, V <= 32 * 65535.  The layout has no counterpart
 * in the reference (jnp arrays are row-major); results are bit-identical to tmx_head_sample's. */
int tmx_head_tiles_pack(void* stream, const void* head_w, void* head_tiles, int V, int D);
int tmx_head_sample_tiles(void* stream, const void* x, const void* head_tiles, int M, int D, int V, int mode,
                          float temperature, uint32_t seed_hi, uint32_t seed_lo, const int32_t* step,
                          const int32_t* forbidden, int n_forbidden, const int32_t* eos, int n_eos,
                          int32_t* token_buffer, float* logprobs, uint8_t* done, int buf_len,
                          float* logits_out, void* workspace);

/* The sorting branch of sample_top_p (top_p < 1 and / or top_k > 0),
 * tunix/generate/sampler.py:136-153: candidates = the top_k (or all V) logits in descending
 * order, ties in index order; probs = softmax over the candidates; a candidate is dropped when
 * the cumulative probability before it exceeds top_p; token = Gumbel-max over the survivors
 * with the noise of rank i of row m drawn at linear index m * k + i; logprob =
 * log_softmax(z)[token] over the full vocabulary.  Same outputs as tmx_head_sample.  Nothing is
 * sorted: the logits are bf16, so ranks and cumulative probabilities follow from per-row counts
 * of the 65 536 possible values (three launches after the head kernel, no library call).
 * nucleus_workspace: tmx_nucleus_workspace_bytes(M, V) bytes (one 16-bit key per logit, the
 * per-row value tables and the slice winners); 0 for an unsupported shape. */
size_t tmx_nucleus_workspace_bytes(int M, int V);
int tmx_head_sample_nucleus(void* stream, const void* x, const void* head_w, int M, int D, int V,
                            float temperature, float top_p, int top_k, uint32_t seed_hi,
                            uint32_t seed_lo, const int32_t* step, const int32_t* forbidden,
                            int n_forbidden, const int32_t* eos, int n_eos, int32_t* token_buffer,
                            float* logprobs, uint8_t* done, int buf_len, void* workspace,
                            void* nucleus_workspace, size_t nucleus_workspace_bytes);

/* ---- routed experts (Qwen3 MoE) ----------------------------------------------- */

/* Routing of tunix/models/qwen3/model.py:895-902: scores = bf16(x[B, D] . router_w[D, E]),
 * f32 softmax, top_k (ties: lower expert id), weights renormalised over the top_k and rounded
 * to bf16.  expert_of / weight_of: [B, top_k]. */
int tmx_moe_route(void* stream, const void* x, const void* router_w, int B, int D, int E, int top_k,
                  int32_t* expert_of, float* weight_of);

/* One launch over all experts (the routed pairs of tunix/models/qwen3/model.py:911-939):
 * pair p = token * top_k + slot belongs to expert expert_of[p]; experts nobody routed to are
 * not read.  qweight / scales: E stacked per-expert matrices [K, N] in the q4t / scale layout.
 *   down == 0: x = hidden states [P / top_k, K = D] (row p / top_k), N = 2 F with columns
 *              gate | up; out[p, 0:F] = bf16(silu(gate) * up) (F % 64 == 0)
 *   down != 0: x = activations [P, K = F] (row p); out[p, 0:N] = bf16(x . W_e) (N % 128 == 0)
 * K % 256 == 0, P <= TMX_MAX_MOE_PAIRS. */
int tmx_moe_experts(void* stream, const void* x, int ldx, const void* qweight, const void* scales,
                    const int32_t* expert_of, int P, int top_k, int E, int K, int N, int G, int down,
                    void* out, int ldo);

/* ---- whole decode steps ------------------------------------------------------ */


typedef struct {
  const void* qweight;  /* q4t tiles of the (column-fused) weight [K, N] */
  const void* scales;   /* bf16 [N/32][K/G][32] */
  const void* lora_a_t; /* fused A matrices side by side in fragment order (see tmx_qlora_linear); NULL = no LoRA */
  const void* lora_b;   /* bf16 [rank, N]: B matrices side by side */
  int K, N, G, rank, r_pad;
  float lora_scale;     /* alpha / rank */
} tmx_qlinear_desc;

typedef struct {
  const void* norm1_w;  /* input_layernorm.w [D] bf16 */
  const void* norm2_w;  /* post_attention_layernorm.w [D] */
  const void* q_norm_w; /* Qwen3 q_norm.w [H] or NULL */
  const void* k_norm_w;
  tmx_qlinear_desc qkv;     /* columns: q (N H) | k (Kh H) | v (Kh H) */
  tmx_qlinear_desc o;       /* [N H, D] */
  tmx_qlinear_desc gate_up; /* columns: gate (F) | up (F); MoE: num_experts such matrices stacked */
  tmx_qlinear_desc down;    /* [F, D]; MoE: num_experts stacked */
  const void* router_w;     /* MoE: bf16 [D, num_experts] router kernel, else NULL */
} tmx_layer_desc;

typedef struct {
  int family; /* TMX_FAMILY_* */
  int num_layers, vocab_size, embed_dim, hidden_dim, num_heads, num_kv_heads, head_dim;
  int num_experts, experts_per_tok;
  float rope_theta; /* ignored for TMX_FAMILY_LLAMA3: the reference's Llama3 attention never
                       forwards config.rope_theta, so 1e6 is used (llama3/model.py:356-365) */
  float norm_eps;
  const void* embed;        /* bf16 [V, D] */
  const void* final_norm_w; /* bf16 [D] */
  const void* head;         /* bf16 [V, D]: the embedding table when tied, else lm_head^T */
  const tmx_layer_desc* layers; /* HOST array of num_layers entries */
  const void* head_tiles;   /* NULL, or the head matrix once more in the layout tmx_head_tiles_pack writes (V % 32
                               == 0, D % 64 == 0): steps of up to 64 sequences then stream that copy, every byte
                               in whole cache lines (the 1.05 GB head of the 8B shape: 190 us against 252 us) */
} tmx_model_desc;

/* Mirrors _SamplingState (tunix/generate/sampler.py:53-109); all arrays on the device. */
typedef struct {
  int batch, buf_len, cache_size;
  int32_t* token_buffer; /* [B, buf_len] */
  int32_t* positions;    /* [B, buf_len] */
  uint8_t* input_mask;   /* [B, buf_len] 1 = real token */
  float* logprobs;       /* [B, buf_len] or NULL */
  uint8_t* done;         /* [B] */
  int32_t* step;         /* device scalar: decoding_step */
  void* kv_cache;        /* bf16 [layers][2 (k, v)][B][C][Kh][H] */
  int sampling_mode;     /* TMX_SAMPLE_* */
  float temperature, top_p;
  int top_k;
  uint32_t seed_hi, seed_lo;
  const int32_t* eos_ids;
  int n_eos;
  const int32_t* forbidden;
  int n_forbidden;
  float* logits_out;     /* optional f32 [B, V]: logits of the last executed step */
  void* workspace;
  size_t workspace_bytes;
  void* nucleus_workspace; /* tmx_nucleus_workspace_bytes(B, V); needed when top_p < 1 or top_k > 0 */
  size_t nucleus_workspace_bytes;
  int tokens_per_pass;     /* 0 or 1: one token per sequence and step.  T > 1 (cache fill with
                              sample == 0, or TMX_SAMPLE_SCORE): every pass consumes the T tokens at
                              columns *step .. *step + T - 1 of each sequence as batch * T rows, each
                              attending to the slots up to its own column; *step advances by T.
                              Rows of a pass (batch * T, also for T <= 1): up to TMX_MAX_FILL_ROWS when
                              every projection has K % 128 == 0 (MoE models: rows * experts_per_tok <=
                              TMX_MAX_MOE_PAIRS), else 128.
                              The workspace must be sized for batch * T rows. */
  int share_group;         /* 0 or 1: nothing is shared.  g > 1: the batch is made of consecutive groups of g
                              sequences whose cache slots [0, share_len) and input_mask entries are identical
                              (the samples of one prompt); one-token decode steps then read those slots once
                              per group (see tmx_gqa_decode_attention_shared).  Ignored where the shared walk
                              does not apply (more than 128 sequences, batch % g != 0, the 1..4-row path,
                              tokens_per_pass > 1) */
  int share_len;
} tmx_decode_state;

size_t tmx_decode_workspace_bytes(const tmx_model_desc* model, int batch, int cache_size);

/* Contract on the step counter: the caller keeps *step + n_steps * max(tokens_per_pass, 1) < buf_len
 * (<= cache_size).  The library cannot read the device counter on the host; kernels clamp the
 * column they read and skip writes past buf_len, and token ids are clamped to [0, vocab_size) in
 * the embedding gather (the reference's JAX gathers clamp too), so a violation yields undefined
 * tokens but no access outside the buffers.
 *
 * Enqueues n_steps iterations of the Sampler's decode loop body
 * (tunix/generate/sampler.py:749-793): read token_buffer[:, *step], run the model with
 * the KV cache, select the next token into column *step + 1, ++*step.  With sample == 0
 * the head and token selection are skipped (cache fill: used to walk over prompt tokens).
 * `model`, `state` and model->layers are HOST structures read during the call only. */
int tmx_decode_steps(const tmx_model_desc* model, const tmx_decode_state* state, void* stream,
                     int n_steps, int sample);

/* Some decode kernels hand data from one group of workgroups to another inside a launch (the
 * fused gate | up projection computes its LoRA projection once and passes it on).  The
 * receiving side waits a bounded number of polls; if a wait ever runs out the kernel carries
 * on with zeros and sets a sticky word in the workspace.  This call WAITS for `stream`, reads
 * that word, clears it, and returns TMX_ERR_DEVICE_WAIT if it was set (the tokens produced
 * since the previous check are then not to be trusted), else TMX_OK.  The word lives in the
 * first 256 bytes of state->workspace, which the decode calls never clear: zero-fill them
 * once before the workspace's first use.  No counterpart in the reference (XLA has no such
 * failure mode). */
int tmx_decode_status(const tmx_model_desc* model, const tmx_decode_state* state, void* stream);

/* The same steps with one of them recorded into a HIP graph and replayed n_steps - 1 times
 * (fewer host launches; what the reference gets from jit-compiling the while_loop).  Unlike
 * tmx_decode_steps this call WAITS for its replays before it returns (the graph is private
 * to the call), creates and destroys a stream, an event and a graph, and falls back to plain
 * launches for n_steps < 4 or when capture is unavailable. */
int tmx_decode_steps_graph(const tmx_model_desc* model, const tmx_decode_state* state, void* stream,
                           int n_steps, int sample);

/* Measurement aid (no counterpart in the reference): the same as tmx_decode_steps, but every
 * kernel launch is bracketed by HIP events on `stream`; after enqueuing, the call SYNCHRONISES
 * the stream and adds up the elapsed milliseconds and the launch count per kernel class into
 * the two HOST arrays of TMX_NUM_KERNEL_CLASSES entries.  An event pair around a launch also
 * times the packet processing before and after it; class TMX_K_EMPTY brackets a kernel that
 * does nothing (once per layer), so that callers can subtract that constant. */
#define TMX_K_ROWNORM 0  /* embedding gather / residual + LoRA-B + RMSNorm rows */
#define TMX_K_QKV 1      /* fused q|k|v int4 projection (+ LoRA-A tiles) */
#define TMX_K_ROPE 2     /* LoRA-B + RoPE + KV-cache write */
#define TMX_K_ATTN 3     /* GQA decode attention (+ split combine) */
#define TMX_K_O 4        /* o projection */
#define TMX_K_GATE_UP 5  /* fused gate|up projection */
#define TMX_K_SWIGLU 6
#define TMX_K_DOWN 7     /* down projection */
#define TMX_K_HEAD 8     /* head + log-softmax + token selection (+ finalize) */
#define TMX_K_ADVANCE 9
#define TMX_K_EMPTY 10   /* one empty launch per layer: what an event pair costs by itself */
#define TMX_K_ROUTER 11  /* MoE router: scores, softmax, top-k */
#define TMX_NUM_KERNEL_CLASSES 12
int tmx_decode_steps_profiled(const tmx_model_desc* model, const tmx_decode_state* state, void* stream,
                              int n_steps, int sample, float* class_ms_host, int* class_launches_host);

#ifdef __cplusplus
}
#endif
#endif /* TMX_H_ */
