// Argument blocks and host-side launch functions shared by the translation units.
#pragma once
#include "tmx_common.h"

namespace tmx {

struct QLinearArgs {
  const uint16_t* x;       // [M, K] bf16 row-major
  int ldx;
  const uint4* qw;         // packed int4 tiles
  const uint16_t* scales;  // [N/32][K/G][32] bf16
  const uint16_t* a_t;     // LoRA A in fragment order [K/64][Rpad/32][4][64][8] bf16 (may be null)
  uint16_t* y_bf16;        // [M, N] bf16 (only when nsplit == 1), else null
  float* y_part;           // [nsplit][M][N] f32 planes
  float* t_part;           // [lora splits][M][ldt] f32 LoRA projection planes
  int ldt;
  int M, K, N, G, Rpad;
  int n_main_blocks, nsplit, kt_per_split;
  int lora_blocks_per_split, kt_per_lora_split;  // finer K-slices of the LoRA projection
  // routed-expert use of the 4-wave block (all zero / null / -1 for plain projections)
  int ldy;                 // row stride of y_bf16
  int fixed_slice;         // K-slice index when blockIdx.y means something else (-1: blockIdx.y)
  const int* row_src;      // activation row of tile row i (null: i)
  const int* row_dst;      // output row of tile row i (null: i)
  int pair_off;            // != 0: gate | up pairing, tile distance between a gate tile and its up tile
  // LoRA inside the pair epilogue (fused gate | up kernel): a_t = [A_gate | A_up], Rpad == 32
  const uint16_t* lora_b;  // [lora_r][N] bf16
  int lora_r;
  float lora_ls;
  // LoRA inside the epilogue of the many-rows kernel: t16 = bf16(x . A) [M][ldt16] computed beforehand;
  // a column below seg_end[s] (and not below seg_end[s - 1]) uses t columns s lora_r .. s lora_r + lora_r - 1
  const uint16_t* t16;
  int ldt16;
  int seg_end[3];
  // LoRA projection computed once per launch by extra workgroups and handed over through memory
  // (fused gate | up kernel): hand-over state {arrivals, ready, readers, timeout}, partial tiles, t
  uint32_t* sync;
  uint32_t* sync_status;  // word set to 1 when a consumer's wait runs out (may be null)
  float* sync_part;
  uint16_t* sync_t16;
  int sync_blocks;
  // LoRA delta by the LoRA blocks of a split projection (direct-to-LDS kernel): once every slice of
  // x . A has arrived (sync, sync_t16 as above; lora_b, lora_r, lora_ls, seg_end as above), the LoRA
  // blocks share the columns of delta = bf16(bf16(t . B) * ls), [M][N] bf16, which the consumer adds
  // to the rounded sum of the planes instead of multiplying by B itself
  uint16_t* delta;
  int n_lora_slices;       // slices that hold k-tiles (the launch may have a few more LoRA blocks)
};

// What qlinear_base needs to let the LoRA blocks produce the delta (all or nothing).
struct LoraDelta {
  uint16_t* delta;         // [M][N] bf16 out
  const uint16_t* lora_b;  // [r][N]
  int r;
  float ls;
  int seg_end[3];          // column ends of the fused matrices (multiples of 32)
  void* sync_ws;           // qlinear_delta_sync_bytes(M, Rpad) bytes, first 16 zero between launches (the kernel leaves them so)
  uint32_t* status;        // may be null
};
size_t qlinear_delta_sync_bytes(int M, int Rpad);
// true when qlinear_base(..., &ld) with these shapes runs the kernel that fills ld.delta
bool qlinear_delta_ok(int M, int K, int N, int Rpad, int r, int nsplit);

// Routed experts (Qwen3 MoE): one launch multiplies, for every expert, the rows routed to it.
struct MoeArgs {
  const uint16_t* x;       // gate|up: normed hidden states [B, D]; down: activations [P, F]
  int ldx;
  const uint4* qw;         // [E] stacked q4t matrices
  const uint16_t* scales;  // [E] stacked scale arrays
  size_t qw_stride, sc_stride;  // elements between consecutive experts
  const int32_t* expert_of;     // [P] expert of pair p = token * top_k + slot
  int P, top_k;
  int K, N, G;             // per-expert matrix [K, N] (gate|up: N = 2 F)
  uint16_t* out;           // gate|up: act [P, F]; down: y [P, D]
  int ldo;
};

struct RouterArgs {
  const uint16_t* x;       // [B, D] normed hidden states
  const uint16_t* w;       // [D, E] bf16 router kernel
  int D, E, top_k;
  int32_t* expert_of;      // [B, top_k]
  float* weight_of;        // [B, top_k] renormalised routing weights (bf16 values)
};

// The LoRA-B half applied by the consumer of a projection.
struct LoraIn {
  const float* t_part;  // [nsplit][M][ldt] f32 planes of x . A (null: no LoRA)
  int ldt, nsplit;
  const uint16_t* b;    // [r][N] bf16
  int r;
  float ls;             // alpha / rank
};

struct RowNormArgs {
  // source of the row: an embedding gather (embed != null) or y (+ LoRA) (+ residual)
  const uint16_t* embed;        // [V, D]
  int vocab;                    // V (ids are clamped to [0, V)); 0: no clamp
  const int32_t* token_buffer;  // [B, L]
  const int32_t* step;          // device scalar: column of token_buffer to read
  int buf_len;
  int tpp;                      // tokens per pass: row m is sequence m / tpp at column *step + m % tpp (0: 1)
  const int32_t* positions;     // [B, L] (embedding mode: fills rope_tab)
  float* rope_tab;              // [B][half][2] sin, cos of this step (may be null)
  int half;
  float theta;
  const uint16_t* y_bf16;       // [M, D] base projection output, or
  const float* y_part;          // [nsplit][M][D] f32 planes
  int nsplit;
  LoraIn lora;
  const uint16_t* delta;        // [M, D] bf16 LoRA delta made by the projection (replaces lora), or null
  const uint16_t* moe_y;        // [M * top_k, D] routed-expert outputs (replaces y when set)
  const float* moe_w;           // [M * top_k] routing weights
  int top_k;
  const uint16_t* residual;     // [M, D] (null: none)
  uint16_t* x_out;              // [M, D] new residual stream (null: not stored)
  const uint16_t* norm_w;       // [D] (null: no norm output)
  uint16_t* xn_out;             // [M, D]
  int D;
  float eps;
  int family;
  RouterArgs router;            // router.w != null: the row's workgroup also routes the token from xn (MoE layers)
};

struct RopeArgs {
  const uint16_t* qkv_bf16;  // [B, (N + 2 Kh) * H], or
  const float* qkv_part;     // [nsplit][B][(N + 2 Kh) * H]
  int nsplit;
  LoraIn lora;               // t columns: x.A_q | x.A_k | x.A_v
  const uint16_t* q_norm_w;  // [H] (Qwen3) or null
  const uint16_t* k_norm_w;
  const int32_t* positions;  // [B, L]
  const int32_t* step;
  int buf_len;
  int tpp;                   // tokens per pass (0: 1): row m is sequence m / tpp at slot *step + m % tpp
  const float* rope_tab;     // [B][H/2][2] or null (then sin/cos are computed here)
  uint16_t* q_out;           // [B, N * H]
  uint16_t* kcache;          // [B, C, Kh, H]
  uint16_t* vcache;
  int N, Kh, H, C;
  float theta, eps;
  int family;
};

struct SwigluArgs {
  const uint16_t* gu_bf16;  // [M, 2F]: gate columns then up columns, or
  const float* gu_part;     // [nsplit][M][2F]
  int nsplit;
  LoraIn lora;              // t columns: x.A_gate | x.A_up
  uint16_t* act;            // [M, F]
  int F;
};

struct AttnArgs {
  const uint16_t* q;       // [B, N * H] bf16 (already rotated)
  const uint16_t* kcache;  // [B, C, Kh, H]
  const uint16_t* vcache;
  const uint8_t* input_mask;  // [B, L], 1 = real token
  const int32_t* step;        // device scalar: newest valid cache slot
  int buf_len;
  uint16_t* out;     // [B, N * H] bf16
  float* partial;    // [B, Kh, nsplit, G, H + 2] (nsplit > 1)
  int B, N, Kh, C, nsplit, chunk;
  float scale;
  int tpp;  // tokens per pass (0: 1): query row m belongs to sequence m / tpp and sees slots <= *step + m % tpp
  // Shared prompt slots (G samples of one prompt in consecutive rows): share_gs > 1 says that the sequences
  // come in consecutive groups of share_gs whose cache slots [0, share_len) and input_mask entries are
  // identical.  Those slots are then walked once per group (gqa_prefix_kernel, psplits splits, from the
  // group's first sequence), every row walks only its own slots share_len .. *step (nsplit splits), and
  // the nsplit + psplits partial results per row are merged by the rows' walk itself or the combine kernel.
  int share_gs, share_len, psplits;
};

struct HeadArgs {
  const uint16_t* x;  // [M, D] final-normed hidden states
  const uint16_t* w;  // [V, D]
  const uint16_t* w_tiles;  // the same matrix in the tile layout of head_tiles_kernel, or null
  int M, D, V;
  int mode;
  float temperature;
  uint32_t k0, k1;
  const int32_t* step;
  const int32_t* forbidden;
  int n_forbidden;
  float* logits_out;  // [M, V] raw f32 logits, optional
  uint16_t* sort_keys;  // [M, V] 16-bit descending key of every bf16 logit: set for the nucleus / top-k branch
  float* part_f;      // [M][nwg][4] = max, sumexp, best key, best z
  int32_t* part_i;    // [M][nwg]
  int nwg;
  // finalize
  int32_t* token_buffer;
  float* logprobs;
  uint8_t* done;
  const int32_t* eos;
  int n_eos;
  int buf_len;
  int tpp;  // tokens per pass (0: 1), score mode only: row m is sequence m / tpp at column *step + m % tpp
  int row_base;  // score mode: x holds rows row_base .. row_base + M - 1 of the pass (chunks of <= 128 rows)
  int row_off;   // set by head_logits when it splits the rows over two launches: x, logits_out, sort_keys and the
                 // partials point at row row_off of the call, whose index the sort keys and the noise counter use
};


struct NucleusArgs {
  const uint16_t* keys;  // [M, V] 16-bit descending keys of the bf16 logits (written by the head kernel)
  uint32_t* ent;         // [M][2 halves][3][32768]: key value | count prefix | mass prefix (f32 bits) of the populated values
  uint32_t* tot;         // [M][2][4]: populated values, candidates, mass (f32 bits), row maximum of z (f32 bits)
  float* pbest;          // [M][ns][4]: noisy key, z, rank (int bits) of each slice's winner
  int ns;                // slices of the rank range per row
  int M, V, k;           // k: candidates kept by top-k (V without top-k)
  float top_p;
  float temperature;     // the keys order the bf16 logits; z = logit / temperature
  uint32_t k0, k1;
  const int32_t* step;
  const float* part_f;   // head partials [M][nwg][4]
  int nwg;
  int32_t* token_buffer;
  float* logprobs;
  uint8_t* done;
  const int32_t* eos;
  int n_eos;
  int buf_len;
};

// One projection of the small-batch step (1..4 rows): prologue | int4 product + LoRA | epilogue in one launch.
struct SbLinearArgs {
  int M;
  const uint16_t* x;        // plain: activations [M, K]; norm: residual stream [M, K], normalised in the prologue
  int ldx;
  const uint16_t* norm_w;   // [K] (norm prologue)
  float eps;
  int family;
  const float* attn_part;   // attention prologue: [M][kh][ns][g][h + 2] split results (output | max | sum)
  int attn_kh, attn_g, attn_h, attn_ns;
  const uint4* qw;
  const uint16_t* scales;
  int K, N, G;
  const uint16_t* a_t;      // LoRA A, fragment order (null: t comes from t_parts, or no LoRA)
  int Rpad;
  const uint16_t* lora_b;   // [lora_r][N] (null: no LoRA)
  int lora_r;
  float lora_ls;
  int seg_end[3];           // column ends of the fused matrices; segment s uses t columns s lora_r ..
  const float* t_parts;     // [t_nparts][M][32] parts of t left by the previous launch (down projection)
  int t_nparts;
  const uint16_t* residual; // [M, N] (residual epilogue)
  uint16_t* y;              // [M, N]; SwiGLU epilogue: act [M, N / 2]
  int ldy;
  int pair_off;             // SwiGLU epilogue: tile distance between a gate tile and its up tile (N / 64)
  const uint16_t* a_next;   // SwiGLU epilogue: A of the next projection (r_pad 32), or null
  float* t_parts_out;       // [N / 64][M][32]
};

struct SbAttnArgs {
  const uint16_t* qkv;      // [B, (N + 2 Kh) H] with the LoRA deltas applied
  const float* rope_tab;    // [B][H / 2][2] sin, cos of this step
  uint16_t* kcache;         // [B, C, Kh, H]
  uint16_t* vcache;
  const uint8_t* input_mask;
  const int32_t* step;
  int buf_len;
  float* partial;           // [B][Kh][nsplit][G][H + 2]
  int B, N, Kh, C, nsplit;
  float scale;
  const uint16_t* q_norm_w;  // [H] per-head RMSNorm of q and k before the rotation (Qwen3), or null
  const uint16_t* k_norm_w;
  float eps;
  int family;                // rotation rounding: TMX_FAMILY_*
};

int sb_linear(hipStream_t st, const SbLinearArgs& a, int pro, int epi);  // pro: 0 plain, 1 norm, 2 attention merge; epi: 0 plain, 1 residual, 2 SwiGLU
bool sb_linear_ok(int M, int K, int N, int G, int rank, int rpad, bool norm);
int sb_attn(hipStream_t st, SbAttnArgs a, int H);
bool sb_attn_ok(int N, int Kh, int H);
int sb_attn_splits(int B, int Kh, int C);
size_t sb_attn_partial_bytes(int B, int N, int Kh, int H, int C);

int row_norm(hipStream_t st, const RowNormArgs& a, int M);
int rope_kvwrite(hipStream_t st, const RopeArgs& a, int B);
int swiglu(hipStream_t st, const SwigluArgs& a, int M);
int advance_step(hipStream_t st, int32_t* step, int by);
int empty_launch(hipStream_t st);  // measurement aid: a kernel that does nothing
int gqa_decode(hipStream_t st, AttnArgs a, int H);
size_t attn_partial_bytes(int B, int N, int Kh, int H, int C);
// the same when the rows may share prompt slots (AttnArgs::share_gs > 1): room for the prefix partials too
size_t attn_shared_partial_bytes(int B, int N, int Kh, int H, int C);
bool attn_share_ok(int B, int N, int Kh, int H, int C, int share_gs, int share_len);
int moe_route(hipStream_t st, const RouterArgs& a, int B);
int moe_experts(hipStream_t st, const MoeArgs& a, int E, bool down);
int head_sample(hipStream_t st, HeadArgs a);
// any number of rows in 256 x 256 blocks (greedy, sampling without the sorting branch, scoring); needs
// D % 128 == 0, no forbidden ids, no logits output; part_f / part_i sized [M][ceil(V / 256)]
int head_wide(hipStream_t st, HeadArgs a);
bool head_wide_ok(const HeadArgs& a);
int head_wide_logits(hipStream_t st, HeadArgs& a);  // the wide kernel without the finalize launch
int head_logits(hipStream_t st, HeadArgs& a);  // the vocabulary kernel alone; fills a.nwg
int head_sample_nucleus(hipStream_t st, HeadArgs a, float top_p, int top_k, void* ws, size_t ws_bytes);
size_t nucleus_bytes(int M, int V);
size_t head_partial_bytes(int M, int V);
int qlinear_num_splits(int K, int N, int M);
int qlinear_num_lora_splits(int K, int N);
// sync_ws: qlinear_gate_up_sync_bytes(M, K) bytes whose first 16 are zero between launches (the kernel
// leaves them so), or null: then every workgroup multiplies x by A itself
int qlinear_gate_up_swiglu(hipStream_t st, const void* x, int ldx, const void* qw, const void* scales,
                           const void* a_t, const void* lora_b, int r, float ls, void* act, int M, int K,
                           int F, int G, void* sync_ws, uint32_t* status = nullptr);
size_t qlinear_gate_up_sync_bytes(int M, int K);
int zero_words(hipStream_t st, uint32_t* p, int n);  // p[0 .. n) = 0 by a small kernel
int device_cus();  // compute units of the current device (256 when none answers)
// 0 when the fused gate | up launch cannot hand its LoRA projection over for this shape on this device
size_t qlinear_gate_up_handover_bytes(int M, int K, int F, int r);
// Many rows (M > 128), unsplit: y_bf16 = bf16(bf16(x . W) + bf16(bf16(t . B) ls)) in one pass, t = bf16(x . A)
// computed by a LoRA-only launch of the same kernel and a small reduction (t_part: f32 planes, t16: bf16
// [M][TMX_MAX_RPAD] scratch).  seg_end: column ends of the fused matrices (q | k | v, gate | up), unused
// entries = N.  TMX_ERR_UNSUPPORTED when the shape needs K-slices or the rank is not a multiple of 8.
int qlinear_wide_lora(hipStream_t st, const void* x, int ldx, const void* qw, const void* scales, const void* a_t,
                      const void* lora_b, int r, float ls, const int* seg_end, void* y_bf16, float* t_part,
                      uint16_t* t16, int M, int K, int N, int G, int Rpad);
int qlinear_base(hipStream_t st, const void* x, int ldx, const void* qw, const void* scales,
                 const void* a_t, void* y_bf16, float* y_part, float* t_part, int ldt, int M, int K,
                 int N, int G, int Rpad, int nsplit, const LoraDelta* ld = nullptr);

}  // namespace tmx
