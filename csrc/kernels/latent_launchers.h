// Host-side launch entry points of the kernels in seq_mix.hip, latent_attention.hip and glu_moe.hip: the
// mechanisms of models whose layers carry per-sequence state, attend over a cached low-rank latent, and feed
// forward through clamped gated units (dense, or routed by sigmoid scores).
//
// Every launcher enqueues on the given stream, allocates nothing and never synchronises (hipGraph-capturable).
// Activations are bf16 or fp32 (`f32` flag: the whole model in 32-bit); the residual stream, the carried
// state, norm statistics, rotary angles, router scores and attention scores / weights are always fp32.
// Shape preconditions are checked by the op layer (csrc/bindings/latent_ops.cpp) before any launch.
#pragma once
#include <hip/hip_runtime.h>

// ---- seq_mix.hip -------------------------------------------------------------------------------------
// x[row] = hist0[row] = table[token], token = src[row] >= 0 ? prev[src[row]] : ids[row]
void launch_embed_rows(const int* ids, const int* src, const int* prev, const void* table, float* x, float* hist0,
                       int T, int d, int f32, hipStream_t s);
// h = x + (x_prev - x) * mu;  prev_row[row] >= 0: that row of x; -1: zeros; <= -2: state[-(v + 2)]
void launch_token_shift(const float* x, const void* mu, const int* prev_row, const float* state, long long state_stride,
                        void* h, int T, int d, int f32, hipStream_t s);
// x += layer_norm(delta) * w, with optional (a) save of the old x rows into state[save[row]] (save >= 0),
// (b) depth mix: hist[idx] = x_new; x = sum_{j <= idx} coef[j] * hist[j], (c) activation-dtype copy of the result
void launch_add_layer_norm(const void* delta, int delta_f32, const void* w, float eps, float* x, const int* save,
                           float* state, long long state_stride, float* hist, long long hist_stride, const float* coef,
                           int hist_idx, void* out_act, int T, int d, int f32, hipStream_t s);
// out[i] = layer_norm(x[rows ? rows[i] : i]) * w
void launch_layer_norm(const float* x, const long long* rows, const void* w, float eps, void* out, int n, int d,
                       int f32, hipStream_t s);

// ---- latent_attention.hip ----------------------------------------------------------------------------
struct LatentPrepArgs {
  const void* z;        // [T][nz] projections of the mixer input: q latent | kv latent | shared rotary key
  int nz, q_rank, kv_rank, rot;  // nz: row stride of z; kv_rank == 0: no kv part (the layer attends another's cache)
  int half_dims;        // 0: rotary pairs (2i, 2i + 1); > 0: entry i pairs with i + half_dims / 2, later entries pass
  const void* wq;       // [q_rank] norm weight
  const void* wkv;      // [kv_rank]
  float eps;
  const int* positions;
  const int* slots;     // cache row of each token (-1: no write)
  const float* rope;    // [max_pos][rot / 2][2] cos, sin
  void* cq;             // [T][q_rank]
  void* cache;          // [rows][kv_rank + rot]
};
void launch_latent_prep(const LatentPrepArgs& a, int T, int f32, hipStream_t s);
// rotary of src[t][h][0..rot) -> dst[t][h][0..rot) (element strides given); half_dims as in LatentPrepArgs
void launch_rope_pairs(const void* src, long long s_t, long long s_h, void* dst, long long d_t, long long d_h,
                       const int* positions, const float* rope, int T, int H, int rot, int half_dims, int f32,
                       hipStream_t s);
struct LatentAttnArgs {
  const void* q;        // [T][H][Dk]: absorbed query (kv_rank) | rotated query (rot)
  const void* cache;    // [blocks][BS][Dk]
  const int* block_tables;  // [seqs][max_blocks]
  const int* row_seq;   // [T]
  const int* positions; // [T]: a row sees keys 0..position (window > 0: position - window + 1..position)
  int window;           // 0: no limit
  void* out;            // [T][H][kv_rank]: softmax-weighted sum of the latents
  float* part_o;        // split-KV partials (decode form): [T][H][parts][kv_rank], [T][H][parts][2]
  float* part_ml;
  int T, H, Dk, kv_rank, BS, max_blocks;
  int bs_shift;            // log2(BS), or -1 if BS is no power of two
  int parts, part_tokens;  // split-KV: partition p of a row covers part_tokens keys from first + p * part_tokens on,
                           // first = the row's first visible key
  float scale;
  // prompt form of the MFMA kernel: 64-row query tiles (sequence, first row within the sequence's run) over the
  // runs cu_q[seq] .. cu_q[seq + 1]; nullptr: one query row per sequence (decode steps)
  const int* tiles;
  const int* cu_q;
  int ntiles;
};
// impl: 0 = MFMA kernel where the shapes allow (bf16, Dk % 32 == 0, kv_rank % 16 == 0, Dk <= 576, kv_rank <= 512),
// 1 = always the one-wave-per-(row, head) kernel (all shapes, both dtypes).  Returns the implementation used.
int launch_latent_attn(const LatentAttnArgs& a, int f32, int impl, hipStream_t s);

// ---- glu_moe.hip -------------------------------------------------------------------------------------
// gu [R][2F] = gate | up  ->  out [R][F] = g' * sigmoid(alpha * g') * (u' + 1), g' = min(g, limit), u' = clamp(u, +-limit)
void launch_clamped_glu(const void* gu, void* out, int R, int F, float limit, float alpha, int f32, hipStream_t s);
// scores = sigmoid(x . Wr[e]) in fp32; the k largest -> ids [T][k], w [T][k]
void launch_sigmoid_topk(const void* x, const void* Wr, int T, int d, int E, int k, int* ids, float* w, int f32,
                         hipStream_t s);
// offsets [E + 1] = exclusive scan of the per-expert counts of ids [R]; cursor [E] = 0
void launch_expert_offsets(const int* ids, int R, int E, int* offsets, int* cursor, hipStream_t s);
// xs[dst[a]] = w[a] * x[a / k] with dst[a] = offsets[ids[a]] + (arrival order within the expert)
void launch_scatter_scaled(const void* x, const int* ids, const float* w, int k, int R, int d, const int* offsets,
                           int* cursor, void* xs, int* dst, int f32, hipStream_t s);
// y[r] = xs[r] @ W[e]^T for the rows r of expert e's segment (W [E][N][K])
void launch_grouped_linear(const void* xs, const void* W, const int* offsets, int E, int R, int N, int K, void* y,
                           int f32, hipStream_t s);
// out[t] = sum_j y[dst[t * k + j]] (+ extra[t])
void launch_gather_sum(const void* y, const int* dst, int k, const void* extra, float* out, int T, int d, int f32,
                       hipStream_t s);
