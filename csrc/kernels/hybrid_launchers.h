// Host-side launch entry points of the kernels in hybrid_rows.hip, stream_rows.hip, window_attention.hip and
// decay_scan.hip: the
// mechanisms of models that put windowed softmax attention beside linear recurrences with decaying state, use
// state-space layers with a carried convolution, and add mixer and feed-forward to the stream from one norm.
//
// Every launcher enqueues on the given stream, allocates nothing and never synchronises (hipGraph-capturable).
// Activations are bf16 or fp32 (`f32` flag: the whole model in 32-bit); the residual stream, recurrent states,
// norm statistics, rotary angles, decays, step sizes, router scores and attention scores / weights are always fp32.
// Inputs that are column ranges of a wider matrix carry their row stride (`ld`, in elements).  Shape preconditions
// are checked by the op layer (csrc/bindings/hybrid_ops.cpp) before any launch.
#pragma once
#include <hip/hip_runtime.h>

// ---- hybrid_rows.hip -----------------------------------------------------------------------------------
// x[row] = table[token] / rms * (offset + w), token = src[row] >= 0 ? prev[src[row]] : ids[row]
void launch_embed_norm(const int* ids, const int* src, const int* prev, const void* table, const float* w, float eps,
                       float offset, float* x, int T, int d, int f32, hipStream_t s);
// out[i] = x[rows ? rows[i] : i] / rms * (offset + w)
void launch_rms_norm_rows(const float* x, const long long* rows, const float* w, float eps, float offset, void* out,
                          int n, int d, int f32, hipStream_t s);
// x += sa * (a + bias_a) + sb * b + sc * c (bias_a, b, c optional; each of a, b, c bf16 or fp32: *_f32);
// out (optional, activation dtype) = x_new / rms * (offset + w)
struct ResidualMixArgs {
  float* x;
  const void* a; int a_f32; float sa; const float* bias_a;
  const void* b; int b_f32; float sb;
  const void* c; int c_f32; float sc;
  const float* w; float eps, offset;
  void* out;
  int T, d;
};
void launch_residual_mix_norm(const ResidualMixArgs& a, int f32, hipStream_t s);
// z[t] = q (H dk) | k (G dk) | v (G dv), + bias (optional); q and k turn on their first 2 * pairs entries by
// rope[pos][pair] (optional): entries (2i, 2i + 1) together, or with `half` entry i with entry i + pairs;
// q -> q_out [T][H][dk]; k, v -> cache rows `slot` (>= 0) of k_cache [rows][G][dk], v_cache [rows][G][dv]
struct QkvRopeArgs {
  const void* z; long long ldz;
  const float* bias;
  int H, G, dk, dv, pairs, half;
  const int* positions;
  const int* slots;
  const float* rope;   // [max_pos][pairs][2] cos, sin (scaled)
  void* q_out;
  void* k_cache;
  void* v_cache;
};
void launch_qkv_rope_cache(const QkvRopeArgs& a, int T, int f32, hipStream_t s);
// s = silu(gate); gate_first: out = rms_g(y s) w, else out = rms_g(y) w s; rms over groups of `group` columns,
// w [wlen] repeating over the columns
void launch_gated_group_norm(const float* y, const void* gate, long long ldg, const float* w, int wlen, float eps,
                             int group, int gate_first, void* out, int T, int C, int f32, hipStream_t s);
// run i = rows cu_q[i] .. cu_q[i + 1] (cu_q null: row i alone); inputs before a run: state[slot] [taps - 1][C] where
// prev_row[first] <= -2 (slot = -(v + 2)), else zero.  out = silu(b + sum_j w[c][taps - 1 - j] x[t - j][c])
struct ConvArgs {
  const void* xin; long long ldx;
  const void* w;       // [C][taps] activation dtype
  const float* b;      // [C]
  void* state;         // [slots][taps - 1][C] activation dtype
  long long state_stride;
  const int* cu_q;
  const int* row_seq;
  const int* prev_row;
  const int* save_slot;
  void* out;           // [T][C]
  int T, C, taps, runs;
};
void launch_causal_conv_silu(const ConvArgs& a, int f32, hipStream_t s);
void launch_conv_state_update(const ConvArgs& a, int f32, hipStream_t s);
// out = relu(a)^2
void launch_relu_sq(const void* a, long long lda, void* out, int R, int F, int f32, hipStream_t s);
// out = silu(gate) * up
void launch_silu_mul(const void* gate, long long ldg, const void* up, long long ldu, void* out, int R, int F, int f32,
                     hipStream_t s);
// s = softmax(x . Wr[e]) over En outputs (fp32); the k largest of s + corr (corr optional; ties: lowest index) -> ids,
// w = their s (renorm: over their sum + 1e-20).  groups > 1: the outputs form equal groups of neighbours, and only
// entries of the `keep` groups with the largest best entry can be chosen
void launch_softmax_topk(const void* x, const void* Wr, const float* corr, int T, int d, int En, int k, int groups,
                         int keep, int renorm, int* ids, float* w, int f32, hipStream_t s);
// out[t] = sum_j w[a] * (ids[a] >= E ? h[t] : y[dst[a]]) + sigmoid(sgate[t]) * shared[t], a = t k + j
void launch_moe_mix(const void* y, const int* dst, const int* ids, const float* w, int k, int E, const void* h,
                    const void* shared, const void* sgate, long long ldsg, float* out, int T, int d, int f32,
                    hipStream_t s);

// x[row] = table[token] * scale, token as for launch_embed_norm
void launch_embed_scale(const int* ids, const int* src, const int* prev, const void* table, float scale, float* x, int T,
                        int d, int f32, hipStream_t s);
// ConvArgs with xin / state / w fp32, w tap-major [taps][C], no bias: out (activation dtype) = x + sum_j w[taps - 1 - j][c]
// x[t - j][c];
// the carried taps are then stored by launch_conv_state_update(a, 1, s) -- or by this launch itself where every row is a
// run of its own (cu_q null) and save_slot is given
void launch_residual_conv(const ConvArgs& a, int f32, hipStream_t s);
// x = (alpha x + delta) / rms * w, in place on the fp32 stream (delta in the activation dtype).  With cv.h set (every row
// a run of its own): also h = x_new + conv(x_new) over the row's carried taps (as launch_residual_conv), which move on
struct NormConvArgs {
  const float* w;        // [taps][d]
  float* state;          // [slots][taps - 1][d]
  long long state_stride;
  const int* prev_row;
  const int* save_slot;
  void* h;               // [T][d] activation dtype, or null: no convolution
  int taps;
};
void launch_post_rms_norm(float* x, float alpha, const void* delta, const float* w, float eps, int T, int d,
                          const NormConvArgs& cv, int f32, hipStream_t s);
// z[t] = q (H dk) | k (G dk) | v (G dv); q_out [T][H][dk] = q / rms_head * wq * q_mult[h]; cache rows `slot` (>= 0):
// k_cache [rows][G][dk] = k / rms_head * wk, v_cache [rows][G][dv] = v
struct QkNormArgs {
  const void* z; long long ldz;
  int H, G, dk, dv;
  const float* wq;      // [dk]
  const float* wk;      // [dk]
  const float* q_mult;  // [H] or null
  float eps;
  const int* slots;
  void* q_out;
  void* k_cache;
  void* v_cache;
};
void launch_qk_norm_cache(const QkNormArgs& a, int T, int f32, hipStream_t s);
// out = gelu_tanh(gate) * up
void launch_gelu_tanh_mul(const void* gate, long long ldg, const void* up, long long ldu, void* out, int R, int F, int f32,
                          hipStream_t s);
// out = a * sigmoid(gate) (out may be a)
void launch_sigmoid_mul(const void* a, long long lda, const void* gate, long long ldg, void* out, int R, int F, int f32,
                        hipStream_t s);

// ---- window_attention.hip ------------------------------------------------------------------------------
struct WindowAttnArgs {
  const void* q;        // [T][H][dk]
  const void* k_cache;  // [blocks][BS][G][dk]
  const void* v_cache;  // [blocks][BS][G][dv]
  const int* block_tables;  // [seqs][max_blocks]
  const int* row_seq;   // [T]
  const int* positions; // [T]: row sees positions max(0, p - window + 1) .. p
  const void* gate;     // [T][H] (row stride ldg) or null: output times sigmoid(gate)
  long long ldg;
  const float* bias;    // [2][H] or null: score of a key at distance n lowered by bias[0][h] * ln(1 + bias[1][h] * n)
  const float* sink;    // [H] or null: the softmax's denominator also holds exp(sink[h])
  void* out;            // [T][H][dv]
  int T, H, G, dk, dv, BS, max_blocks, window;
  int keep_first;       // positions 0 .. keep_first - 1 of the sequence stay visible past the window
  int bs_shift;         // log2(BS), or -1 if BS is no power of two (set by the launcher)
  float scale;
  // packed prompt form for the tiled kernel: 64-row query tiles (sequence, first row within the run)
  const int* tiles;
  const int* cu_q;
  int ntiles;
};
// Returns the implementation used: 0 = one wave per (row, head) (all shapes, both dtypes), 1 = tiled MFMA (bf16).
int launch_window_attn(const WindowAttnArgs& a, int f32, int impl, hipStream_t s);

// ---- decay_scan.hip ------------------------------------------------------------------------------------
struct DecayScanArgs {
  int mode;             // 0: decay per key channel = sigmoid(dz + dbias)^(1 / tau); 1: step size b = softplus(dz +
                        // dbias[h]), decay per head = exp(-exp(rate[h]) b), input scaled by b; 2: log gates
                        // i = tau tanh((dz[h] + dbias[h]) / tau), f = logsigmoid(tau tanh((dz[H + h] + dbias[H + h]) / tau))
                        // with the running maximum m_t = max(f + m_(t-1), i): decay exp(f + m_(t-1) - m_t), input scaled
                        // by exp(i - m_t); dz fp32 [T][2 H]; value column `vcols` is fed by 1 (the normaliser), state row N
                        // carries m (the same value in every column), mout [T][H] receives m_t
  const void* q; long long ldq;   // [T][(H / hpg) N]
  const void* k; long long ldk;
  const void* v; long long ldv;   // [T][H P]
  const void* dz; long long ldd;  // mode 0: [T][H N]; mode 1: [T][H]
  const float* dbias;   // mode 0: [H N]; mode 1: [H]
  const float* rate;    // mode 1: [H]
  float tau;            // mode 0; mode 2: the gates' soft cap
  const float* skip;    // [H] or null: out += skip[h] * v
  float q_scale;
  int H, N, P, hpg;     // P: columns of the state and of out (mode 2: vcols + 1)
  int vcols;            // columns of v
  float* mout;          // mode 2
  float* state;         // [slots][H][N][P] (mode 2: [slots][H][N + 1][P])
  long long state_stride;
  const int* cu_q;      // runs (null: every row its own run)
  const int* prev_row;
  const int* save_slot;
  int runs, T;
  float* out;           // [T][H][P]
};
void launch_decay_scan(const DecayScanArgs& a, int f32, hipStream_t s);

// ---- stream_rows.hip -----------------------------------------------------------------------------------
// x[row][s] (s < S) = table[token] + pair_table[(p mul_prev + token mul_cur) mod buckets]; p = the token of row
// prev_row[row] (>= 0), tok_state[-(prev_row[row] + 2)] (<= -2) or none (-1: row `buckets` of pair_table); pair_table null:
// the token rows alone.  save_slot (rows that are runs of their own): tok_state[save_slot[row]] = token
struct PairHashArgs {
  const int* ids; const int* src; const int* prev;
  const void* table;
  const void* pair_table;
  long long buckets, mul_prev, mul_cur;
  const int* prev_row;
  int* tok_state;
  const int* save_slot;
  float* x;             // [T][S][d]
  int T, S, d;
};
void launch_embed_pair_hash(const PairHashArgs& a, int f32, hipStream_t s);
// tok_state[save_slot[last]] = ids[last] for every run cu_q[i] .. cu_q[i + 1]
void launch_token_state_update(const int* ids, int* tok_state, const int* cu_q, const int* save_slot, int runs,
                               hipStream_t s);
// Residual streams xs [T][S][d].  With a: y = sa a + sb b (b optional), xs[.][t] = sum_s mix[s][t] xs[.][s] + outc[t] y
// for the rows < T.  With out: out[i] = rms_norm(sum_s inc[s] xs[rows ? rows[i] : i][s]) * w for i < n (inc null: ones)
struct HyperMixArgs {
  float* xs;
  const void* a; int a_f32; float sa;
  const void* b; int b_f32; float sb;
  const float* mix;     // [S][S] indexed [from][to]
  const float* outc;    // [S]
  const float* inc;     // [S] or null
  const float* w; float eps;
  const long long* rows;
  void* out;            // [n][d] activation dtype
  int T, n, S, d;
};
void launch_hyper_mix_norm(const HyperMixArgs& a, int f32, hipStream_t s);
// z[t] = q (H dk) | k (G dk) | v (G dv) through y_t = sum_j w[c][j] z_(t - taps + 1 + j) over every run (inputs before a
// run from state[slot] [taps - 1][C] where prev_row[first] <= -2, else zero); q -> q_out, k and v / rms_head(v) -> the
// cache rows `slot` (>= 0).  save_slot with cu_q null: the launch moves the row's carried taps on itself
struct ConvQkvArgs {
  const void* z; long long ldz;
  const void* w;        // [C][taps] activation dtype
  void* state;          // [slots][taps - 1][C] activation dtype
  long long state_stride;
  const int* cu_q;
  const int* row_seq;
  const int* prev_row;
  const int* save_slot;
  const int* slots;
  void* q_out;
  void* k_cache;
  void* v_cache;
  float v_eps;
  int T, C, taps, H, G, dk, dv;
};
void launch_conv_qkv_cache(const ConvQkvArgs& a, int f32, hipStream_t s);
// y [T][H][P + 1] (column P: n . q), m [T][H]: out = y / (max(|n . q|, exp(-m)) + 1e-6) / rms_head * w * sigmoid(gate)
void launch_memory_norm_gate(const float* y, const float* m, const void* gate, long long ldg, const float* w, float eps,
                             void* out, int T, int H, int P, int f32, hipStream_t s);
// x = cap tanh(x / cap)
void launch_logit_softcap(float* x, long long n, float cap, hipStream_t s);
// glu_moe.hip (declared with the latent family's launchers): launch_clamped_glu, the expert-segment kernels
