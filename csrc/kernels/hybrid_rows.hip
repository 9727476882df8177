// Row kernels of the hybrid model family (windowed attention beside linear recurrences, state-space layers, one norm
// feeding mixer and feed-forward):
//
//   embed_norm          x = table[token] / rms * (offset + w)               (fp32 stream)
//   rms_norm_rows       norm of (gathered) stream rows into the activation dtype
//   residual_mix_norm   x += sa (a + bias) + sb b + sc c in fp32, and the next layer's normalised input from the same pass
//   qkv_rope_cache      bias + scaled interleaved-pair rotary of q / k, paged key / value cache write
//   gated_group_norm    silu gate and RMS norm over column groups, in either order
//   causal_conv_silu    per-channel causal convolution over a run of rows with carried taps, + silu
//   conv_state_update   the newest taps - 1 inputs of every run into its sequence's state slot
//   relu_sq, silu_mul   feed-forward activations on column ranges of a fused projection
//   softmax_topk        router: fp32 softmax over all outputs, choice by score + correction, weights = plain scores
//   moe_mix             weighted sum of the chosen experts' rows (identity experts: the input row) + gated shared expert
//   embed_scale         x = table[token] * scale                            (fp32 stream)
//   residual_conv       sublayer input x + causal per-channel convolution of the fp32 stream, carried taps fp32
//   post_rms_norm       norm after the sum: x = rms_norm(alpha x + delta) * w, in place on the fp32 stream
//   qk_norm_cache       per-head RMS norm of queries (times a per-head factor) and keys, paged key / value cache write
//   gelu_tanh_mul, sigmoid_mul   gated activations on column ranges of a fused projection
//
// One workgroup per row unless noted; columns strided over the threads (coalesced), any width.  All statistics,
// rotations, gates and sums are fp32; only the stored activations take the activation dtype T (bf16 or float).
#include "common.h"
#include "hybrid_launchers.h"

namespace {

constexpr int NT = 256;

SYM_DEV float ldf(const void* p, int f32, long long i) {
  return f32 ? reinterpret_cast<const float*>(p)[i] : (float)reinterpret_cast<const bf16*>(p)[i];
}

SYM_DEV float sigmoidf(float v) { return 1.f / (1.f + expf(-v)); }
SYM_DEV float silu_exact(float v) { return v / (1.f + expf(-v)); }
// 0.5 v (1 + tanh(u)) = v sigmoid(2 u), u = sqrt(2 / pi) (v + 0.044715 v^3)
SYM_DEV float gelu_tanh_exact(float v) {
  const float u = 0.7978845608028654f * (v + 0.044715f * v * v * v);
  return v / (1.f + expf(-2.f * u));
}

template <typename T, int BT>
__global__ __launch_bounds__(BT) void embed_norm_kernel(const int* __restrict__ ids, const int* __restrict__ src,
                                                        const int* __restrict__ prev, const T* __restrict__ table,
                                                        const float* __restrict__ w, float eps, float offset,
                                                        float* __restrict__ x, int d) {
  __shared__ float scratch[BT / 64];
  const int row = blockIdx.x;
  const int sr = src ? src[row] : -1;
  const long long tok = sr >= 0 ? prev[sr] : ids[row];
  const T* t = table + tok * d;
  float sq = 0.f;
  for (int c = threadIdx.x; c < d; c += BT) {
    const float v = (float)t[c];
    sq += v * v;
  }
  const float r = 1.f / sqrtf(block_sum<BT>(sq, scratch) / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += BT) x[(long long)row * d + c] = (float)t[c] * r * (offset + w[c]);
}

template <typename T, int BT>
__global__ __launch_bounds__(BT) void rms_norm_rows_kernel(const float* __restrict__ x, const long long* __restrict__ rows,
                                                           const float* __restrict__ w, float eps, float offset,
                                                           T* __restrict__ out, int d) {
  __shared__ float scratch[BT / 64];
  const int i = blockIdx.x;
  const float* xr = x + (rows ? rows[i] : (long long)i) * d;
  float sq = 0.f;
  for (int c = threadIdx.x; c < d; c += BT) sq += xr[c] * xr[c];
  const float r = 1.f / sqrtf(block_sum<BT>(sq, scratch) / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += BT) out[(long long)i * d + c] = (T)(xr[c] * r * (offset + w[c]));
}

template <typename T, int BT>
__global__ __launch_bounds__(BT) void residual_mix_norm_kernel(ResidualMixArgs a) {
  __shared__ float scratch[BT / 64];
  const int row = blockIdx.x, d = a.d;
  float* xr = a.x + (long long)row * d;
  const long long o = (long long)row * d;
  float sq = 0.f;
  for (int c = threadIdx.x; c < d; c += BT) {
    float s = ldf(a.a, a.a_f32, o + c);
    if (a.bias_a) s += a.bias_a[c];
    s *= a.sa;
    if (a.b) s += a.sb * ldf(a.b, a.b_f32, o + c);
    if (a.c) s += a.sc * ldf(a.c, a.c_f32, o + c);
    const float xn = xr[c] + s;
    xr[c] = xn;
    sq += xn * xn;
  }
  if (!a.out) return;
  const float r = 1.f / sqrtf(block_sum<BT>(sq, scratch) / (float)d + a.eps);
  T* out = reinterpret_cast<T*>(a.out) + o;
  // (each thread re-reads the columns it wrote itself)
  for (int c = threadIdx.x; c < d; c += BT) out[c] = (T)(xr[c] * r * (a.offset + a.w[c]));
}

template <typename T, int BT>
__global__ __launch_bounds__(BT) void qkv_rope_cache_kernel(QkvRopeArgs a) {
  const int row = blockIdx.x;
  const T* z = reinterpret_cast<const T*>(a.z) + (long long)row * a.ldz;
  const int nq = a.H * a.dk, nk = a.G * a.dk, nv = a.G * a.dv;
  const int rot = 2 * a.pairs;
  const float* cs = a.rope ? a.rope + (long long)a.positions[row] * rot : nullptr;   // [pairs][2]
  const int slot = a.slots[row];
  T* qo = reinterpret_cast<T*>(a.q_out) + (long long)row * nq;
  T* kc = slot >= 0 ? reinterpret_cast<T*>(a.k_cache) + (long long)slot * nk : nullptr;
  T* vc = slot >= 0 ? reinterpret_cast<T*>(a.v_cache) + (long long)slot * nv : nullptr;
  for (int i = threadIdx.x; i < nq + nk; i += BT) {
    const int e = i < nq ? i % a.dk : (i - nq) % a.dk;   // entry within its head
    float v = (float)z[i] + (a.bias ? a.bias[i] : 0.f);
    if (e < rot) {
      if (a.half) {                                      // entry e with entry e +- pairs, table pair e mod pairs
        const bool lo = e < a.pairs;
        const int j = lo ? i + a.pairs : i - a.pairs, pi = lo ? e : e - a.pairs;
        const float u = (float)z[j] + (a.bias ? a.bias[j] : 0.f);
        const float c = cs[2 * pi], s = cs[2 * pi + 1];
        v = lo ? v * c - u * s : v * c + u * s;
      } else {
        const int j = i - e + (e ^ 1);                   // the pair's other entry
        const float u = (float)z[j] + (a.bias ? a.bias[j] : 0.f);
        const float c = cs[e & ~1], s = cs[(e & ~1) + 1];
        v = (e & 1) ? v * c + u * s : v * c - u * s;
      }
    }
    if (i < nq) qo[i] = (T)v;
    else if (kc) kc[i - nq] = (T)v;
  }
  if (vc)
    for (int i = threadIdx.x; i < nv; i += BT)
      vc[i] = (T)((float)z[nq + nk + i] + (a.bias ? a.bias[nq + nk + i] : 0.f));
}

// grid (T, C / group); BT threads over the group's columns
template <typename T, int BT>
__global__ __launch_bounds__(BT) void gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ gate,
                                                              long long ldg, const float* __restrict__ w, int wlen,
                                                              float eps, int group, int gate_first, T* __restrict__ out,
                                                              int C) {
  __shared__ float scratch[BT / 64];
  const int row = blockIdx.x, c0 = blockIdx.y * group;
  const float* yr = y + (long long)row * C + c0;
  const T* gr = gate + (long long)row * ldg + c0;
  float sq = 0.f;
  for (int c = threadIdx.x; c < group; c += BT) {
    float v = yr[c];
    if (gate_first) v *= silu_exact((float)gr[c]);
    sq += v * v;
  }
  const float r = 1.f / sqrtf(block_sum<BT>(sq, scratch) / (float)group + eps);
  T* orow = out + (long long)row * C + c0;
  for (int c = threadIdx.x; c < group; c += BT) {
    const float g = silu_exact((float)gr[c]);
    const float wv = w[(c0 + c) % wlen];
    orow[c] = (T)(gate_first ? yr[c] * g * r * wv : yr[c] * r * wv * g);
  }
}

// grid (T, ceil(C / NT)): one thread per (row, channel)
template <typename T>
__global__ __launch_bounds__(NT) void causal_conv_silu_kernel(ConvArgs a) {
  const int row = blockIdx.x, c = blockIdx.y * NT + threadIdx.x;
  if (c >= a.C) return;
  const int s0 = a.cu_q ? a.cu_q[a.row_seq[row]] : row;
  const int j = row - s0, taps = a.taps;
  const int pr = a.prev_row[s0];
  const T* st = pr <= -2 ? reinterpret_cast<const T*>(a.state) + (long long)(-(pr + 2)) * a.state_stride : nullptr;
  const T* x = reinterpret_cast<const T*>(a.xin);
  const T* w = reinterpret_cast<const T*>(a.w) + (long long)c * taps;
  float acc = a.b[c];
  for (int i = 0; i < taps; ++i) {       // i positions back
    float v = 0.f;
    if (i <= j) v = (float)x[(long long)(row - i) * a.ldx + c];
    else if (st) v = (float)st[(long long)(taps - 1 - (i - j)) * a.C + c];
    acc += (float)w[taps - 1 - i] * v;
  }
  reinterpret_cast<T*>(a.out)[(long long)row * a.C + c] = (T)(acc * sigmoidf(acc));
}

constexpr int MAX_TAPS = 16;

// grid (runs, ceil(C / NT)): one thread per (run, channel) owns that channel of the run's state slot
template <typename T>
__global__ __launch_bounds__(NT) void conv_state_update_kernel(ConvArgs a) {
  const int run = blockIdx.x, c = blockIdx.y * NT + threadIdx.x;
  if (c >= a.C) return;
  const int s0 = a.cu_q ? a.cu_q[run] : run, s1 = a.cu_q ? a.cu_q[run + 1] : run + 1;
  if (s1 <= s0) return;
  const int sv = a.save_slot[s1 - 1];
  if (sv < 0) return;
  const int keep = a.taps - 1, n = s1 - s0;
  const int pr = a.prev_row[s0];
  T* base = reinterpret_cast<T*>(a.state);
  const T* old = pr <= -2 ? base + (long long)(-(pr + 2)) * a.state_stride : nullptr;
  const T* x = reinterpret_cast<const T*>(a.xin);
  T vals[MAX_TAPS];
#pragma unroll
  for (int m = 0; m < MAX_TAPS; ++m) {
    if (m < keep) {
      const int back = keep - m;       // 1 = the newest input
      T v = (T)0.f;
      if (back <= n) v = x[(long long)(s1 - back) * a.ldx + c];
      else if (old) v = old[(long long)(keep - (back - n)) * a.C + c];
      vals[m] = v;
    }
  }
  T* dst = base + (long long)sv * a.state_stride;
#pragma unroll
  for (int m = 0; m < MAX_TAPS; ++m)
    if (m < keep) dst[(long long)m * a.C + c] = vals[m];
}

template <typename T>
__global__ __launch_bounds__(NT) void relu_sq_kernel(const T* __restrict__ a, long long lda, T* __restrict__ out, int R,
                                                     int F) {
  const long long n = (long long)R * F;
  for (long long i = (long long)blockIdx.x * NT + threadIdx.x; i < n; i += (long long)gridDim.x * NT) {
    const long long r = i / F, c = i - r * F;
    const float v = fmaxf((float)a[r * lda + c], 0.f);
    out[i] = (T)(v * v);
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void silu_mul_kernel(const T* __restrict__ g, long long ldg, const T* __restrict__ u,
                                                      long long ldu, T* __restrict__ out, int R, int F) {
  const long long n = (long long)R * F;
  for (long long i = (long long)blockIdx.x * NT + threadIdx.x; i < n; i += (long long)gridDim.x * NT) {
    const long long r = i / F, c = i - r * F;
    const float gv = (float)g[r * ldg + c];
    out[i] = (T)(gv * sigmoidf(gv) * (float)u[r * ldu + c]);
  }
}

// x . w over d entries by one wave: 16-byte loads, several in flight (a decode step has a handful of rows, so the
// latency of a load after a load is what such a launch costs); any width and alignment through the scalar tail
template <typename T>
SYM_DEV float wave_dot(const T* __restrict__ x, const T* __restrict__ w, int d, int lane) {
  float acc = 0.f;
  int done = 0;
  if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) == 0) {
    if constexpr (sizeof(T) == 2) {
      const int nv = d >> 3;
#pragma unroll 4
      for (int i = lane; i < nv; i += 64) {
        float a[8], b[8];
        load8(reinterpret_cast<const bf16*>(x) + 8 * i, a);
        load8(reinterpret_cast<const bf16*>(w) + 8 * i, b);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc += a[j] * b[j];
      }
      done = nv << 3;
    } else {
      const int nv = d >> 2;
#pragma unroll 4
      for (int i = lane; i < nv; i += 64) {
        const float4 a = reinterpret_cast<const float4*>(x)[i], b = reinterpret_cast<const float4*>(w)[i];
        acc += a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
      }
      done = nv << 2;
    }
  }
  for (int c = done + lane; c < d; c += 64) acc += (float)x[c] * (float)w[c];
  return wave_sum(acc);
}

// One workgroup per token: the four waves share the router outputs (a wave per output, lanes over the width), then the
// first wave normalises and picks.  Dynamic LDS: En floats.  groups > keep: the outputs form equal groups of
// neighbours; the `keep` groups with the largest best entry (of score + correction) are picked first, and only their
// entries can be chosen.
template <typename T>
__global__ __launch_bounds__(NT) void softmax_topk_kernel(const T* __restrict__ x, const T* __restrict__ Wr,
                                                          const float* __restrict__ corr, int d, int En, int k, int groups,
                                                          int keep, int renorm, int* __restrict__ ids,
                                                          float* __restrict__ w) {
  extern __shared__ float sc[];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* xr = x + (long long)t * d;
  for (int e = wave; e < En; e += NT / 64) {
    const float acc = wave_dot<T>(xr, Wr + (long long)e * d, d, lane);
    if (lane == 0) sc[e] = acc;
  }
  __syncthreads();
  if (wave == 0) {
    float m = -INFINITY;
    for (int e = lane; e < En; e += 64) m = fmaxf(m, sc[e]);
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < En; e += 64) sum += expf(sc[e] - m);
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    for (int e = lane; e < En; e += 64) sc[e] = expf(sc[e] - m) * inv;   // (each lane rewrites the entries it read)
  }
  __syncthreads();
  if (wave) return;
  const bool grouped = groups > 1 && keep < groups;
  const int per = grouped ? En / groups : En;
  unsigned long long elig = ~0ull;   // bit g: group g's entries can be chosen (groups <= 64; the same in every lane)
  if (grouped) {
    float gbest = -INFINITY;         // lane g: the best entry of group g
    if (lane < groups)
      for (int e = lane * per; e < (lane + 1) * per; ++e) gbest = fmaxf(gbest, sc[e] + (corr ? corr[e] : 0.f));
    elig = 0;
    for (int j = 0; j < keep; ++j) {   // the keep best groups, one at a time (ties: the lowest index)
      float best = (lane < groups && !((elig >> lane) & 1)) ? gbest : -INFINITY;
      int bi = best > -INFINITY ? lane : 0x7fffffff;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
      }
      if (bi < groups) elig |= 1ull << bi;
    }
  }
  unsigned long long taken = 0;   // bit i: this lane's entry lane + 64 i is chosen (En <= 4096)
  float wsum = 0.f;
  for (int j = 0; j < k; ++j) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane, i = 0; e < En; e += 64, ++i) {
      if ((taken >> i) & 1) continue;
      if (grouped && !((elig >> (e / per)) & 1)) continue;
      const float v = sc[e] + (corr ? corr[e] : 0.f);
      if (v > best) { best = v; bi = e; }     // ascending e: the lowest index wins a tie within the lane
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    if (bi >= En) bi = j;   // only with non-finite scores: keep the id a valid segment index for the kernels downstream
    if ((bi & 63) == lane) taken |= 1ull << (bi >> 6);
    wsum += sc[bi];
    if (lane == 0) {
      ids[(long long)t * k + j] = bi;
      w[(long long)t * k + j] = sc[bi];
    }
  }
  if (renorm && lane == 0) {
    const float den = wsum + 1e-20f;
    for (int j = 0; j < k; ++j) w[(long long)t * k + j] = sc[ids[(long long)t * k + j]] / den;
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void moe_mix_kernel(const T* __restrict__ y, const int* __restrict__ dst,
                                                     const int* __restrict__ ids, const float* __restrict__ w, int k, int E,
                                                     const T* __restrict__ h, const T* __restrict__ shared,
                                                     const T* __restrict__ sgate, long long ldsg, float* __restrict__ out,
                                                     int d) {
  const int t = blockIdx.x;
  const float sg = shared ? sigmoidf((float)sgate[(long long)t * ldsg]) : 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    float acc = 0.f;
    for (int j = 0; j < k; ++j) {
      const long long a = (long long)t * k + j;
      const float v = ids[a] >= E ? (float)h[(long long)t * d + c] : (float)y[(long long)dst[a] * d + c];
      acc += w[a] * v;
    }
    if (shared) acc += sg * (float)shared[(long long)t * d + c];
    out[(long long)t * d + c] = acc;
  }
}

template <typename T, int BT>
__global__ __launch_bounds__(BT) void embed_scale_kernel(const int* __restrict__ ids, const int* __restrict__ src,
                                                         const int* __restrict__ prev, const T* __restrict__ table,
                                                         float scale, float* __restrict__ x, int d) {
  const int row = blockIdx.x;
  const int sr = src ? src[row] : -1;
  const long long tok = sr >= 0 ? prev[sr] : ids[row];
  const T* t = table + tok * d;
  for (int c = threadIdx.x; c < d; c += BT) x[(long long)row * d + c] = (float)t[c] * scale;
}

// grid (T, ceil(C / NT)): one thread per (row, channel).  x and the carried taps are fp32, the output takes the
// activation dtype: out = x + sum_i w[c][taps - 1 - i] x[t - i][c]
template <typename T>
__global__ __launch_bounds__(NT) void residual_conv_kernel(ConvArgs a) {
  const int row = blockIdx.x, c = blockIdx.y * NT + threadIdx.x;
  if (c >= a.C) return;
  const int s0 = a.cu_q ? a.cu_q[a.row_seq[row]] : row;
  const int j = row - s0, taps = a.taps;
  const int pr = a.prev_row[s0];
  const float* st = pr <= -2 ? reinterpret_cast<const float*>(a.state) + (long long)(-(pr + 2)) * a.state_stride : nullptr;
  const float* x = reinterpret_cast<const float*>(a.xin);
  const float* w = reinterpret_cast<const float*>(a.w) + c;     // [taps][C]
  float acc = x[(long long)row * a.ldx + c];
  for (int i = 0; i < taps; ++i) {       // i positions back
    float v = 0.f;
    if (i <= j) v = x[(long long)(row - i) * a.ldx + c];
    else if (st) v = st[(long long)(taps - 1 - (i - j)) * a.C + c];
    acc += w[(long long)(taps - 1 - i) * a.C] * v;
  }
  reinterpret_cast<T*>(a.out)[(long long)row * a.C + c] = (T)acc;
  // rows that are runs of their own (decode steps): this thread alone reads and writes its channel of the row's slot, so
  // the carried taps move on here (older ones one place down, the row's input on top)
  if (!a.cu_q && a.save_slot && taps > 1) {
    const int sv = a.save_slot[row];
    if (sv < 0) return;
    const int keep = taps - 1;
    float vals[MAX_TAPS];
#pragma unroll
    for (int m = 0; m < MAX_TAPS; ++m)
      if (m < keep) vals[m] = m + 1 < keep ? (st ? st[(long long)(m + 1) * a.C + c] : 0.f) : x[(long long)row * a.ldx + c];
    float* dst = reinterpret_cast<float*>(a.state) + (long long)sv * a.state_stride;
#pragma unroll
    for (int m = 0; m < MAX_TAPS; ++m)
      if (m < keep) dst[(long long)m * a.C + c] = vals[m];
  }
}

// The same for prompt-sized launches with C and the row stride multiples of 4: a thread takes four channels (16-byte
// loads of the stream and of the tap-major weights, which it keeps in registers) and walks CONV_ROWS consecutive rows,
// grid (ceil(T / CONV_ROWS), ceil(C / 4 / NT)).  The taps never move on here (runs of several rows).
constexpr int CONV_ROWS = 8;
template <typename T, int TAPS>     // TAPS: the tap count where it is at most 4, else 0 (any count up to MAX_TAPS)
__global__ __launch_bounds__(NT) void residual_conv_vec_kernel(ConvArgs a) {
  constexpr int NTAP = TAPS ? TAPS : MAX_TAPS;
  const int row0 = blockIdx.x * CONV_ROWS, c = (blockIdx.y * NT + threadIdx.x) * 4;
  if (c >= a.C) return;
  const int taps = TAPS ? TAPS : a.taps;
  const float* x = reinterpret_cast<const float*>(a.xin);
  float4 wv[NTAP];     // wv[i]: the weights of the input i positions back
#pragma unroll
  for (int i = 0; i < NTAP; ++i)
    if (i < taps)
      wv[i] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(a.w) + (long long)(taps - 1 - i) * a.C + c);
  for (int r = 0; r < CONV_ROWS; ++r) {
    const int row = row0 + r;
    if (row >= a.T) return;
    const int s0 = a.cu_q ? a.cu_q[a.row_seq[row]] : row;
    const int j = row - s0;
    const float* st = nullptr;
    if (j < taps - 1) {
      const int pr = a.prev_row[s0];
      if (pr <= -2) st = reinterpret_cast<const float*>(a.state) + (long long)(-(pr + 2)) * a.state_stride;
    }
    const float4 own = *reinterpret_cast<const float4*>(x + (long long)row * a.ldx + c);
    float4 acc = own;
#pragma unroll
    for (int i = 0; i < NTAP; ++i) {       // i positions back
      if (i < taps) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i == 0) v = own;
        else if (i <= j) v = *reinterpret_cast<const float4*>(x + (long long)(row - i) * a.ldx + c);
        else if (st) v = *reinterpret_cast<const float4*>(st + (long long)(taps - 1 - (i - j)) * a.C + c);
        const float4 wt = wv[i];
        acc.x += wt.x * v.x, acc.y += wt.y * v.y, acc.z += wt.z * v.z, acc.w += wt.w * v.w;
      }
    }
    T* o = reinterpret_cast<T*>(a.out) + (long long)row * a.C + c;
    if constexpr (sizeof(T) == 2) {
      bf16x4 pk;
      pk[0] = (bf16)acc.x, pk[1] = (bf16)acc.y, pk[2] = (bf16)acc.z, pk[3] = (bf16)acc.w;
      *reinterpret_cast<bf16x4*>(o) = pk;
    } else {
      *reinterpret_cast<float4*>(o) = acc;
    }
  }
}

// one workgroup per row; the row's sums stay in registers between the two passes (up to PER columns per thread, wider
// rows recompute)
template <typename T, int BT>
__global__ __launch_bounds__(BT) void post_rms_norm_kernel(float* __restrict__ x, float alpha, const T* __restrict__ delta,
                                                           const float* __restrict__ w, float eps, int d) {
  __shared__ float scratch[BT / 64];
  constexpr int PER = 8;
  const long long o = (long long)blockIdx.x * d;
  float v[PER];
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int c = threadIdx.x + i * BT;
    v[i] = c < d ? alpha * x[o + c] + (float)delta[o + c] : 0.f;
    sq += v[i] * v[i];
  }
  for (int c = threadIdx.x + PER * BT; c < d; c += BT) {
    const float u = alpha * x[o + c] + (float)delta[o + c];
    sq += u * u;
  }
  const float r = 1.f / sqrtf(block_sum<BT>(sq, scratch) / (float)d + eps);
  // (each thread rewrites only the columns it read itself)
  for (int c = threadIdx.x + PER * BT; c < d; c += BT) x[o + c] = (alpha * x[o + c] + (float)delta[o + c]) * r * w[c];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int c = threadIdx.x + i * BT;
    if (c < d) x[o + c] = v[i] * r * w[c];
  }
}

// The same for rows that are runs of their own (decode steps), and in the same launch the next sublayer's input
// h = x_new + conv(x_new) from the row's carried taps, which move on: a thread owns its columns of the row and of the
// row's slot.  One column pass of BT threads keeps its weights, taps and carried inputs in registers, loaded before the
// row's reduction so that only the arithmetic follows it; wider rows take further passes.  TAPS: the tap count where it
// is at most 8 (exact register arrays), 0 for any count up to MAX_TAPS.
template <typename T, int BT, int TAPS>
__global__ __launch_bounds__(BT) void post_rms_norm_conv_kernel(float* __restrict__ x, float alpha,
                                                                const T* __restrict__ delta, const float* __restrict__ w,
                                                                float eps, int d, NormConvArgs cv) {
  __shared__ float scratch[BT / 64];
  constexpr int KEEP = TAPS ? TAPS - 1 : MAX_TAPS - 1;
  const int row = blockIdx.x;
  const long long o = (long long)row * d;
  const int taps = TAPS ? TAPS : cv.taps, keep = taps - 1;
  const int pr = cv.prev_row[row], sv = cv.save_slot[row];
  const float* st = pr <= -2 ? cv.state + (long long)(-(pr + 2)) * cv.state_stride : nullptr;
  float* dst = sv >= 0 ? cv.state + (long long)sv * cv.state_stride : nullptr;
  const int c0 = threadIdx.x;
  float v0 = 0.f, w0 = 0.f, cw[KEEP + 1], old[KEEP];
  if (c0 < d) {
    v0 = alpha * x[o + c0] + (float)delta[o + c0];
    w0 = w[c0];
#pragma unroll
    for (int m = 0; m <= KEEP; ++m)
      if (m <= keep) cw[m] = cv.w[(long long)m * d + c0];
#pragma unroll
    for (int m = 0; m < KEEP; ++m)
      if (m < keep) old[m] = st ? st[(long long)m * d + c0] : 0.f;      // old[m]: the input keep - m positions back
  }
  float sq = v0 * v0;
  for (int c = c0 + BT; c < d; c += BT) {
    const float u = alpha * x[o + c] + (float)delta[o + c];
    sq += u * u;
  }
  const float r = 1.f / sqrtf(block_sum<BT>(sq, scratch) / (float)d + eps);
  T* h = reinterpret_cast<T*>(cv.h);
  for (int c = c0 + BT; c < d; c += BT) {     // further passes: loads after the reduction
    const float xn = (alpha * x[o + c] + (float)delta[o + c]) * r * w[c];
    const float* cwp = cv.w + c;      // [taps][d]
    float acc = xn + cwp[(long long)keep * d] * xn, prev = 0.f;
    for (int m = 0; m < keep; ++m) {
      const float ov = st ? st[(long long)m * d + c] : 0.f;
      acc += cwp[(long long)m * d] * ov;
      if (dst && m > 0) dst[(long long)(m - 1) * d + c] = ov;   // (this thread alone reads and writes column c of the slot)
      prev = ov;
    }
    (void)prev;
    if (dst && keep > 0) dst[(long long)(keep - 1) * d + c] = xn;
    x[o + c] = xn;
    h[o + c] = (T)acc;
  }
  if (c0 >= d) return;
  const float xn = v0 * r * w0;
  float acc = xn + cw[keep] * xn;
#pragma unroll
  for (int m = 0; m < KEEP; ++m)
    if (m < keep) acc += cw[m] * old[m];
  x[o + c0] = xn;
  h[o + c0] = (T)acc;
  if (dst) {
#pragma unroll
    for (int m = 0; m < KEEP; ++m)
      if (m < keep) dst[(long long)m * d + c0] = m + 1 < keep ? old[m + 1 < KEEP ? m + 1 : m] : xn;
  }
}

// grid (T, ceil((H + G) / 4)), 4 waves: one wave per query or key head normalises it (lanes over the head's entries);
// the workgroups then copy the value heads in strides.
template <typename T>
__global__ __launch_bounds__(NT) void qk_norm_cache_kernel(QkNormArgs a) {
  const int row = blockIdx.x, lane = threadIdx.x & 63;
  const int head = blockIdx.y * (NT / 64) + (threadIdx.x >> 6);
  const T* z = reinterpret_cast<const T*>(a.z) + (long long)row * a.ldz;
  const int slot = a.slots[row];
  const int nq = a.H * a.dk, nk = a.G * a.dk, nv = a.G * a.dv;
  if (head < a.H + a.G) {
    const bool isq = head < a.H;
    const T* src = z + (long long)head * a.dk;           // query heads, then key heads, contiguous
    float sq = 0.f;
    for (int e = lane; e < a.dk; e += 64) {
      const float v = (float)src[e];
      sq += v * v;
    }
    float r = 1.f / sqrtf(wave_sum(sq) / (float)a.dk + a.eps);
    const float* w = isq ? a.wq : a.wk;
    T* dst = nullptr;
    if (isq) {
      dst = reinterpret_cast<T*>(a.q_out) + ((long long)row * a.H + head) * a.dk;
      if (a.q_mult) r *= a.q_mult[head];
    } else if (slot >= 0) {
      dst = reinterpret_cast<T*>(a.k_cache) + ((long long)slot * a.G + (head - a.H)) * a.dk;
    }
    if (dst)
      for (int e = lane; e < a.dk; e += 64) dst[e] = (T)((float)src[e] * w[e] * r);
  }
  if (slot >= 0) {
    T* vc = reinterpret_cast<T*>(a.v_cache) + (long long)slot * nv;
    for (int i = blockIdx.y * NT + threadIdx.x; i < nv; i += gridDim.y * NT) vc[i] = z[nq + nk + i];
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void gelu_tanh_mul_kernel(const T* __restrict__ g, long long ldg, const T* __restrict__ u,
                                                           long long ldu, T* __restrict__ out, int R, int F) {
  const long long n = (long long)R * F;
  for (long long i = (long long)blockIdx.x * NT + threadIdx.x; i < n; i += (long long)gridDim.x * NT) {
    const long long r = i / F, c = i - r * F;
    const float gv = (float)g[r * ldg + c];
    out[i] = (T)(gelu_tanh_exact(gv) * (float)u[r * ldu + c]);
  }
}

// bf16, F and both row strides multiples of 8, 16-byte aligned views: eight columns per thread (prompt-sized launches
// are bandwidth-bound)
__global__ __launch_bounds__(NT) void gelu_tanh_mul_vec_kernel(const bf16* __restrict__ g, long long ldg,
                                                               const bf16* __restrict__ u, long long ldu,
                                                               bf16* __restrict__ out, long long nvec, int F) {
  const long long i = (long long)blockIdx.x * NT + threadIdx.x;
  if (i >= nvec) return;
  const int fv = F >> 3;
  const long long r = i / fv;
  const int c = (int)(i - r * fv) * 8;
  float gv[8], uv[8], y[8];
  load8(g + r * ldg + c, gv);
  load8(u + r * ldu + c, uv);
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = gelu_tanh_exact(gv[j]) * uv[j];
  store8(out + r * F + c, y);
}

template <typename T>
__global__ __launch_bounds__(NT) void sigmoid_mul_kernel(const T* a, long long lda, const T* __restrict__ g,
                                                         long long ldg, T* out, int R, int F) {
  const long long n = (long long)R * F;
  for (long long i = (long long)blockIdx.x * NT + threadIdx.x; i < n; i += (long long)gridDim.x * NT) {
    const long long r = i / F, c = i - r * F;
    out[i] = (T)((float)a[r * lda + c] * sigmoidf((float)g[r * ldg + c]));
  }
}

int ew_grid(long long n) {
  long long g = (n + NT - 1) / NT;
  return (int)(g < 1 ? 1 : (g > 16384 ? 16384 : g));
}

}  // namespace

// rows of a decode step: 1024 threads per row make a wide row one or two passes deep instead of eight
static inline bool wide_rows(int rows, int width) { return rows <= 512 && width >= 1024; }

#define DISPATCH_T(f32, ...)            \
  if (f32) {                            \
    using T = float;                    \
    __VA_ARGS__                         \
  } else {                              \
    using T = bf16;                     \
    __VA_ARGS__                         \
  }

void launch_embed_norm(const int* ids, const int* src, const int* prev, const void* table, const float* w, float eps,
                       float offset, float* x, int T_, int d, int f32, hipStream_t s) {
  if (T_ <= 0) return;
  if (wide_rows(T_, d)) {
    DISPATCH_T(f32, (embed_norm_kernel<T, 1024><<<T_, 1024, 0, s>>>(ids, src, prev, (const T*)table, w, eps, offset, x, d));)
  } else {
    DISPATCH_T(f32, (embed_norm_kernel<T, NT><<<T_, NT, 0, s>>>(ids, src, prev, (const T*)table, w, eps, offset, x, d));)
  }
}

void launch_rms_norm_rows(const float* x, const long long* rows, const float* w, float eps, float offset, void* out,
                          int n, int d, int f32, hipStream_t s) {
  if (n <= 0) return;
  if (wide_rows(n, d)) {
    DISPATCH_T(f32, (rms_norm_rows_kernel<T, 1024><<<n, 1024, 0, s>>>(x, rows, w, eps, offset, (T*)out, d));)
  } else {
    DISPATCH_T(f32, (rms_norm_rows_kernel<T, NT><<<n, NT, 0, s>>>(x, rows, w, eps, offset, (T*)out, d));)
  }
}

void launch_residual_mix_norm(const ResidualMixArgs& a, int f32, hipStream_t s) {
  if (a.T <= 0) return;
  if (wide_rows(a.T, a.d)) {
    DISPATCH_T(f32, (residual_mix_norm_kernel<T, 1024><<<a.T, 1024, 0, s>>>(a));)
  } else {
    DISPATCH_T(f32, (residual_mix_norm_kernel<T, NT><<<a.T, NT, 0, s>>>(a));)
  }
}

void launch_qkv_rope_cache(const QkvRopeArgs& a, int T_, int f32, hipStream_t s) {
  if (T_ <= 0) return;
  if (wide_rows(T_, a.H * a.dk)) {
    DISPATCH_T(f32, (qkv_rope_cache_kernel<T, 1024><<<T_, 1024, 0, s>>>(a));)
  } else {
    DISPATCH_T(f32, (qkv_rope_cache_kernel<T, NT><<<T_, NT, 0, s>>>(a));)
  }
}

void launch_gated_group_norm(const float* y, const void* gate, long long ldg, const float* w, int wlen, float eps,
                             int group, int gate_first, void* out, int T_, int C, int f32, hipStream_t s) {
  if (T_ <= 0) return;
  dim3 grid(T_, C / group);
  if (group <= 256) {
    DISPATCH_T(f32, (gated_group_norm_kernel<T, 64><<<grid, 64, 0, s>>>(y, (const T*)gate, ldg, w, wlen, eps, group,
                                                                          gate_first, (T*)out, C));)
  } else if (wide_rows(T_, group)) {
    DISPATCH_T(f32, (gated_group_norm_kernel<T, 1024><<<grid, 1024, 0, s>>>(y, (const T*)gate, ldg, w, wlen, eps, group,
                                                                              gate_first, (T*)out, C));)
  } else {
    DISPATCH_T(f32, (gated_group_norm_kernel<T, NT><<<grid, NT, 0, s>>>(y, (const T*)gate, ldg, w, wlen, eps, group,
                                                                          gate_first, (T*)out, C));)
  }
}

void launch_causal_conv_silu(const ConvArgs& a, int f32, hipStream_t s) {
  if (a.T <= 0) return;
  dim3 grid(a.T, (a.C + NT - 1) / NT);
  DISPATCH_T(f32, causal_conv_silu_kernel<T><<<grid, NT, 0, s>>>(a);)
}

void launch_conv_state_update(const ConvArgs& a, int f32, hipStream_t s) {
  if (a.runs <= 0 || a.taps <= 1) return;
  dim3 grid(a.runs, (a.C + NT - 1) / NT);
  DISPATCH_T(f32, conv_state_update_kernel<T><<<grid, NT, 0, s>>>(a);)
}

void launch_relu_sq(const void* a, long long lda, void* out, int R, int F, int f32, hipStream_t s) {
  if (R <= 0) return;
  DISPATCH_T(f32, relu_sq_kernel<T><<<ew_grid((long long)R * F), NT, 0, s>>>((const T*)a, lda, (T*)out, R, F);)
}

void launch_silu_mul(const void* gate, long long ldg, const void* up, long long ldu, void* out, int R, int F, int f32,
                     hipStream_t s) {
  if (R <= 0) return;
  DISPATCH_T(f32, silu_mul_kernel<T><<<ew_grid((long long)R * F), NT, 0, s>>>((const T*)gate, ldg, (const T*)up, ldu,
                                                                              (T*)out, R, F);)
}

void launch_softmax_topk(const void* x, const void* Wr, const float* corr, int T_, int d, int En, int k, int groups,
                         int keep, int renorm, int* ids, float* w, int f32, hipStream_t s) {
  if (T_ <= 0) return;
  const size_t lds = (size_t)En * sizeof(float);
  DISPATCH_T(f32, softmax_topk_kernel<T><<<T_, NT, lds, s>>>((const T*)x, (const T*)Wr, corr, d, En, k, groups, keep,
                                                             renorm, ids, w);)
}

void launch_moe_mix(const void* y, const int* dst, const int* ids, const float* w, int k, int E, const void* h,
                    const void* shared, const void* sgate, long long ldsg, float* out, int T_, int d, int f32,
                    hipStream_t s) {
  if (T_ <= 0) return;
  DISPATCH_T(f32, moe_mix_kernel<T><<<T_, NT, 0, s>>>((const T*)y, dst, ids, w, k, E, (const T*)h, (const T*)shared,
                                                     (const T*)sgate, ldsg, out, d);)
}

void launch_embed_scale(const int* ids, const int* src, const int* prev, const void* table, float scale, float* x, int T_,
                        int d, int f32, hipStream_t s) {
  if (T_ <= 0) return;
  if (wide_rows(T_, d)) {
    DISPATCH_T(f32, (embed_scale_kernel<T, 1024><<<T_, 1024, 0, s>>>(ids, src, prev, (const T*)table, scale, x, d));)
  } else {
    DISPATCH_T(f32, (embed_scale_kernel<T, NT><<<T_, NT, 0, s>>>(ids, src, prev, (const T*)table, scale, x, d));)
  }
}

void launch_residual_conv(const ConvArgs& a, int f32, hipStream_t s) {
  if (a.T <= 0) return;
  const bool moves = !a.cu_q && a.save_slot;      // the launch that also moves the taps on keeps one channel per thread
  if (!moves && a.T >= 256 && a.C % 4 == 0 && a.ldx % 4 == 0 && (reinterpret_cast<uintptr_t>(a.xin) & 15) == 0 &&
      (reinterpret_cast<uintptr_t>(a.state) & 15) == 0 && a.state_stride % 4 == 0 &&
      (reinterpret_cast<uintptr_t>(a.w) & 15) == 0 && (reinterpret_cast<uintptr_t>(a.out) & 15) == 0) {
    dim3 grid((a.T + CONV_ROWS - 1) / CONV_ROWS, (a.C / 4 + NT - 1) / NT);
    if (a.taps == 4) {
      DISPATCH_T(f32, (residual_conv_vec_kernel<T, 4><<<grid, NT, 0, s>>>(a));)
    } else if (a.taps == 3) {
      DISPATCH_T(f32, (residual_conv_vec_kernel<T, 3><<<grid, NT, 0, s>>>(a));)
    } else if (a.taps == 2) {
      DISPATCH_T(f32, (residual_conv_vec_kernel<T, 2><<<grid, NT, 0, s>>>(a));)
    } else {
      DISPATCH_T(f32, (residual_conv_vec_kernel<T, 0><<<grid, NT, 0, s>>>(a));)
    }
    return;
  }
  dim3 grid(a.T, (a.C + NT - 1) / NT);
  DISPATCH_T(f32, residual_conv_kernel<T><<<grid, NT, 0, s>>>(a);)
}

template <typename T, int BT>
static void post_rms_norm_conv_taps(float* x, float alpha, const void* delta, const float* w, float eps, int T_, int d,
                                    const NormConvArgs& cv, hipStream_t s) {
  switch (cv.taps) {
    case 2: post_rms_norm_conv_kernel<T, BT, 2><<<T_, BT, 0, s>>>(x, alpha, (const T*)delta, w, eps, d, cv); break;
    case 3: post_rms_norm_conv_kernel<T, BT, 3><<<T_, BT, 0, s>>>(x, alpha, (const T*)delta, w, eps, d, cv); break;
    case 4: post_rms_norm_conv_kernel<T, BT, 4><<<T_, BT, 0, s>>>(x, alpha, (const T*)delta, w, eps, d, cv); break;
    default: post_rms_norm_conv_kernel<T, BT, 0><<<T_, BT, 0, s>>>(x, alpha, (const T*)delta, w, eps, d, cv); break;
  }
}

void launch_post_rms_norm(float* x, float alpha, const void* delta, const float* w, float eps, int T_, int d,
                          const NormConvArgs& cv, int f32, hipStream_t s) {
  if (T_ <= 0) return;
  if (cv.h) {
    if (d > 256) {
      DISPATCH_T(f32, (post_rms_norm_conv_taps<T, 1024>(x, alpha, delta, w, eps, T_, d, cv, s));)
    } else {
      DISPATCH_T(f32, (post_rms_norm_conv_taps<T, NT>(x, alpha, delta, w, eps, T_, d, cv, s));)
    }
    return;
  }
  if (wide_rows(T_, d)) {
    DISPATCH_T(f32, (post_rms_norm_kernel<T, 1024><<<T_, 1024, 0, s>>>(x, alpha, (const T*)delta, w, eps, d));)
  } else {
    DISPATCH_T(f32, (post_rms_norm_kernel<T, NT><<<T_, NT, 0, s>>>(x, alpha, (const T*)delta, w, eps, d));)
  }
}

void launch_qk_norm_cache(const QkNormArgs& a, int T_, int f32, hipStream_t s) {
  if (T_ <= 0) return;
  dim3 grid(T_, (a.H + a.G + NT / 64 - 1) / (NT / 64));
  DISPATCH_T(f32, qk_norm_cache_kernel<T><<<grid, NT, 0, s>>>(a);)
}

void launch_gelu_tanh_mul(const void* gate, long long ldg, const void* up, long long ldu, void* out, int R, int F, int f32,
                          hipStream_t s) {
  if (R <= 0) return;
  const auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (!f32 && F % 8 == 0 && ldg % 8 == 0 && ldu % 8 == 0 && al(gate) && al(up) && al(out)) {
    const long long nvec = (long long)R * F / 8;
    gelu_tanh_mul_vec_kernel<<<(unsigned)((nvec + NT - 1) / NT), NT, 0, s>>>((const bf16*)gate, ldg, (const bf16*)up, ldu,
                                                                           (bf16*)out, nvec, F);
    return;
  }
  DISPATCH_T(f32, gelu_tanh_mul_kernel<T><<<ew_grid((long long)R * F), NT, 0, s>>>((const T*)gate, ldg, (const T*)up,
                                                                                   ldu, (T*)out, R, F);)
}

void launch_sigmoid_mul(const void* a, long long lda, const void* gate, long long ldg, void* out, int R, int F, int f32,
                        hipStream_t s) {
  if (R <= 0) return;
  DISPATCH_T(f32, sigmoid_mul_kernel<T><<<ew_grid((long long)R * F), NT, 0, s>>>((const T*)a, lda, (const T*)gate, ldg,
                                                                                 (T*)out, R, F);)
}
