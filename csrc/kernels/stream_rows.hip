// Row kernels of models with several residual streams, a hashed token-pair embedding, convolved attention projections
// and a matrix memory with a normaliser:
//
//   embed_pair_hash      every stream = table[token] + pair_table[hash(previous token, token)]   (fp32 streams)
//   token_state_update   a run's last token into its sequence's state slot
//   hyper_mix_norm       streams <- streams M + c_out y (all at once), and the next sublayer's input rms_norm(c_in . streams)
//                        from the same pass; also the plain gathered sum + norm in front of the output head
//   conv_qkv_cache       causal per-channel convolution of q | k | v with carried taps, unit-RMS value heads, paged cache write
//                        (a workgroup per (row, head))
//   memory_norm_gate     o / (max(|n . q|, exp(-m)) + 1e-6), unit RMS per head, weight, sigmoid gate
//   logit_softcap        cap tanh(logits / cap)
//
// One workgroup per row unless noted; columns strided over the threads (coalesced), any width.  All statistics, mixing
// and sums are fp32; only the stored activations take the activation dtype T (bf16 or float).
#include "common.h"
#include "hybrid_launchers.h"

namespace {

constexpr int NT = 256;
constexpr int MAX_S = 8;      // residual streams
constexpr int MAX_TAPS = 16;

SYM_DEV float ldf(const void* p, int f32, long long i) {
  return f32 ? reinterpret_cast<const float*>(p)[i] : (float)reinterpret_cast<const bf16*>(p)[i];
}
SYM_DEV float sigmoidf(float v) { return 1.f / (1.f + expf(-v)); }

SYM_DEV long long token_of(const int* ids, const int* src, const int* prev, int row) {
  const int sr = src ? src[row] : -1;
  return sr >= 0 ? prev[sr] : ids[row];
}

template <typename T, int BT>
__global__ __launch_bounds__(BT) void embed_pair_hash_kernel(PairHashArgs a) {
  const int row = blockIdx.x, d = a.d, S = a.S;
  const long long tok = token_of(a.ids, a.src, a.prev, row);
  long long prow = -1;
  if (a.pair_table) {
    const int pr = a.prev_row[row];
    if (pr == -1) {
      prow = a.buckets;
    } else {
      const long long ptok = pr >= 0 ? token_of(a.ids, a.src, a.prev, pr) : a.tok_state[-(pr + 2)];
      const long long n = a.buckets;
      prow = ((ptok * a.mul_prev + tok * a.mul_cur) % n + n) % n;
    }
  }
  const T* t = reinterpret_cast<const T*>(a.table) + tok * d;
  const T* pt = prow >= 0 ? reinterpret_cast<const T*>(a.pair_table) + prow * d : nullptr;
  float* x = a.x + (long long)row * S * d;
  for (int c = threadIdx.x; c < d; c += BT) {
    float v = (float)t[c];
    if (pt) v += (float)pt[c];
    for (int s = 0; s < S; ++s) x[(long long)s * d + c] = v;
  }
  // rows that are runs of their own: the row's token becomes the carried one (after every thread has read the old one)
  if (a.save_slot) {
    __syncthreads();
    const int sv = a.save_slot[row];
    if (threadIdx.x == 0 && sv >= 0) a.tok_state[sv] = (int)tok;
  }
}

__global__ __launch_bounds__(NT) void token_state_update_kernel(const int* __restrict__ ids, int* __restrict__ tok_state,
                                                                const int* __restrict__ cu_q,
                                                                const int* __restrict__ save_slot, int runs) {
  const int run = blockIdx.x * NT + threadIdx.x;
  if (run >= runs) return;
  const int s0 = cu_q ? cu_q[run] : run, s1 = cu_q ? cu_q[run + 1] : run + 1;
  if (s1 <= s0) return;
  const int sv = save_slot[s1 - 1];
  if (sv >= 0) tok_state[sv] = ids[s1 - 1];
}

// Dynamic LDS: d floats (the mixed input u of the row, kept between the two passes) + S S + 2 S floats.
template <typename T, int BT>
__global__ __launch_bounds__(BT) void hyper_mix_norm_kernel(HyperMixArgs a) {
  extern __shared__ float lds[];
  __shared__ float scratch[BT / 64];
  const int row = blockIdx.x, d = a.d, S = a.S;
  float* us = lds;                 // [d]
  float* ms = lds + d;             // [S][S] mix, then [S] outc, [S] inc
  const bool upd = a.a != nullptr && row < a.T;
  const bool emit = a.out != nullptr && row < a.n;
  for (int i = threadIdx.x; i < S * S + 2 * S; i += BT) {
    float v = 1.f;
    if (i < S * S) v = a.mix ? a.mix[i] : 0.f;
    else if (i < S * S + S) v = a.outc ? a.outc[i - S * S] : 0.f;
    else v = a.inc ? a.inc[i - S * S - S] : 1.f;
    ms[i] = v;
  }
  __syncthreads();
  const float* outc = ms + S * S;
  const float* inc = outc + S;
  const long long xrow = a.rows ? a.rows[row] : (long long)row;
  float* x = a.xs + xrow * S * d;
  const long long o = (long long)row * d;
  float sq = 0.f;
  for (int c = threadIdx.x; c < d; c += BT) {
    float xv[MAX_S];
#pragma unroll
    for (int s = 0; s < MAX_S; ++s)
      if (s < S) xv[s] = x[(long long)s * d + c];
    if (upd) {
      float y = a.sa * ldf(a.a, a.a_f32, o + c);
      if (a.b) y += a.sb * ldf(a.b, a.b_f32, o + c);
      float nv[MAX_S];
#pragma unroll
      for (int t = 0; t < MAX_S; ++t) {
        if (t < S) {
          float acc = outc[t] * y;
#pragma unroll
          for (int s = 0; s < MAX_S; ++s)
            if (s < S) acc += ms[s * S + t] * xv[s];
          nv[t] = acc;
        }
      }
#pragma unroll
      for (int t = 0; t < MAX_S; ++t)
        if (t < S) {
          xv[t] = nv[t];
          x[(long long)t * d + c] = nv[t];
        }
    }
    if (emit) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < MAX_S; ++s)
        if (s < S) u += inc[s] * xv[s];
      us[c] = u;
      sq += u * u;
    }
  }
  if (!emit) return;     // (row-uniform)
  const float r = 1.f / sqrtf(block_sum<BT>(sq, scratch) / (float)d + a.eps);
  T* out = reinterpret_cast<T*>(a.out) + o;
  // (each thread re-reads the columns it wrote itself)
  for (int c = threadIdx.x; c < d; c += BT) out[c] = (T)(us[c] * r * a.w[c]);
}

// grid (T, H + 2 G): one workgroup of CQ threads per (row, head of q | k | v), a thread per channel (wider heads: several).
// A value head is brought to unit RMS before it is stored.  The small workgroups give a decode step's few rows a few
// hundred of them; a thread's taps and carried inputs are loads that do not depend on one another.
constexpr int CQ = 128;
constexpr int CQ_PER = 4;     // channels per thread kept in registers: heads up to 512 wide
template <typename T>
__global__ __launch_bounds__(CQ) void conv_qkv_cache_kernel(ConvQkvArgs a) {
  __shared__ float scratch[CQ / 64];
  const int row = blockIdx.x, unit = blockIdx.y, C = a.C, taps = a.taps;
  const int nq = a.H * a.dk, nk = a.G * a.dk;
  // the unit's channels [c0, c0 + width) and where they go
  int c0, width;
  T* dst_out;
  const int slot = a.slots[row];
  bool vhead = false;
  if (unit < a.H) {
    c0 = unit * a.dk, width = a.dk;
    dst_out = reinterpret_cast<T*>(a.q_out) + (long long)row * nq + c0;
  } else if (unit < a.H + a.G) {
    const int g = unit - a.H;
    c0 = nq + g * a.dk, width = a.dk;
    dst_out = slot >= 0 ? reinterpret_cast<T*>(a.k_cache) + (long long)slot * nk + g * a.dk : nullptr;
  } else {
    const int g = unit - a.H - a.G;
    c0 = nq + nk + g * a.dv, width = a.dv;
    dst_out = slot >= 0 ? reinterpret_cast<T*>(a.v_cache) + ((long long)slot * a.G + g) * a.dv : nullptr;
    vhead = true;
  }
  const int s0 = a.cu_q ? a.cu_q[a.row_seq[row]] : row;
  const int j = row - s0;
  const int pr = a.prev_row[s0];
  const T* st = pr <= -2 ? reinterpret_cast<const T*>(a.state) + (long long)(-(pr + 2)) * a.state_stride : nullptr;
  const T* z = reinterpret_cast<const T*>(a.z);
  const T* w = reinterpret_cast<const T*>(a.w);
  const int sv = (!a.cu_q && a.save_slot) ? a.save_slot[row] : -1;
  T* dst = sv >= 0 ? reinterpret_cast<T*>(a.state) + (long long)sv * a.state_stride : nullptr;
  float y[CQ_PER];
  float sq = 0.f;
#pragma unroll
  for (int u = 0; u < CQ_PER; ++u) {
    const int e = threadIdx.x + u * CQ;
    y[u] = 0.f;
    if (e < width) {
      const int c = c0 + e;
      float acc = 0.f;
      for (int i = 0; i < taps; ++i) {       // i positions back
        float v = 0.f;
        if (i <= j) v = (float)z[(long long)(row - i) * a.ldz + c];
        else if (st) v = (float)st[(long long)(taps - 1 - (i - j)) * C + c];
        acc += (float)w[(long long)c * taps + taps - 1 - i] * v;
      }
      y[u] = acc;
      sq += acc * acc;
      // rows that are runs of their own: this thread alone reads and writes its channel of the row's slot, so the
      // carried taps move on here (older ones one place down, the row's input on top)
      if (dst && taps > 1) {
        const int keep = taps - 1;
        T vals[MAX_TAPS];
#pragma unroll
        for (int m = 0; m < MAX_TAPS; ++m)
          if (m < keep) vals[m] = m + 1 < keep ? (st ? st[(long long)(m + 1) * C + c] : (T)0.f) : z[(long long)row * a.ldz + c];
#pragma unroll
        for (int m = 0; m < MAX_TAPS; ++m)
          if (m < keep) dst[(long long)m * C + c] = vals[m];
      }
    }
  }
  float r = 1.f;
  if (vhead) r = 1.f / sqrtf(block_sum<CQ>(sq, scratch) / (float)a.dv + a.v_eps);     // (unit-uniform branch)
  if (!dst_out) return;
#pragma unroll
  for (int u = 0; u < CQ_PER; ++u) {
    const int e = threadIdx.x + u * CQ;
    if (e < width) dst_out[e] = (T)(y[u] * r);
  }
}

// grid (T, H), one wave per (row, head)
template <typename T>
__global__ __launch_bounds__(64) void memory_norm_gate_kernel(const float* __restrict__ y, const float* __restrict__ m,
                                                              const T* __restrict__ gate, long long ldg,
                                                              const float* __restrict__ w, float eps, T* __restrict__ out,
                                                              int H, int P) {
  const int row = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* yr = y + ((long long)row * H + h) * (P + 1);
  const float den = fmaxf(fabsf(yr[P]), expf(-m[(long long)row * H + h])) + 1e-6f;
  float sq = 0.f;
  for (int c = lane; c < P; c += 64) {
    const float o = yr[c] / den;
    sq += o * o;
  }
  const float r = 1.f / sqrtf(wave_sum(sq) / (float)P + eps);
  const T* gr = gate + (long long)row * ldg + (long long)h * P;
  T* orow = out + ((long long)row * H + h) * P;
  for (int c = lane; c < P; c += 64)
    orow[c] = (T)(yr[c] / den * r * w[(long long)h * P + c] * sigmoidf((float)gr[c]));
}

__global__ __launch_bounds__(NT) void logit_softcap_kernel(float* __restrict__ x, long long n, float cap) {
  for (long long i = (long long)blockIdx.x * NT + threadIdx.x; i < n; i += (long long)gridDim.x * NT)
    x[i] = cap * tanhf(x[i] / cap);
}

// a decode-sized launch of wide rows: more threads per row (fewer passes over the columns)
bool wide_rows(int rows, int d) { return rows <= 256 && d >= 2048; }

}  // namespace

#define DISPATCH_T(f32, ...)      \
  if (f32) {                      \
    using T = float;              \
    __VA_ARGS__                   \
  } else {                        \
    using T = bf16;               \
    __VA_ARGS__                   \
  }

void launch_embed_pair_hash(const PairHashArgs& a, int f32, hipStream_t s) {
  if (a.T <= 0) return;
  if (wide_rows(a.T, a.d)) {
    DISPATCH_T(f32, (embed_pair_hash_kernel<T, 1024><<<a.T, 1024, 0, s>>>(a));)
  } else {
    DISPATCH_T(f32, (embed_pair_hash_kernel<T, NT><<<a.T, NT, 0, s>>>(a));)
  }
}

void launch_token_state_update(const int* ids, int* tok_state, const int* cu_q, const int* save_slot, int runs,
                               hipStream_t s) {
  if (runs <= 0) return;
  token_state_update_kernel<<<(runs + NT - 1) / NT, NT, 0, s>>>(ids, tok_state, cu_q, save_slot, runs);
}

void launch_hyper_mix_norm(const HyperMixArgs& a, int f32, hipStream_t s) {
  const int rows = a.a ? (a.out && a.n > a.T ? a.n : a.T) : (a.out ? a.n : 0);
  if (rows <= 0) return;
  const size_t lds = (size_t)(a.d + a.S * a.S + 2 * a.S) * sizeof(float);
  if (wide_rows(rows, a.d)) {
    DISPATCH_T(f32, (hyper_mix_norm_kernel<T, 1024><<<rows, 1024, lds, s>>>(a));)
  } else {
    DISPATCH_T(f32, (hyper_mix_norm_kernel<T, NT><<<rows, NT, lds, s>>>(a));)
  }
}

void launch_conv_qkv_cache(const ConvQkvArgs& a, int f32, hipStream_t s) {
  if (a.T <= 0) return;
  dim3 grid(a.T, a.H + 2 * a.G);
  DISPATCH_T(f32, conv_qkv_cache_kernel<T><<<grid, CQ, 0, s>>>(a);)
}

void launch_memory_norm_gate(const float* y, const float* m, const void* gate, long long ldg, const float* w, float eps,
                             void* out, int T_, int H, int P, int f32, hipStream_t s) {
  if (T_ <= 0) return;
  dim3 grid(T_, H);
  DISPATCH_T(f32, memory_norm_gate_kernel<T><<<grid, 64, 0, s>>>(y, m, (const T*)gate, ldg, w, eps, (T*)out, H, P);)
}

void launch_logit_softcap(float* x, long long n, float cap, hipStream_t s) {
  if (n <= 0) return;
  const long long blocks = (n + NT - 1) / NT;
  logit_softcap_kernel<<<(unsigned)(blocks < 4096 ? blocks : 4096), NT, 0, s>>>(x, n, cap);
}
