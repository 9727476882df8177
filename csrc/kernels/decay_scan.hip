// Linear recurrence with decaying matrix state, the common core of gated linear attention and state-space layers:
//
//     S_t = diag(a_t) S_(t-1) + b_t k_t v_t^T          S [N x P] fp32 per (sequence, head)
//     o_t = S_t^T (q_scale q_t) (+ skip_h v_t)
//
// mode 0 (channel gate): a_t[n] = sigmoid(dz_t[n] + dbias[n])^(1 / tau) = exp(logsigmoid(.) / tau), b_t = 1
// mode 1 (step size):    b_t = softplus(dz_t + dbias[h]), a_t = exp(-exp(rate[h]) b_t) for every n
// mode 2 (log gates):    i_t = c tanh(. / c), f_t = logsigmoid(c tanh(. / c)) from fp32 pre-activations, a running maximum
//                        m_t = max(f_t + m_(t-1), i_t) (m = 0 at a sequence's start), a_t = exp(f_t + m_(t-1) - m_t),
//                        b_t = exp(i_t - m_t).  One more value column is fed by v = 1: its state is the normaliser n_t and
//                        its output n_t . q_t.  m travels in one more row of the state, the same value in every column, so
//                        that each column's owner reads and writes its own copy (no workgroup reads what another writes);
//                        it is chained token by token by the first wave while a batch is staged.
//
// The state walks token by token in fp32, in the same order however a prompt is cut into steps, so a position's
// output does not depend on the cut.  A run of rows (one sequence's tokens of this step) starts from its state slot
// (or zero at position 0) and ends in it.
//
// Work split: grid (P / 64 column tiles, heads, runs), 256 threads.  Wave w owns 16 value columns; inside a wave the
// lanes are 16 columns x 4 slices of the key channels, so a lane keeps N / 4 state entries of one column in
// registers and a token's output is a 4-lane sum (two cross-lane adds).  The per-token vectors that all columns
// share (q, k, the decays) are staged through LDS for CH tokens at a time by the whole workgroup, with the
// transcendental part of the decay evaluated once per (token, channel) there; the next batch's global loads are in
// flight while the current batch is computed (two LDS buffers, one barrier per batch).
#include "common.h"
#include "hybrid_launchers.h"

namespace {

constexpr int NT = 256;
// A wave's lanes are PCOLS value columns x SLICES slices of the key channels (PCOLS * SLICES = 64): 16 x 4, or 8 x 8
// when heads x columns x sequences would leave SIMDs with a single wave (more, shorter waves hide each other's latency).

SYM_DEV float softplus_exact(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// NPL: state entries per lane (>= ceil(N / SLICES)); CH: tokens staged per batch
template <typename T, int MODE, int NPL, int CH, int SLICES>
__global__ __launch_bounds__(NT) void decay_scan_kernel(DecayScanArgs a) {
  extern __shared__ float lds[];
  constexpr int PCOLS = 64 / SLICES;
  constexpr int NPAD = NPL * SLICES;
  constexpr int LROW = SLICES * (NPL + 4);                  // a token's LDS row: the four slices 16 bytes apart in bank
                                                            // space, so the lanes' four addresses of a read do not collide
  constexpr int EPT = CH * NPAD / NT;                       // staged (token, channel) entries per thread
  constexpr int ASZ = MODE == 0 ? CH * LROW : (MODE == 1 ? 2 : 3) * CH;   // decays per channel, or (decay, step(, max)) per token
  constexpr int BUF = 2 * CH * LROW + ASZ;
  static_assert(CH * NPAD % NT == 0, "staging split");
  const int N = a.N, P = a.P;
  const int h = blockIdx.y, run = blockIdx.z;
  const int s0 = a.cu_q ? a.cu_q[run] : run, s1 = a.cu_q ? a.cu_q[run + 1] : run + 1;
  if (s1 <= s0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pc = lane & (PCOLS - 1), ns = lane / PCOLS;
  const int p = blockIdx.x * (PCOLS * (NT / 64)) + wave * PCOLS + pc;
  const bool pin = p < P;
  const int n0 = ns * NPL;
  const int l0 = ns * (NPL + 4);
  const int grp = h / a.hpg;
  const int pr = a.prev_row[s0];
  const int sv = a.save_slot[s1 - 1];
  float S[NPL];
  if (pr <= -2 && pin) {
    const float* st = a.state + (long long)(-(pr + 2)) * a.state_stride + (long long)h * (N + (MODE == 2)) * P + p;
#pragma unroll
    for (int i = 0; i < NPL; ++i) S[i] = n0 + i < N ? st[(long long)(n0 + i) * P] : 0.f;
  } else {
#pragma unroll
    for (int i = 0; i < NPL; ++i) S[i] = 0.f;
  }
  // mode 2: the running maximum, chained by the first wave (every lane of it holds the same value); a workgroup reads
  // the copy in its first column (every workgroup has one)
  float mrun = 0.f;
  if (MODE == 2 && pr <= -2)
    mrun = a.state[(long long)(-(pr + 2)) * a.state_stride + ((long long)h * (N + 1) + N) * P + blockIdx.x * (PCOLS * (NT / 64))];
  const T* q = reinterpret_cast<const T*>(a.q) + (long long)grp * N;
  const T* k = reinterpret_cast<const T*>(a.k) + (long long)grp * N;
  const T* v = reinterpret_cast<const T*>(a.v) + (long long)h * a.vcols + p;
  const bool vin = p < a.vcols;        // (mode 2: column vcols is fed by 1)
  const T* dz = reinterpret_cast<const T*>(a.dz);
  const float skip = a.skip ? a.skip[h] : 0.f;
  const float inv_tau = MODE == 0 ? 1.f / a.tau : 0.f;
  const float rate = MODE == 1 ? expf(a.rate[h]) : 0.f;
  // a batch's inputs travel global -> registers (issued before the previous batch is computed) -> LDS (with the
  // transcendental part of the decay evaluated once per (token, channel)); two LDS buffers, one barrier per batch
  float rq[EPT], rk[EPT], rz[EPT], vn[CH], rdt = 0.f, rdf = 0.f, mlast = 0.f;
  auto fetch = [&](int t0) {
    const int nt = min(CH, s1 - t0);
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
      const int i = threadIdx.x + NT * u;
      const int tt = i / NPAD, n = i - tt * NPAD;
      const bool in = tt < nt && n < N;
      const long long r = t0 + tt;
      rq[u] = in ? (float)q[r * a.ldq + n] : 0.f;
      rk[u] = in ? (float)k[r * a.ldk + n] : 0.f;
      if (MODE == 0) rz[u] = in ? (float)dz[r * a.ldd + (long long)h * N + n] + a.dbias[(long long)h * N + n] : 0.f;
    }
    if (MODE == 1 && threadIdx.x < CH)
      rdt = (int)threadIdx.x < nt ? (float)dz[(long long)(t0 + threadIdx.x) * a.ldd + h] + a.dbias[h] : 0.f;
    if (MODE == 2 && threadIdx.x < CH) {
      const float* gz = reinterpret_cast<const float*>(a.dz) + (long long)(t0 + threadIdx.x) * a.ldd;
      rdt = (int)threadIdx.x < nt ? gz[h] + a.dbias[h] : 0.f;
      rdf = (int)threadIdx.x < nt ? gz[a.H + h] + a.dbias[a.H + h] : 0.f;
    }
#pragma unroll
    for (int tt = 0; tt < CH; ++tt)
      vn[tt] = (tt < nt && pin) ? (MODE == 2 && !vin ? 1.f : (float)v[(long long)(t0 + tt) * a.ldv]) : 0.f;
  };
  auto commit = [&](float* buf, int nt) {
    float* qS = buf;
    float* kS = buf + CH * LROW;
    float* aS = kS + CH * LROW;
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
      const int i = threadIdx.x + NT * u;
      const int tt = i / NPAD, n = i - tt * NPAD;
      const int o = tt * LROW + (n / NPL) * (NPL + 4) + n % NPL;
      qS[o] = rq[u] * a.q_scale;
      kS[o] = rk[u];
      if (MODE == 0) aS[o] = expf(-softplus_exact(-rz[u]) * inv_tau);   // logsigmoid(z) = -softplus(-z); padding: k = q = 0
    }
    if (MODE == 1 && threadIdx.x < CH) {
      const float b = softplus_exact(rdt);
      aS[threadIdx.x] = expf(-rate * b);
      aS[CH + threadIdx.x] = b;
    }
    if (MODE == 2 && threadIdx.x < 64) {      // the first wave: lane tt has token tt's pre-activations
      const float cap = a.tau;
      const float li = cap * tanhf(rdt / cap);
      const float lf = -softplus_exact(-(cap * tanhf(rdf / cap)));
      // the chain m_t = max(f_t + m_(t-1), i_t) is an add and a max per token; lane tt keeps its token's pair
      // (m_(t-1), m_t) and evaluates the two exponentials afterwards, all lanes at once
      float mp = 0.f, mm = 0.f;
#pragma unroll
      for (int tt = 0; tt < CH; ++tt) {
        const float it = __shfl(li, tt, 64), ft = __shfl(lf, tt, 64);
        const float mn = fmaxf(ft + mrun, it);
        if ((int)threadIdx.x == tt) mp = mrun, mm = mn;
        if (tt < nt) mrun = mn;
      }
      if (threadIdx.x < CH) {
        aS[threadIdx.x] = expf(lf + mp - mm);
        aS[CH + threadIdx.x] = expf(li - mm);
        aS[2 * CH + threadIdx.x] = mm;
      }
    }
  };
  fetch(s0);
  int flip = 0;
  for (int t0 = s0; t0 < s1; t0 += CH, flip ^= 1) {
    const int nt = min(CH, s1 - t0);
    float* buf = lds + flip * BUF;
    commit(buf, nt);
    float vr[CH];
#pragma unroll
    for (int tt = 0; tt < CH; ++tt) vr[tt] = vn[tt];
    __syncthreads();   // this batch's vectors are in LDS; every thread has finished the batch before the last (same buffer)
    if (t0 + CH < s1) fetch(t0 + CH);
    const float* qS = buf;
    const float* kS = buf + CH * LROW;
    const float* aS = kS + CH * LROW;
    float po[CH];
#pragma unroll
    for (int tt = 0; tt < CH; ++tt) {
      po[tt] = 0.f;
      if (tt < nt) {
        const float* qr = qS + tt * LROW + l0;
        const float* kr = kS + tt * LROW + l0;
        float u = vr[tt], o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
        // 16-byte LDS reads (rows, slices and buffers all start at multiples of four floats)
        const float4* q4 = reinterpret_cast<const float4*>(qr);
        const float4* k4 = reinterpret_cast<const float4*>(kr);
        if (MODE >= 1) {
          u *= aS[CH + tt];
          const float at = aS[tt];
#pragma unroll
          for (int i = 0; i < NPL / 4; ++i) {
            const float4 kv = k4[i], qv = q4[i];
            S[4 * i + 0] = at * S[4 * i + 0] + kv.x * u;
            S[4 * i + 1] = at * S[4 * i + 1] + kv.y * u;
            S[4 * i + 2] = at * S[4 * i + 2] + kv.z * u;
            S[4 * i + 3] = at * S[4 * i + 3] + kv.w * u;
            o0 += S[4 * i + 0] * qv.x, o1 += S[4 * i + 1] * qv.y, o2 += S[4 * i + 2] * qv.z, o3 += S[4 * i + 3] * qv.w;
          }
        } else {
          const float4* a4 = reinterpret_cast<const float4*>(aS + tt * LROW + l0);
#pragma unroll
          for (int i = 0; i < NPL / 4; ++i) {
            const float4 kv = k4[i], qv = q4[i], av = a4[i];
            S[4 * i + 0] = av.x * S[4 * i + 0] + kv.x * u;
            S[4 * i + 1] = av.y * S[4 * i + 1] + kv.y * u;
            S[4 * i + 2] = av.z * S[4 * i + 2] + kv.z * u;
            S[4 * i + 3] = av.w * S[4 * i + 3] + kv.w * u;
            o0 += S[4 * i + 0] * qv.x, o1 += S[4 * i + 1] * qv.y, o2 += S[4 * i + 2] * qv.z, o3 += S[4 * i + 3] * qv.w;
          }
        }
        po[tt] = (o0 + o1) + (o2 + o3);
      }
    }
    // the slices' partial sums of the whole batch meet in one go: the tokens' cross-lane adds are independent of one
    // another, so their latencies overlap (done per token they sat on the serial path)
#pragma unroll
    for (int sh = PCOLS; sh < 64; sh <<= 1)
#pragma unroll
      for (int tt = 0; tt < CH; ++tt) po[tt] += __shfl_xor(po[tt], sh, 64);
    if (ns == 0 && pin)
#pragma unroll
      for (int tt = 0; tt < CH; ++tt)
        if (tt < nt) a.out[((long long)(t0 + tt) * a.H + h) * P + p] = po[tt] + skip * vr[tt];
    if (MODE == 2) {
      mlast = aS[2 * CH + nt - 1];
      if (blockIdx.x == 0 && (int)threadIdx.x < nt) a.mout[(long long)(t0 + threadIdx.x) * a.H + h] = aS[2 * CH + threadIdx.x];
    }
  }
  if (sv >= 0 && pin) {
    float* st = a.state + (long long)sv * a.state_stride + (long long)h * (N + (MODE == 2)) * P + p;
#pragma unroll
    for (int i = 0; i < NPL; ++i)
      if (n0 + i < N) st[(long long)(n0 + i) * P] = S[i];
    if (MODE == 2 && ns == 0) st[(long long)N * P] = mlast;
  }
}

template <typename T, int MODE, int NPL, int CH, int SLICES>
void launch_one(const DecayScanArgs& a, hipStream_t s) {
  const int cols = (64 / SLICES) * (NT / 64);
  dim3 grid((a.P + cols - 1) / cols, a.H, a.runs);
  const int lrow = SLICES * (NPL + 4);
  const size_t lds = (size_t)2 * (2 * CH * lrow + (MODE == 0 ? CH * lrow : (MODE == 1 ? 2 : 3) * CH)) * sizeof(float);
  decay_scan_kernel<T, MODE, NPL, CH, SLICES><<<grid, NT, lds, s>>>(a);
}

template <typename T, int MODE>
void launch_mode(const DecayScanArgs& a, hipStream_t s) {
  // waves with 16 columns each; under two per SIMD (1024 SIMDs) and enough key channels: 8 columns x 8 slices
  const long long waves16 = (long long)a.runs * a.H * ((a.P + 15) / 16);
  if (waves16 < 2048 && a.N >= 64 && a.T > a.runs) {
    const int need = (a.N + 7) / 8;
    if (need <= 8) launch_one<T, MODE, 8, 16, 8>(a, s);
    else if (need <= 16) launch_one<T, MODE, 16, 16, 8>(a, s);
    else launch_one<T, MODE, 32, 8, 8>(a, s);      // N <= 256 (checked by the op layer)
    return;
  }
  const int need = (a.N + 3) / 4;
  if (need <= 4) launch_one<T, MODE, 4, 16, 4>(a, s);
  else if (need <= 8) launch_one<T, MODE, 8, 16, 4>(a, s);
  else if (need <= 16) launch_one<T, MODE, 16, 16, 4>(a, s);
  else if (need <= 32) launch_one<T, MODE, 32, 16, 4>(a, s);
  else launch_one<T, MODE, 64, 8, 4>(a, s);   // N <= 256; half the batch keeps LDS under 64 KB
}

}  // namespace

void launch_decay_scan(const DecayScanArgs& a, int f32, hipStream_t s) {
  if (a.runs <= 0 || a.T <= 0) return;
  if (f32) {
    if (a.mode == 0) launch_mode<float, 0>(a, s);
    else if (a.mode == 1) launch_mode<float, 1>(a, s);
    else launch_mode<float, 2>(a, s);
  } else {
    if (a.mode == 0) launch_mode<bf16, 0>(a, s);
    else if (a.mode == 1) launch_mode<bf16, 1>(a, s);
    else launch_mode<bf16, 2>(a, s);
  }
}
