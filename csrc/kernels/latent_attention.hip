// Attention over a cached low-rank latent (one shared "key/value head" for all query heads).
//
// The cache holds, per token, the normalised latent c [kv_rank] followed by one rotated key part k_r [rot]
// shared by every head.  With the per-head up-projections folded into the query and the output,
//
//     score(t, j, h) = (W_uk[h]^T q_nope[t, h]) . c[j] + q_rot[t, h] . k_r[j]          (times the scale)
//     out(t, h)      = W_uv[h] . sum_j softmax_j(score)(t, j, h) c[j]
//
// so the attention kernel is multi-query attention whose key row is the whole cache row [kv_rank + rot] and whose
// value row is its first kv_rank entries: every cache row is read once for all heads, and nothing but the cache
// row is ever materialised per token.
//
//   latent_prep   per token: RMS-norm the query latent; RMS-norm the kv latent and rotate the shared key part into
//                 the token's cache row (statistics and angles in fp32)
//   rope_pairs    rotary of a strided [T][H][rot] slice: interleaved pairs (dimension 2i with 2i + 1) or the half
//                 layout (dimension i with i + dims / 2, dimensions past dims passing)
//   latent_attn   causal softmax attention over the paged latent cache, optionally limited to a sliding window of
//                 the newest keys; scores, weights and accumulators fp32.
//                 Two implementations: the MFMA kernel (bf16, tiled shapes) and a one-wave-per-(row, head) kernel
//                 for every other shape and for the 32-bit model.
//
// MFMA kernel (v_mfma_f32_16x16x32_bf16, 4 waves, 64 query vectors per workgroup: 64 rows of one head for prompt
// tiles, one row's heads for decode steps with split-KV partitions).  Per 32-key tile the workgroup stages the cache
// rows ONCE for all its query vectors -- key-major for the scores, and the latent part a second time transposed
// (dim-major) for the weighted sum: the score product contracts over the row's dims and the value product over the
// keys, an MFMA operand wants its contraction index contiguous per lane, and keys and values are the same bytes here,
// so one transpose per tile is inherent; it happens on the way into LDS, off the HBM / L2 path.  Both products run
// swapped (S^T = K Q^T, O^T = V^T P^T): the query fragments stay in registers for the whole key loop, the packed
// bf16 weights of a lane ARE its B operand of the second product (the 32 keys of a tile are consumed in the order
// the accumulator layout hands them out, and the V^T fragment reads follow the same order), and the softmax
// statistics of a query vector live in the 4 lanes that share its accumulator column.
#include "common.h"
#include "latent_launchers.h"

namespace {

constexpr int NT = 256;

// entries (first, second) of rotary pair p in a vector of `rot` entries.  Interleaved (half_dims == 0): (2p, 2p + 1).
// Half layout: pair p < half_dims / 2 is (p, p + half_dims / 2); the pairs after those are the passing entries
// half_dims .., two by two (their table entries are the identity).
SYM_DEV void pair_entries(int p, int half_dims, int& e0, int& e1) {
  if (half_dims == 0) {
    e0 = 2 * p, e1 = 2 * p + 1;
  } else if (p < half_dims / 2) {
    e0 = p, e1 = p + half_dims / 2;
  } else {
    e0 = half_dims + 2 * (p - half_dims / 2), e1 = e0 + 1;
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void latent_prep_kernel(LatentPrepArgs a) {
  __shared__ float scratch[NT / 64];
  const int row = blockIdx.x;
  const T* z = (const T*)a.z + (long long)row * a.nz;
  float ss = 0.f;
  for (int c = threadIdx.x; c < a.q_rank; c += NT) {
    const float v = (float)z[c];
    ss += v * v;
  }
  const float rq = 1.f / sqrtf(block_sum<NT>(ss, scratch) / (float)a.q_rank + a.eps);
  T* cq = (T*)a.cq + (long long)row * a.q_rank;
  const T* wq = (const T*)a.wq;
  for (int c = threadIdx.x; c < a.q_rank; c += NT) cq[c] = (T)((float)z[c] * rq * (float)wq[c]);
  if (a.kv_rank == 0) return;
  const int slot = a.slots[row];
  const T* zk = z + a.q_rank;
  ss = 0.f;
  for (int c = threadIdx.x; c < a.kv_rank; c += NT) {
    const float v = (float)zk[c];
    ss += v * v;
  }
  const float rk = 1.f / sqrtf(block_sum<NT>(ss, scratch) / (float)a.kv_rank + a.eps);
  if (slot < 0) return;
  T* out = (T*)a.cache + (long long)slot * (a.kv_rank + a.rot);
  const T* wkv = (const T*)a.wkv;
  for (int c = threadIdx.x; c < a.kv_rank; c += NT) out[c] = (T)((float)zk[c] * rk * (float)wkv[c]);
  const float* cs = a.rope + (long long)a.positions[row] * a.rot;
  for (int i = threadIdx.x; i < a.rot / 2; i += NT) {
    int e0, e1;
    pair_entries(i, a.half_dims, e0, e1);
    const float u = (float)zk[a.kv_rank + e0], v = (float)zk[a.kv_rank + e1];
    const float co = cs[2 * i], si = cs[2 * i + 1];
    out[a.kv_rank + e0] = (T)(u * co - v * si);
    out[a.kv_rank + e1] = (T)(v * co + u * si);
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void rope_pairs_kernel(const T* __restrict__ src, long long s_t, long long s_h,
                                                        T* __restrict__ dst, long long d_t, long long d_h,
                                                        const int* __restrict__ positions,
                                                        const float* __restrict__ rope, int H, int rot,
                                                        int half_dims) {
  const int row = blockIdx.x;
  const float* cs = rope + (long long)positions[row] * rot;
  const int half = rot / 2;
  for (int i = threadIdx.x; i < H * half; i += NT) {
    const int h = i / half, p = i - h * half;
    int e0, e1;
    pair_entries(p, half_dims, e0, e1);
    const T* s = src + row * s_t + h * s_h;
    T* o = dst + row * d_t + h * d_h;
    const float u = (float)s[e0], v = (float)s[e1];
    const float co = cs[2 * p], si = cs[2 * p + 1];
    o[e0] = (T)(u * co - v * si);
    o[e1] = (T)(v * co + u * si);
  }
}

// fp32 dot of a query held in LDS with one cache row (16-byte loads when the row length allows)
SYM_DEV float dot_row(const float* q, const bf16* r, int n) {
  float s = 0.f;
  if ((n & 7) == 0) {
    for (int c = 0; c < n; c += 8) {
      float f[8];
      load8(r + c, f);
#pragma unroll
      for (int i = 0; i < 8; ++i) s += q[c + i] * f[i];
    }
  } else {
    for (int c = 0; c < n; ++c) s += q[c] * (float)r[c];
  }
  return s;
}

SYM_DEV float dot_row(const float* q, const float* r, int n) {
  float s = 0.f;
  if ((n & 3) == 0) {
    for (int c = 0; c < n; c += 4) {
      const float4 f = *reinterpret_cast<const float4*>(r + c);
      s += q[c] * f.x + q[c + 1] * f.y + q[c + 2] * f.z + q[c + 3] * f.w;
    }
  } else {
    for (int c = 0; c < n; ++c) s += q[c] * r[c];
  }
  return s;
}


// One wave per (query row, head, key partition).  Each lane scores one key of a 64-key tile (the query in LDS, the
// cache row streamed), the tile's softmax statistics are wave reductions, and the weighted sum of the latents
// keeps kv_rank / 64 accumulators per lane (coalesced row reads, the weight broadcast by a lane read).
// parts == 1: the normalised output goes to `out`; otherwise unnormalised partials + (max, sum) go to part_o /
// part_ml and latent_attn_merge_kernel combines them.
template <typename T, int MAXR>
__global__ __launch_bounds__(64) void latent_attn_wave_kernel(LatentAttnArgs a) {
  extern __shared__ float qs[];
  const int row = blockIdx.x, h = blockIdx.y, part = blockIdx.z;
  const int lane = threadIdx.x;
  const int nkeys = a.positions[row] + 1;
  const int lo = a.window > 0 ? max(0, nkeys - a.window) : 0;     // the first key the row sees
  const int k0 = a.parts > 1 ? lo + part * a.part_tokens : lo;
  const int k1 = a.parts > 1 ? min(nkeys, k0 + a.part_tokens) : nkeys;
  const T* q = (const T*)a.q + ((long long)row * a.H + h) * a.Dk;
  for (int c = lane; c < a.Dk; c += 64) qs[c] = (float)q[c];
  __syncthreads();
  const int* bt = a.block_tables + (long long)a.row_seq[row] * a.max_blocks;
  const T* cache = (const T*)a.cache;
  float m = -INFINITY, l = 0.f;
  float o[MAXR];
#pragma unroll
  for (int i = 0; i < MAXR; ++i) o[i] = 0.f;
  for (int base = k0; base < k1; base += 64) {
    const int key = base + lane;
    const bool valid = key < k1;
    int crow = 0;
    float s = -INFINITY;
    if (valid) {
      crow = bt[key / a.BS] * a.BS + key % a.BS;
      s = dot_row(qs, cache + (long long)crow * a.Dk, a.Dk) * a.scale;
    }
    const float m_new = fmaxf(m, wave_max(s));   // finite: the tile holds at least one key the row sees
    const float alpha = expf(m - m_new);
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int i = 0; i < MAXR; ++i) o[i] *= alpha;
    const int n = min(64, k1 - base);
    for (int j = 0; j < n; ++j) {
      const float pj = __shfl(p, j, 64);
      const T* r = cache + (long long)__shfl(crow, j, 64) * a.Dk;
#pragma unroll
      for (int i = 0; i < MAXR; ++i) {
        const int c = lane + 64 * i;
        if (c < a.kv_rank) o[i] += pj * (float)r[c];
      }
    }
    m = m_new;
  }
  if (a.parts == 1) {
    T* out = (T*)a.out + ((long long)row * a.H + h) * a.kv_rank;
    const float inv = 1.f / l;
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
      const int c = lane + 64 * i;
      if (c < a.kv_rank) out[c] = (T)(o[i] * inv);
    }
  } else {
    const long long pi = ((long long)row * a.H + h) * a.parts + part;
    float* po = a.part_o + pi * a.kv_rank;
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
      const int c = lane + 64 * i;
      if (c < a.kv_rank) po[c] = o[i];
    }
    if (lane == 0) {
      a.part_ml[2 * pi] = m;  // -inf, 0 for a partition past the row's keys
      a.part_ml[2 * pi + 1] = l;
    }
  }
}

// Combine the split-KV partials of one (row, head): four waves.  The per-partition weights exp(m_p - m) are computed
// once (threads over partitions, kept in LDS); then wave w sums partitions w, w + 4, .. with every lane owning up to
// 8 latent dims in registers (a partition's loads all in flight), and the four partial sums meet in LDS.
template <typename T>
__global__ __launch_bounds__(256) void latent_attn_merge_kernel(LatentAttnArgs a) {
  __shared__ float wp[1024];
  __shared__ float red[4][512];
  __shared__ float stat[8];
  const int row = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long long p0 = ((long long)row * a.H + h) * a.parts;
  // partitions that hold keys: the row's range starts at its window's first key (at 0 without a window)
  const int seen = a.window > 0 ? min(a.positions[row] + 1, a.window) : a.positions[row] + 1;
  const int np = min(a.parts, (seen + a.part_tokens - 1) / a.part_tokens);
  float m = -INFINITY;
  for (int p = tid; p < np; p += 256) m = fmaxf(m, a.part_ml[2 * (p0 + p)]);
  m = wave_max(m);
  if (lane == 0) stat[wave] = m;
  __syncthreads();
  m = fmaxf(fmaxf(stat[0], stat[1]), fmaxf(stat[2], stat[3]));
  float l = 0.f;
  for (int p = tid; p < np; p += 256) {
    const float w = __expf(a.part_ml[2 * (p0 + p)] - m);
    wp[p] = w;
    l += a.part_ml[2 * (p0 + p) + 1] * w;
  }
  l = wave_sum(l);
  if (lane == 0) stat[4 + wave] = l;
  __syncthreads();
  const float inv = 1.f / (stat[4] + stat[5] + stat[6] + stat[7]);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int p = wave; p < np; p += 4) {
    const float* po = a.part_o + (p0 + p) * a.kv_rank;
    const float w = wp[p];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = lane + 64 * i;
      if (c < a.kv_rank) acc[i] += po[c] * w;
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) red[wave][lane + 64 * i] = acc[i];
  __syncthreads();
  T* out = (T*)a.out + ((long long)row * a.H + h) * a.kv_rank;
  for (int c = tid; c < a.kv_rank; c += 256) out[c] = (T)((red[0][c] + red[1][c] + red[2][c] + red[3][c]) * inv);
}

constexpr int KT = 32;        // keys per staged tile
constexpr int LDV = KT + 4;   // row pitch (elements) of the transposed latent tile

// NW waves per workgroup in QG = NW / DSPLIT groups of 16 query vectors; the DSPLIT waves of a group share the
// query vectors (each computes the scores and the softmax, redundantly and identically) and split the latent dims
// of the weighted sum, which divides the accumulator registers -- the bulk of a wave's registers at kv_rank 512 --
// so that two waves fit a SIMD and one's LDS latency hides behind the other's MFMAs.
// Prompt form (DECODE = false): a tile of 16 * QG rows of one head.  Decode form: one row, 16 * QG of its heads, one
// key partition per workgroup (few heads: fewer groups, more dim splitting, so no wave idles).
// The next tile's cache rows are fetched into registers while the current tile is multiplied (the global latency
// hides behind the MFMAs); they go to LDS between two barriers at the top of the next iteration.
// EXACT: Dk == 32 * NKM and kv_rank == 16 * RTM, so the unrolled MFMA loops carry no bounds tests (a test on a
// runtime count makes the compiler compute the MFMA anyway and select the accumulator afterwards: four selects,
// through the accumulator registers, per MFMA).  The inexact instantiation serves every smaller tiled shape.
template <int NKM, int RTM, bool DECODE, int NW, int DSPLIT, bool EXACT>
__global__ __launch_bounds__(64 * NW) void latent_attn_mfma_kernel(LatentAttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int NTH = 64 * NW;
  constexpr int QG = NW / DSPLIT;                       // query-vector groups
  constexpr int RTD = RTM / DSPLIT;                     // 16-dim output tiles per wave (upper bound)
  constexpr int CSTEP = NTH / 32;                       // 16-byte chunks of a row taken per pass of the workgroup
  constexpr int CHM = (NKM * 4 + CSTEP - 1) / CSTEP;    // passes (chunks per thread)
  // up to 9 passes stay in registers across the multiply (prefetch); workgroups of fewer waves have more passes per
  // thread than registers to spare and stage in batches instead (no prefetch: they run one or two tiles)
  static_assert(CHM <= 9, "a thread keeps one tile's share of cache rows in registers");
  constexpr int NB = CHM;
  const int Dk = a.Dk, r = a.kv_rank, H = a.H;
  const int nk = EXACT ? NKM : Dk >> 5, rtd = EXACT ? RTD : (r >> 4) / DSPLIT, nchunk = EXACT ? NKM * 4 : Dk >> 3;
  const int ldk = Dk + 8;
  // two LDS stages, each [KT][ldk] key-major cache rows + [r][LDV] latent part dim-major; tile t lives in stage
  // t & 1, so tile t + 1 is written while tile t is still being multiplied
  const int stage_elems = KT * ldk + r * LDV;
  bf16* const stage0 = reinterpret_cast<bf16*>(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int qg = wave % QG, dh = wave / QG;             // this wave's query group and latent-dim share
  int seq, qrow, head, limit, k_lo, k_hi, wave_hi, wave_lo, part = 0;  // wave_lo: keys every query vector of the wave sees
  bool valid, wave_active;
  if constexpr (DECODE) {
    qrow = blockIdx.x;
    seq = a.row_seq[qrow];
    head = blockIdx.y * 16 * QG + qg * 16 + n;
    valid = head < H;
    wave_active = blockIdx.y * 16 * QG + qg * 16 < H;
    limit = a.positions[qrow];
    part = blockIdx.z;
    const int first = a.window > 0 ? max(0, limit + 1 - a.window) : 0;
    k_lo = a.parts > 1 ? first + part * a.part_tokens : first;
    k_hi = a.parts > 1 ? min(limit + 1, k_lo + a.part_tokens) : limit + 1;
    if (k_lo >= k_hi) return;  // a partition past this row's keys: the merge never reads it
    wave_hi = k_hi;
    wave_lo = limit + 1;
  } else {
    seq = a.tiles[2 * blockIdx.x];
    const int off = a.tiles[2 * blockIdx.x + 1];
    const int q0 = a.cu_q[seq], qlen = a.cu_q[seq + 1] - q0;
    if (off >= qlen) return;  // padding tile
    const int rin = off + qg * 16 + n;
    valid = rin < qlen;
    wave_active = off + qg * 16 < qlen;
    qrow = q0 + min(rin, qlen - 1);
    head = blockIdx.y;
    limit = a.positions[qrow];
    k_lo = a.window > 0 ? max(0, a.positions[q0 + off] + 1 - a.window) : 0;   // the tile's first row looks back farthest
    k_hi = a.positions[q0 + min(off + 16 * QG - 1, qlen - 1)] + 1;       // a run's rows are consecutive positions
    wave_hi = a.positions[q0 + min(off + qg * 16 + 15, qlen - 1)] + 1;
    wave_lo = a.positions[q0 + min(off + qg * 16, qlen - 1)] + 1;
  }
  const bf16* qp = (const bf16*)a.q + ((long long)qrow * H + min(head, H - 1)) * Dk;
  bf16x8 qf[NKM];
#pragma unroll
  for (int s = 0; s < NKM; ++s)
    if (EXACT || s < nk) qf[s] = *reinterpret_cast<const bf16x8*>(qp + s * 32 + g * 8);
  f32x4 o[RTD];  // output tile dt of this wave covers dims (dh * rtd + dt) * 16 ..
#pragma unroll
  for (int i = 0; i < RTD; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int* bt = a.block_tables + (long long)seq * a.max_blocks;
  const bf16* cache = (const bf16*)a.cache;
  const int key_in = tid & 31, c0 = tid >> 5;
  uint4 pre[NB];
  auto fetch = [&](int k0, int i0) {
    const int key = min(k0 + key_in, k_hi - 1);
    const int blk = a.bs_shift >= 0 ? key >> a.bs_shift : key / a.BS;  // (no integer divide for power-of-two blocks)
    const bf16* src = cache + ((long long)bt[blk] * a.BS + (key - blk * a.BS)) * Dk;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int c = c0 + (i0 + i) * CSTEP;
      if (c < nchunk) pre[i] = *reinterpret_cast<const uint4*>(src + c * 8);
    }
  };
  auto stash = [&](int i0, bf16* Ks) {
    bf16* Vt = Ks + KT * ldk;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int c = c0 + (i0 + i) * CSTEP;
      if (c < nchunk) {
        Pack8 pk;
        pk.u = pre[i];
        *reinterpret_cast<uint4*>(Ks + key_in * ldk + c * 8) = pk.u;
        if (c * 8 < r) {
#pragma unroll
          for (int j = 0; j < 8; ++j) Vt[(c * 8 + j) * LDV + key_in] = pk.h[j];
        }
      }
    }
  };
  // Per tile: barrier A (everyone is done with the previous tile's value product and score exchange, so the other
  // stage and the exchange area may be overwritten; the stage written during the previous tile is visible) and, where
  // wave pairs exchange scores, barrier B (this tile's exchanged scores are visible).  The global fetch of tile t + 2 is issued right after tile t + 1 went to LDS and has a whole
  // tile of work to land.
  fetch(k_lo, 0);
  stash(0, stage0);
  if (k_lo + KT < k_hi) fetch(k_lo + KT, 0);
  int cur = 0;
  for (int k0 = k_lo; k0 < k_hi; k0 += KT, cur ^= 1) {
    const bf16* Ks = stage0 + cur * stage_elems;
    const bf16* Vt = Ks + KT * ldk;
    __syncthreads();  // A
    if (k0 + KT < k_hi) {
      stash(0, stage0 + (cur ^ 1) * stage_elems);
      if (k0 + 2 * KT < k_hi) fetch(k0 + 2 * KT, 0);
    }
    // S^T: rows = keys (sub * 16 + g * 4 + i), column = this lane's query vector n
    // (the same for the waves that share a query group; with a window, a tile wholly before the first key of the wave's
    // first row is seen by none of its rows)
    const bool active = wave_active && k0 < wave_hi && (a.window <= 0 || k0 + KT > wave_lo - a.window);
    f32x4 st[2];
    if constexpr (DSPLIT == 2) {
      // the two waves of a query group each score one 16-key subtile (four accumulator chains over the k steps) and
      // swap the results through LDS: half the score MFMAs and key-tile reads of computing both subtiles twice
      f32x4* xch = reinterpret_cast<f32x4*>(stage0 + 2 * stage_elems);  // [QG][2][64]
      f32x4 mine = {0.f, 0.f, 0.f, 0.f};
      if (active) {
        f32x4 acc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        const bf16* kr = Ks + (dh * 16 + n) * ldk + g * 8;
#pragma unroll
        for (int s = 0; s < NKM; ++s)
          if (EXACT || s < nk) acc[s & 3] = mfma16(*reinterpret_cast<const bf16x8*>(kr + s * 32), qf[s], acc[s & 3]);
        mine = (acc[0] + acc[1]) + (acc[2] + acc[3]);
        xch[(qg * 2 + dh) * 64 + lane] = mine;
      }
      __syncthreads();  // B
      if (!active) continue;
      st[0] = mine;                                         // (own subtile first; put in key order below)
      st[1] = xch[(qg * 2 + 1 - dh) * 64 + lane];
    } else {
      if (!active) continue;  // (no exchange: barrier A alone orders the stages)
      // (four independent accumulator chains: both 16-key subtiles, even and odd k steps)
      f32x4 acc[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
      const bf16* kr = Ks + n * ldk + g * 8;
#pragma unroll
      for (int s = 0; s < NKM; ++s)
        if (EXACT || s < nk) {
          acc[s & 1] = mfma16(*reinterpret_cast<const bf16x8*>(kr + s * 32), qf[s], acc[s & 1]);
          acc[2 + (s & 1)] = mfma16(*reinterpret_cast<const bf16x8*>(kr + 16 * ldk + s * 32), qf[s], acc[2 + (s & 1)]);
        }
      st[0] = acc[0] + acc[1];
      st[1] = acc[2] + acc[3];
    }
    if constexpr (DSPLIT == 2) {
      if (dh) {  // st[] indexed by a runtime dh above: keep it in registers
        const f32x4 t = st[0];
        st[0] = st[1];
        st[1] = t;
      }
    }
    // scale; mask only where a tile reaches past some query vector's last key (the diagonal tiles, the range's tail)
    // (wave-uniform; with a window also the tiles that start before the first key of the wave's last row)
    const bool edge = k0 + KT > wave_lo || k0 + KT > k_hi || (a.window > 0 && k0 < wave_hi - a.window);
    const int low = a.window > 0 ? limit + 1 - a.window : 0;  // this query vector's first key
    float mx = -INFINITY;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = st[sub][i] * a.scale;
        if (edge) {
          const int key = k0 + sub * 16 + g * 4 + i;
          if (key > limit || key >= k_hi || key < low) v = -INFINITY;
        }
        st[sub][i] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // deferred rescale: the running maximum moves (and the accumulators are rescaled, a pass over every accumulator
    // register) only when some query vector's maximum grew by more than 8; until then weights may reach e^8, which
    // fp32 sums and bf16 products hold as well as values below 1.  The first tile always takes the branch.
    if (__any(mx > m + 8.f)) {
      // (without a window every query vector sees the first key of its range; with one, a vector may have seen nothing
      // yet: its maximum stays -inf and nothing of it is rescaled)
      const float m_new = fmaxf(m, mx);
      const float alpha = m_new == -INFINITY ? 1.f : __expf(m - m_new);
      l *= alpha;
#pragma unroll
      for (int dt = 0; dt < RTD; ++dt)
        if (EXACT || dt < rtd) o[dt] = o[dt] * alpha;
      m = m_new;
    }
    float ps = 0.f;
    Pack8 pb;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = m == -INFINITY ? 0.f : __expf(st[sub][i] - m);
        ps += p;
        pb.h[sub * 4 + i] = (bf16)p;
      }
    ps += __shfl_xor(ps, 16, 64);
    ps += __shfl_xor(ps, 32, 64);
    l += ps;
    // O^T += V^T P^T: k index g * 8 + j of the product is key g * 4 + j (j < 4) / 16 + g * 4 + j - 4 of the tile
    const bf16* vr = Vt + (dh * rtd * 16 + n) * LDV + g * 4;
#pragma unroll
    for (int dt = 0; dt < RTD; ++dt)
      if (EXACT || dt < rtd) {
        Pack8 va;
        const uint2 lo = *reinterpret_cast<const uint2*>(vr + dt * 16 * LDV);
        const uint2 hi = *reinterpret_cast<const uint2*>(vr + dt * 16 * LDV + 16);
        va.u = make_uint4(lo.x, lo.y, hi.x, hi.y);
        o[dt] = mfma16(va.v, pb.v, o[dt]);
      }
  }
  if (!valid) return;
  // o[dt][i]: dim (dh * rtd + dt) * 16 + g * 4 + i of query vector n
  if (a.parts == 1) {
    bf16* out = (bf16*)a.out + ((long long)qrow * H + head) * r + dh * rtd * 16;
    const float inv = 1.f / l;
#pragma unroll
    for (int dt = 0; dt < RTD; ++dt)
      if (EXACT || dt < rtd) {
        bf16x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (bf16)(o[dt][i] * inv);
        *reinterpret_cast<bf16x4*>(out + dt * 16 + g * 4) = v;
      }
  } else {
    const long long pi = ((long long)qrow * H + head) * a.parts + part;
    float* po = a.part_o + pi * r + dh * rtd * 16;
#pragma unroll
    for (int dt = 0; dt < RTD; ++dt)
      if (EXACT || dt < rtd) *reinterpret_cast<f32x4*>(po + dt * 16 + g * 4) = o[dt];
    if (g == 0 && dh == 0) {
      a.part_ml[2 * pi] = m;
      a.part_ml[2 * pi + 1] = l;
    }
  }
}

template <int NKM, int RTM, bool DECODE, int NW, int DSPLIT, bool EXACT>
void mfma_launch_one(const LatentAttnArgs& a, dim3 grid, hipStream_t s) {
  const size_t lds = 2 * ((size_t)KT * (a.Dk + 8) + (size_t)a.kv_rank * LDV) * sizeof(bf16) +  // two stages
                     (DSPLIT == 2 ? (NW / 2) * 2 * 64 * sizeof(f32x4) : 0);  // + the score exchange of the wave pairs
  static bool raised = false;  // (per instantiation) dynamic LDS beyond the 64 KB default
  if (!raised) {
    hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attn_mfma_kernel<NKM, RTM, DECODE, NW, DSPLIT, EXACT>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    raised = true;
  }
  latent_attn_mfma_kernel<NKM, RTM, DECODE, NW, DSPLIT, EXACT><<<grid, 64 * NW, lds, s>>>(a);
}

template <int NKM, int RTM, bool EXACT>
void mfma_launch(const LatentAttnArgs& a, hipStream_t s) {
  const int rt = a.kv_rank / 16;
  if (a.tiles) {
    // 64 rows of one head; eight waves (each row group twice, half the latent dims each) where the dims split
    // (8 x 1024 tokens, 16 heads, kv_rank 512: 1090 -> 900 us)
    if (rt % 2 == 0) mfma_launch_one<NKM, RTM, false, 8, 2, EXACT>(a, dim3(a.ntiles, a.H), s);
    else mfma_launch_one<NKM, RTM, false, 4, 1, false>(a, dim3(a.ntiles, a.H), s);
    return;
  }
  // decode rows.  Up to 16 heads: one query group computes, the other three waves only stage (splitting the dims
  // over them re-reads the key tile four times: 64 x 2048 tokens 119 vs 104 us); up to 32 heads: two groups x two
  // dim halves; more: four groups x two (eight waves).  Odd tile counts fall back to unsplit dims.
  if (a.H <= 16 || rt % 2) mfma_launch_one<NKM, RTM, true, 4, 1, EXACT>(a, dim3(a.T, (a.H + 63) / 64, a.parts), s);
  else if (a.H <= 32) mfma_launch_one<NKM, RTM, true, 4, 2, EXACT>(a, dim3(a.T, (a.H + 31) / 32, a.parts), s);
  else mfma_launch_one<NKM, RTM, true, 8, 2, EXACT>(a, dim3(a.T, (a.H + 63) / 64, a.parts), s);
}

bool mfma_dispatch(const LatentAttnArgs& a, hipStream_t s) {
  const int nk = a.Dk / 32, rt = a.kv_rank / 16;
  if (a.Dk % 32 || a.kv_rank % 16 || nk > 18 || rt > 32 || a.part_tokens % KT) return false;
  if (nk == 18 && rt == 32) mfma_launch<18, 32, true>(a, s);       // latent 512 + rotary 64
  else mfma_launch<18, 32, false>(a, s);                           // every other tiled shape
  return true;
}

template <typename T>
void attn_dispatch(const LatentAttnArgs& a, hipStream_t s) {
  dim3 grid(a.T, a.H, a.parts);
  const size_t lds = (size_t)a.Dk * sizeof(float);
  const int nr = (a.kv_rank + 63) / 64;
  if (nr <= 1) latent_attn_wave_kernel<T, 1><<<grid, 64, lds, s>>>(a);
  else if (nr <= 2) latent_attn_wave_kernel<T, 2><<<grid, 64, lds, s>>>(a);
  else if (nr <= 4) latent_attn_wave_kernel<T, 4><<<grid, 64, lds, s>>>(a);
  else latent_attn_wave_kernel<T, 8><<<grid, 64, lds, s>>>(a);
}

}  // namespace


void launch_latent_prep(const LatentPrepArgs& a, int T, int f32, hipStream_t s) {
  if (T <= 0) return;
  if (f32) latent_prep_kernel<float><<<T, NT, 0, s>>>(a);
  else latent_prep_kernel<bf16><<<T, NT, 0, s>>>(a);
}

void launch_rope_pairs(const void* src, long long s_t, long long s_h, void* dst, long long d_t, long long d_h,
                       const int* positions, const float* rope, int T, int H, int rot, int half_dims, int f32,
                       hipStream_t s) {
  if (T <= 0 || rot <= 0) return;
  if (f32)
    rope_pairs_kernel<float><<<T, NT, 0, s>>>((const float*)src, s_t, s_h, (float*)dst, d_t, d_h, positions, rope, H, rot,
                                              half_dims);
  else
    rope_pairs_kernel<bf16><<<T, NT, 0, s>>>((const bf16*)src, s_t, s_h, (bf16*)dst, d_t, d_h, positions, rope, H, rot,
                                             half_dims);
}

int launch_latent_attn(const LatentAttnArgs& a, int f32, int impl, hipStream_t s) {
  if (a.T <= 0) return 0;
  int used = 1;
  if (!f32 && impl != 1 && (a.tiles ? a.ntiles > 0 : true) && mfma_dispatch(a, s)) used = 0;
  else if (f32) attn_dispatch<float>(a, s);
  else attn_dispatch<bf16>(a, s);
  if (a.parts > 1) {
    if (f32) latent_attn_merge_kernel<float><<<dim3(a.T, a.H), 256, 0, s>>>(a);
    else latent_attn_merge_kernel<bf16><<<dim3(a.T, a.H), 256, 0, s>>>(a);
  }
  return used;
}
