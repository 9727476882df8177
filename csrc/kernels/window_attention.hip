// Sliding-window softmax attention with grouped key / value heads over a paged cache, with an optional per-head
// sigmoid output gate and an optional per-head logarithmic distance bias (the score of a key n positions back is
// lowered by b1_h ln(1 + b2_h n)).
//
// Row r (position p of sequence row_seq[r]) sees positions max(0, p - window + 1) .. p and, with keep_first, the
// sequence's first keep_first positions (at their true places in the cache); with a sink the softmax's denominator of
// head h also holds exp(sink[h]), a logit without key or value; query head h reads key / value
// head h / (H / G).  Key and value head sizes are independent (dk, dv).  Scores, softmax statistics, weights and the
// weighted sum are fp32.
//
// window_attn_wave_kernel: one to eight waves per (row, head), every shape, bf16 or fp32.  The window is walked in
// tiles of 64 keys: each lane scores one key (the query sits in LDS as fp32, the key row is read in 16-byte pieces
// where the head size allows), the wave forms the tile's running max / sum, then the lanes switch to value columns
// and add the tile's weighted value rows (weights read lane by lane, value rows read coalesced).
#include "common.h"
#include "hybrid_launchers.h"

namespace {

constexpr int MAX_VCOLS = 8;  // value columns per lane: dv <= 512

// Value columns of a lane.  Plain: lane + 64 i.  PAIR (even dv): two neighbouring columns per load, 128 (i / 2) + 2 lane
// + (i & 1): half the load instructions of the value walk, which is a chain of dependent batches in a decode step.
template <bool PAIR>
SYM_DEV int vcol(int lane, int i) {
  return PAIR ? 128 * (i >> 1) + 2 * lane + (i & 1) : lane + 64 * i;
}
template <bool PAIR>
SYM_DEV int vcols(int dv) {   // accumulator slots in use
  return PAIR ? 2 * ((dv + 127) >> 7) : (dv + 63) >> 6;
}
SYM_DEV void load_pair(const bf16* p, float& a, float& b) {
  const unsigned int w = *reinterpret_cast<const unsigned int*>(p);
  a = __uint_as_float(w << 16);
  b = __uint_as_float(w & 0xffff0000u);
}
SYM_DEV void load_pair(const float* p, float& a, float& b) {
  const float2 w = *reinterpret_cast<const float2*>(p);
  a = w.x, b = w.y;
}

// cache row of position kp of a sequence (block table bt): a shift and a mask for power-of-two blocks
SYM_DEV long long cache_row(const int* __restrict__ bt, int kp, int BS, int shift) {
  return shift >= 0 ? ((long long)bt[kp >> shift] << shift) + (kp & (BS - 1)) : (long long)bt[kp / BS] * BS + kp % BS;
}

// REP dot products of one key row with the REP query vectors of its head group (qs [REP][dk], fp32)
template <typename T, int REP>
SYM_DEV void dot_rows(const T* __restrict__ k, const float* __restrict__ qs, int dk, float* out) {
#pragma unroll
  for (int r = 0; r < REP; ++r) out[r] = 0.f;
  int e = 0;
  if constexpr (sizeof(T) == 2) {
    if ((dk & 7) == 0 && (reinterpret_cast<uintptr_t>(k) & 15) == 0) {
      for (; e < dk; e += 8) {
        float f[8];
        load8(reinterpret_cast<const bf16*>(k) + e, f);
#pragma unroll
        for (int r = 0; r < REP; ++r)
#pragma unroll
          for (int i = 0; i < 8; ++i) out[r] += f[i] * qs[r * dk + e + i];
      }
    }
  } else {
    if ((dk & 3) == 0 && (reinterpret_cast<uintptr_t>(k) & 15) == 0) {
      for (; e < dk; e += 4) {
        const float4 f = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(k) + e);
#pragma unroll
        for (int r = 0; r < REP; ++r) {
          const float* q = qs + r * dk + e;
          out[r] += f.x * q[0] + f.y * q[1] + f.z * q[2] + f.w * q[3];
        }
      }
    }
  }
  for (; e < dk; ++e) {
    const float kv = (float)k[e];
#pragma unroll
    for (int r = 0; r < REP; ++r) out[r] += kv * qs[r * dk + e];
  }
}

// grid (H / REP, T), NW waves.  A workgroup serves REP query heads that share one key / value head (REP = H / G where
// that is 1, 2, 4 or 8, else 1 with one workgroup per head): a key row is read once for the REP scores, a value row
// once for the REP accumulators.  Wave w walks the key tiles w, w + NW, ... of the row's window with its own running
// max / sum / accumulators; the waves' partial results meet in LDS at the end (rows of a decode step have few (row,
// head) pairs and long windows: NW > 1 shortens each wave's walk).  Dynamic LDS: REP dk + NW REP (2 + 64 nvc) floats.
template <typename T, int NW, int REP, bool PAIR>
__global__ __launch_bounds__(64 * NW) void window_attn_wave_kernel(WindowAttnArgs a) {
  extern __shared__ float lds[];
  float* qs = lds;                      // [REP][dk]
  float* part = lds + REP * a.dk;       // [NW][REP][2 + 64 nvc]: m, l, acc
  const int h0 = blockIdx.x * REP, row = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = h0 / (a.H / a.G);
  const int nvc = vcols<PAIR>(a.dv), pstride = 2 + 64 * nvc;
  const int p = a.positions[row];
  const int j0 = max(0, p - a.window + 1);
  // the keys of the row in walking order: the kept first positions that lie before the window, then the window
  const int kf = min(a.keep_first, j0), total = kf + p - j0 + 1;
  const int* bt = a.block_tables + (long long)a.row_seq[row] * a.max_blocks;
  const T* q = reinterpret_cast<const T*>(a.q) + ((long long)row * a.H + h0) * a.dk;   // REP heads: contiguous
  for (int e = threadIdx.x; e < REP * a.dk; e += 64 * NW) qs[e] = (float)q[e] * a.scale;
  __syncthreads();
  const T* kc = reinterpret_cast<const T*>(a.k_cache);
  const T* vc = reinterpret_cast<const T*>(a.v_cache);
  float acc[REP][MAX_VCOLS];
  float m[REP], l[REP], b1[REP], b2[REP];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    b1[r] = a.bias ? a.bias[h0 + r] : 0.f;
    b2[r] = a.bias ? a.bias[a.H + h0 + r] : 0.f;
    m[r] = -INFINITY, l[r] = 0.f;
#pragma unroll
    for (int i = 0; i < MAX_VCOLS; ++i) acc[r][i] = 0.f;
  }
  for (int t0 = 64 * wave; t0 < total; t0 += 64 * NW) {
    const int idx = t0 + lane;
    const bool on = idx < total;
    const int j = idx < kf ? idx : j0 + idx - kf;
    float sc[REP], w[REP];
    long long slot = 0;                       // lanes past the row's last key: weight 0 on a finite row (slot 0)
    if (on) {
      slot = cache_row(bt, j, a.BS, a.bs_shift);
      dot_rows<T, REP>(kc + (slot * a.G + g) * a.dk, qs, a.dk, sc);
      if (a.bias) {
        // (the 32-bit model takes log1pf; bf16 activations the hardware logarithm, whose error is far below their rounding)
        const float dist = (float)(p - j);
#pragma unroll
        for (int r = 0; r < REP; ++r)
          sc[r] -= b1[r] * (sizeof(T) == 4 ? log1pf(b2[r] * dist) : __logf(1.f + b2[r] * dist));
      }
    }
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      const float s = on ? sc[r] : -INFINITY;
      const float mt = fmaxf(m[r], wave_max(s));
      w[r] = on ? expf(s - mt) : 0.f;
      const float corr = expf(m[r] - mt);     // first tile: exp(-inf) = 0 on an all-zero accumulator
      l[r] = l[r] * corr + wave_sum(w[r]);
      m[r] = mt;
#pragma unroll
      for (int i = 0; i < MAX_VCOLS; ++i) acc[r][i] *= corr;
    }
    const int nt = min(64, total - t0);
    const int vslot = (int)slot;              // (cache rows fit 31 bits: checked by the op layer)
    // value rows VB at a time: their cache rows come lane by lane from the scoring phase (no block-table walk in this
    // loop), the loads of a batch are issued together and serve all REP heads
    constexpr int VB = REP >= 4 ? 4 : (PAIR ? 16 : 8);
    for (int jj = 0; jj < nt; jj += VB) {
      float pw[REP][VB];
      const T* vr[VB];
#pragma unroll
      for (int u = 0; u < VB; ++u) {
        vr[u] = vc + ((long long)__shfl(vslot, jj + u, 64) * a.G + g) * a.dv;
#pragma unroll
        for (int r = 0; r < REP; ++r) pw[r][u] = __shfl(w[r], jj + u, 64);
      }
      if constexpr (PAIR) {
#pragma unroll
        for (int i = 0; i < MAX_VCOLS; i += 2) {
          const int c = vcol<true>(lane, i);
          if (c < a.dv) {
            float v0[VB], v1[VB];
#pragma unroll
            for (int u = 0; u < VB; ++u) load_pair(vr[u] + c, v0[u], v1[u]);
#pragma unroll
            for (int r = 0; r < REP; ++r)
#pragma unroll
              for (int u = 0; u < VB; ++u) {
                acc[r][i] += pw[r][u] * v0[u];
                acc[r][i + 1] += pw[r][u] * v1[u];
              }
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < MAX_VCOLS; ++i) {
          const int c = lane + 64 * i;
          if (c < a.dv) {
            float vv[VB];
#pragma unroll
            for (int u = 0; u < VB; ++u) vv[u] = (float)vr[u][c];
#pragma unroll
            for (int r = 0; r < REP; ++r)
#pragma unroll
              for (int u = 0; u < VB; ++u) acc[r][i] += pw[r][u] * vv[u];
          }
        }
      }
    }
  }
  if (NW > 1) {
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      float* mine = part + (wave * REP + r) * pstride;
      if (lane == 0) mine[0] = m[r], mine[1] = l[r];
#pragma unroll
      for (int i = 0; i < MAX_VCOLS; ++i)
        if (i < nvc) mine[2 + 64 * i + lane] = acc[r][i];
    }
    __syncthreads();
    if (wave) return;
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      float M = m[r];
      for (int w2 = 1; w2 < NW; ++w2) M = fmaxf(M, part[(w2 * REP + r) * pstride]);
      const float f0 = expf(m[r] - M);
      m[r] = M;
      l[r] *= f0;
#pragma unroll
      for (int i = 0; i < MAX_VCOLS; ++i) acc[r][i] *= f0;
      for (int w2 = 1; w2 < NW; ++w2) {
        const float* o = part + (w2 * REP + r) * pstride;
        const float f = expf(o[0] - M);       // a wave without tiles: exp(-inf) = 0
        l[r] += o[1] * f;
#pragma unroll
        for (int i = 0; i < MAX_VCOLS; ++i)
          if (i < nvc) acc[r][i] += o[2 + 64 * i + lane] * f;
      }
    }
  }
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    const int h = h0 + r;
    float gate = 1.f;
    if (a.gate) {
      const float gv = (float)reinterpret_cast<const T*>(a.gate)[(long long)row * a.ldg + h];
      gate = 1.f / (1.f + expf(-gv));
    }
    if (a.sink) {     // one more term in the denominator: exp(sink - M) with M = max(m, sink)
      const float sk = a.sink[h], M = fmaxf(m[r], sk);
      const float f = expf(m[r] - M);
      l[r] = l[r] * f + expf(sk - M);
      gate *= f;
    }
    const float inv = gate / l[r];
    T* o = reinterpret_cast<T*>(a.out) + ((long long)row * a.H + h) * a.dv;
#pragma unroll
    for (int i = 0; i < MAX_VCOLS; ++i) {
      const int c = vcol<PAIR>(lane, i);
      if (i < nvc && c < a.dv) o[c] = (T)(acc[r][i] * inv);
    }
  }
}

template <typename T, int NW, int REP, bool PAIR>
void launch_wave_rep(const WindowAttnArgs& a, hipStream_t s) {
  dim3 grid(a.H / REP, a.T);
  const int nvc = PAIR ? 2 * ((a.dv + 127) / 128) : (a.dv + 63) / 64;
  const size_t lds = (size_t)(REP * a.dk + (NW > 1 ? NW * REP * (2 + 64 * nvc) : 0)) * sizeof(float);
  window_attn_wave_kernel<T, NW, REP, PAIR><<<grid, 64 * NW, lds, s>>>(a);
}

template <typename T, int NW>
void launch_wave(const WindowAttnArgs& a, hipStream_t s) {
  // the heads of a key / value group in one workgroup where the group is 2, 4 or 8 heads, the partial results fit LDS and
  // the groups alone still give the chip a thousand waves (8 rows x 4 groups measured 45 us grouped, 30 us per head;
  // 64 rows x 8 groups 128 us grouped, 172 us per head)
  const int rep = a.H / a.G, nvc = (a.dv + 63) / 64;
  const bool fits = (size_t)(rep * a.dk + NW * rep * (2 + 64 * nvc)) * sizeof(float) <= 60 * 1024 && rep * nvc <= 16 &&
                    (long long)a.T * a.G * NW >= 1024;
  if constexpr (NW <= 8) {
    if (rep == 8 && fits) return launch_wave_rep<T, NW, 8, false>(a, s);
    if (rep == 4 && fits) return launch_wave_rep<T, NW, 4, false>(a, s);
    if (rep == 2 && fits) return launch_wave_rep<T, NW, 2, false>(a, s);
  }
  // one head per workgroup: value rows two columns per load where the head size is even (rows stay 4-byte aligned)
  if (a.dv % 2 == 0) launch_wave_rep<T, NW, 1, true>(a, s);
  else launch_wave_rep<T, NW, 1, false>(a, s);
}

// ---- tiled kernel for prompt rows (bf16, head sizes DK = DV in {32, 64, 96, 128}) --------------------------------
// grid (query tiles, heads), 4 waves.  A tile is 64 consecutive rows of one sequence's run (the runner's tile list);
// wave w owns rows 16 w .. 16 w + 15.  Keys walk in tiles of 64 from the first position the tile's first row sees to
// the last row's own position; a key tile's rows go to LDS once for the four waves (keys row-major, values
// transposed), scores are MFMA products K Q^T (each lane ends up with one query row's scores of four keys per 16-key
// subtile: the row statistics are two cross-lane steps), the weights go back into the MFMA as bf16 against the
// transposed values with the keys in the order the score fragments already have.  Statistics, masks and the running
// rescale are fp32.
template <int DK, int DV, int RW>   // RW waves: 16 RW query rows per workgroup (RW = 8: the even tiles of the list, two each)
__global__ __launch_bounds__(64 * RW) void window_attn_tile_kernel(WindowAttnArgs a) {
  constexpr int KD = DK / 32, VD = DV / 16, KS = DK + 8, VS = 64 + 8, NTH = 64 * RW;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  bf16* Ks = reinterpret_cast<bf16*>(smem);   // [64][KS]
  bf16* Vt = Ks + 64 * KS;                    // [DV][VS]
  const int tile = blockIdx.x, h = blockIdx.y;
  const int seq = a.tiles[2 * tile], row0 = a.tiles[2 * tile + 1];
  const int r_hi = a.cu_q[seq + 1], first = a.cu_q[seq] + row0;
  if (first >= r_hi || (RW == 8 && (row0 & 64))) return;   // padding tile / the second half of a pair (whole workgroup)
  const int nrows = min(16 * RW, r_hi - first);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane & 15, hq = lane >> 4;
  const int g = h / (a.H / a.G);
  const int my_row = first + 16 * wave + j;
  const bool rv = 16 * wave + j < nrows;
  const int p_first = a.positions[first], p_last = p_first + nrows - 1;
  const int qp = p_first + 16 * wave + j;
  const int* bt = a.block_tables + (long long)a.row_seq[first] * a.max_blocks;
  const bf16* kc = reinterpret_cast<const bf16*>(a.k_cache);
  const bf16* vc = reinterpret_cast<const bf16*>(a.v_cache);
  Pack8 qf[KD];
  {
    const bf16* q = reinterpret_cast<const bf16*>(a.q) + ((long long)my_row * a.H + h) * DK + 8 * hq;
#pragma unroll
    for (int kk = 0; kk < KD; ++kk) {
      if (rv) qf[kk].u = *reinterpret_cast<const uint4*>(q + 32 * kk);
      else qf[kk].u = make_uint4(0, 0, 0, 0);
    }
  }
  f32x4 o[VD];
#pragma unroll
  for (int i = 0; i < VD; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const float sl2 = a.scale * 1.44269504088896341f;
  // distance bias in units of log2(e): b1 ln(1 + b2 n) log2(e) = b1 log2(1 + b2 n)
  const bool biased = a.bias != nullptr;
  const float b1 = biased ? a.bias[h] : 0.f, b2 = biased ? a.bias[a.H + h] : 0.f;
  const int k_lo = max(0, p_first - a.window + 1);
  // cache blocks of 64 tokens or a multiple: a key tile lies in one block, whose number is read one tile ahead (the
  // rows' loads then do not wait for a block-table load of their own)
  const bool one_block = a.bs_shift >= 6;
  // key tiles in walking order: the tiles of the kept first positions that lie before the window's first tile, then the
  // window's tiles up to the last row's own position
  const int kt_win = k_lo & ~63;
  const int kt_first = (a.keep_first > 0 && kt_win > 0) ? 0 : kt_win;
  auto tile_after = [&](int kt) { return (kt < kt_win && kt + 64 >= min(a.keep_first, kt_win)) ? kt_win : kt + 64; };
  int blk_next = one_block ? bt[kt_first >> a.bs_shift] : 0;
  for (int kt = kt_first; kt <= p_last; kt = tile_after(kt)) {
    const long long blk_base = (long long)blk_next << (one_block ? a.bs_shift : 0);
    if (one_block && tile_after(kt) <= p_last) blk_next = bt[tile_after(kt) >> a.bs_shift];
    auto row_of = [&](int kp) {
      return one_block ? blk_base + (kp & (a.BS - 1)) : cache_row(bt, kp, a.BS, a.bs_shift);
    };
    __syncthreads();                          // every wave is done with the previous tile
    for (int id = threadIdx.x; id < 64 * (DK / 8); id += NTH) {
      const int key = id / (DK / 8), ch = id - key * (DK / 8);
      const int kp = kt + key;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (kp <= p_last) {
        const long long slot = row_of(kp);
        v = *reinterpret_cast<const uint4*>(kc + (slot * a.G + g) * DK + 8 * ch);
      }
      *reinterpret_cast<uint4*>(Ks + key * KS + 8 * ch) = v;
    }
    // values transposed: a thread takes 8 columns of two neighbouring keys and stores them as eight 4-byte words (a key
    // pair per word), consecutive lanes writing consecutive words of a column's row.  (Fetching the next tile into
    // registers ahead of the products measured slower: the workgroups sharing a CU already cover the load latency.)
    for (int id = threadIdx.x; id < 32 * (DV / 8); id += NTH) {
      const int ch = id / 32, key = 2 * (id - ch * 32);
      Pack8 va, vb;
      va.u = vb.u = make_uint4(0, 0, 0, 0);
      const int kp = kt + key;
      if (kp <= p_last) {
        const long long slot = row_of(kp);
        va.u = *reinterpret_cast<const uint4*>(vc + (slot * a.G + g) * DV + 8 * ch);
      }
      if (kp + 1 <= p_last) {
        const long long slot = row_of(kp + 1);
        vb.u = *reinterpret_cast<const uint4*>(vc + (slot * a.G + g) * DV + 8 * ch);
      }
#pragma unroll
      for (int m2 = 0; m2 < 4; ++m2) {
        const unsigned int wa = va.w[m2], wb = vb.w[m2];
        unsigned int* dst = reinterpret_cast<unsigned int*>(Vt + (8 * ch + 2 * m2) * VS + key);
        dst[0] = (wa & 0xffffu) | (wb << 16);
        dst[VS / 2] = (wa >> 16) | (wb & 0xffff0000u);
      }
    }
    __syncthreads();
    // scores in units of log2(e): sc[s][e] = scale * log2(e) * q_j . k_(kt + 16 s + 4 hq + e).  A key tile that every
    // row of the wave sees completely (the usual case away from the diagonal and the window's far edge) skips the masks.
    const int wq_lo = p_first + 16 * wave, wq_hi = wq_lo + 15;
    const bool interior = 16 * wave + 15 < nrows && kt + 63 <= wq_lo && (kt > wq_hi - a.window || kt + 63 < a.keep_first);
    float pv[4][4];
    float mx = -INFINITY;
    // 1 + b2 (qp - kp) for key kp = kt + 16 s4 + 4 hq + e is arg0 - b2 (16 s4 + e): one multiply-add per score
    const float arg0 = 1.f + b2 * (float)(qp - kt - 4 * hq), nb1 = -b1;
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) {
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KD; ++kk) {
        Pack8 kf;
        kf.u = *reinterpret_cast<const uint4*>(Ks + (16 * s4 + j) * KS + 32 * kk + 8 * hq);
        acc = mfma16(kf.v, qf[kk].v, acc);
      }
      if (interior) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          pv[s4][e] = acc[e] * sl2;
          if (biased) pv[s4][e] += nb1 * __log2f(arg0 - b2 * (float)(16 * s4 + e));
          mx = fmaxf(mx, pv[s4][e]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int kp = kt + 16 * s4 + 4 * hq + e;
          const bool vis = rv && kp <= qp && (kp > qp - a.window || kp < a.keep_first);
          float sv = acc[e] * sl2;
          if (biased) sv += nb1 * __log2f(arg0 - b2 * (float)(16 * s4 + e));   // (keys past the row: masked below)
          pv[s4][e] = vis ? sv : -INFINITY;
          mx = fmaxf(mx, pv[s4][e]);
        }
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mt = fmaxf(m, mx);
    const float mref = mt == -INFINITY ? 0.f : mt;   // a row that sees nothing yet
    float sum = 0.f;
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        pv[s4][e] = exp2f(pv[s4][e] - mref);
        sum += pv[s4][e];
      }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    if (__any(mt > m)) {                             // some row's running max moved: rescale (else every factor is 1)
      const float corr = exp2f(m - mref);
      l *= corr;
#pragma unroll
      for (int i = 0; i < VD; ++i) o[i] *= corr;
    }
    l += sum;
    m = mt;
    // weighted values: key slots of lane group hq in a 32-key chunk c2 are keys 32 c2 + 4 hq + (0..3) and + 16
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2) {
      Pack8 pf;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        pf.h[e] = (bf16)pv[2 * c2][e];
        pf.h[4 + e] = (bf16)pv[2 * c2 + 1][e];
      }
#pragma unroll
      for (int cb = 0; cb < VD; ++cb) {
        const bf16* vrow = Vt + (16 * cb + j) * VS + 32 * c2 + 4 * hq;
        Pack8 vf;
        const uint2 lo = *reinterpret_cast<const uint2*>(vrow), hi = *reinterpret_cast<const uint2*>(vrow + 16);
        vf.u = make_uint4(lo.x, lo.y, hi.x, hi.y);
        o[cb] = mfma16(vf.v, pf.v, o[cb]);
      }
    }
  }
  if (!rv) return;
  float gate = 1.f;
  if (a.gate) {
    const float gv = (float)reinterpret_cast<const bf16*>(a.gate)[(long long)my_row * a.ldg + h];
    gate = 1.f / (1.f + expf(-gv));
  }
  if (a.sink) {     // one more term in the denominator (m is in units of log2 e)
    const float sk = a.sink[h] * 1.44269504088896341f, M = fmaxf(m, sk);
    const float f = exp2f(m - M);
    l = l * f + exp2f(sk - M);
    gate *= f;
  }
  const float inv = gate / l;
  bf16* out = reinterpret_cast<bf16*>(a.out) + ((long long)my_row * a.H + h) * DV + 4 * hq;
#pragma unroll
  for (int cb = 0; cb < VD; ++cb) {
    bf16x4 w4;
#pragma unroll
    for (int e = 0; e < 4; ++e) w4[e] = (bf16)(o[cb][e] * inv);
    *reinterpret_cast<bf16x4*>(out + 16 * cb) = w4;
  }
}

template <int D>
void launch_tile(const WindowAttnArgs& a, int rw, hipStream_t s) {
  dim3 grid(a.ntiles, a.H);
  const size_t lds = (size_t)(64 * (D + 8) + D * (64 + 8)) * sizeof(bf16);
  if (rw == 8) window_attn_tile_kernel<D, D, 8><<<grid, 512, lds, s>>>(a);
  else window_attn_tile_kernel<D, D, 4><<<grid, 256, lds, s>>>(a);
}

}  // namespace

int launch_window_attn(const WindowAttnArgs& args, int f32, int impl, hipStream_t s) {
  if (args.T <= 0) return 0;
  WindowAttnArgs a = args;
  a.bs_shift = -1;
  for (int b = 0; b < 31; ++b)
    if (a.BS == 1 << b) a.bs_shift = b;
  if (impl >= 1 && !f32 && a.tiles && a.cu_q && a.ntiles > 0 && a.dk == a.dv && a.ntiles <= 65535 * 16) {
    const int rw = impl == 2 ? 8 : 4;
    switch (a.dk) {
      case 32: launch_tile<32>(a, rw, s); return 1;
      case 64: launch_tile<64>(a, rw, s); return 1;
      case 96: launch_tile<96>(a, rw, s); return 1;
      case 128: launch_tile<128>(a, rw, s); return 1;
      default: break;
    }
  }
  // few (row, head) pairs and a long window (decode steps): several waves per pair
  // (a handful of rows over a thousand keys or more: sixteen waves, one or two key tiles each)
  const long long pairs = (long long)a.T * a.H;
  const long long reach = min((long long)a.window, (long long)a.max_blocks * a.BS);   // keys a row can see at most
  const int nw = pairs >= 8192 || a.window <= 128 ? 1
                 : (a.window <= 512 || pairs >= 2048 ? 4 : (pairs <= 512 && reach >= 1024 ? 16 : 8));
  if (f32) {
    if (nw == 1) launch_wave<float, 1>(a, s);
    else if (nw == 4) launch_wave<float, 4>(a, s);
    else if (nw == 8) launch_wave<float, 8>(a, s);
    else launch_wave<float, 16>(a, s);
  } else {
    if (nw == 1) launch_wave<bf16, 1>(a, s);
    else if (nw == 4) launch_wave<bf16, 4>(a, s);
    else if (nw == 8) launch_wave<bf16, 8>(a, s);
    else launch_wave<bf16, 16>(a, s);
  }
  return 0;
}
