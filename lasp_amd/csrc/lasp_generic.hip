// Generic kernels: fp32 FMA arithmetic on LDS-resident tiles, any element type,
// any chunk length (ragged tail masked), d, e <= 128.  They serve the fp32
// configuration (tolerance 1e-3 rules out bf16 operands) and every shape the
// MFMA kernels do not take.  Structure per (b, h, segment) workgroup:
//   - tiles of GB = 32 tokens are converted to fp32 in LDS,
//   - the d x e state lives in LDS in fp32 and is carried across tiles,
//   - every decay exponent is <= 0 (l^i, l^(len-j), l^(i-j) for i >= j), as in
//     lasp/lightning_attention.py:42-52.
// Math per tile follows lasp/lasp_fuse.py:104-124 (forward), :237-260 (dq sweep)
// and :316-350 (reverse dk/dv sweep).
#include "lasp_common.h"

namespace lasp {
namespace {

constexpr int GB = 32;    // tokens per tile
constexpr int NT = 256;   // threads per workgroup
constexpr int LDS_S = GB + 1;

// out(m, n) = sum_k A[m*am + k*ak] * B[k*bk + n*bn]
template <class F>
__device__ __forceinline__ void tile_mm(int M, int N, int K, const float *A, int am, int ak,
                                        const float *B, int bk, int bn, F &&epi) {
  for (int idx = threadIdx.x; idx < M * N; idx += NT) {
    const int m = idx / N, n = idx - m * N;
    const float *a = A + m * am;
    const float *bp = B + n * bn;
    float acc = 0.f;
    for (int kk = 0; kk < K; ++kk) acc = fmaf(a[kk * ak], bp[kk * bk], acc);
    epi(m, n, acc);
  }
}

// two products with a common output index
template <class F>
__device__ __forceinline__ void tile_mm2(int M, int N, int K1, const float *A1, int a1m, int a1k,
                                         const float *B1, int b1k, int b1n, int K2,
                                         const float *A2, int a2m, int a2k, const float *B2,
                                         int b2k, int b2n, F &&epi) {
  for (int idx = threadIdx.x; idx < M * N; idx += NT) {
    const int m = idx / N, n = idx - m * N;
    float acc1 = 0.f, acc2 = 0.f;
    {
      const float *a = A1 + m * a1m;
      const float *bp = B1 + n * b1n;
      for (int kk = 0; kk < K1; ++kk) acc1 = fmaf(a[kk * a1k], bp[kk * b1k], acc1);
    }
    {
      const float *a = A2 + m * a2m;
      const float *bp = B2 + n * b2n;
      for (int kk = 0; kk < K2; ++kk) acc2 = fmaf(a[kk * a2k], bp[kk * b2k], acc2);
    }
    epi(m, n, acc1, acc2);
  }
}

// rows [0, valid) of a (rows x cols) tile from global memory, the rest zero
template <class T>
__device__ __forceinline__ void load_tile(float *dst, int ld, const T *src, int valid, int cols) {
  for (int idx = threadIdx.x; idx < GB * cols; idx += NT) {
    const int r = idx / cols, c = idx - r * cols;
    dst[r * ld + c] = (r < valid) ? elem<T>::load(src + (int64_t)r * cols + c) : 0.f;
  }
}

__device__ __forceinline__ void load_state(float *dst, int ld, const float *src, int rows, int cols) {
  for (int idx = threadIdx.x; idx < rows * cols; idx += NT) {
    const int r = idx / cols, c = idx - r * cols;
    dst[r * ld + c] = src ? src[idx] : 0.f;
  }
}

// lamq[i] = l^i ; lamk[j] = l^(len - j)   (also the mask: M_ij = lamq[i - j])
__device__ __forceinline__ void fill_decay(float *lamq, float *lamk, float s, int len) {
  if (threadIdx.x < GB) {
    lamq[threadIdx.x] = expf(-s * (float)threadIdx.x);
    lamk[threadIdx.x] = expf(-s * (float)(len - (int)threadIdx.x));
  }
}

struct SegRange {
  int bh, seg;
  int64_t t0, t1;  // token range of this segment inside the chunk
};
__device__ __forceinline__ SegRange seg_range(const Geom &g) {
  SegRange r;
  r.bh = blockIdx.x / g.n_seg;
  r.seg = blockIdx.x - r.bh * g.n_seg;
  r.t0 = (int64_t)r.seg * g.seg_len;
  r.t1 = r.t0 + g.seg_len;
  if (r.t1 > g.n) r.t1 = g.n;
  return r;
}

// ------------------------------------------------------------------ local state
// forward mode: state = sum_j l^(L - j) x_j^T y_j    (L = segment length, j from its start)
// reverse mode: state = sum_i l^i       x_i^T y_i
template <class T>
__global__ void __launch_bounds__(NT)
generic_seg_state(const T *__restrict__ X, const T *__restrict__ Y, const float *__restrict__ S,
                  float *__restrict__ states, Geom g, int reverse) {
  extern __shared__ float smem[];
  const int d = g.d, e = g.e, ldd = d + 1, lde = e + 1;
  float *sX = smem;
  float *sY = sX + GB * ldd;
  float *sSt = sY + GB * lde;
  float *lamq = sSt + d * lde;
  float *lamk = lamq + GB;

  const SegRange r = seg_range(g);
  const float s = S[r.bh % g.h];
  const T *Xb = X + (int64_t)r.bh * g.n * d;
  const T *Yb = Y + (int64_t)r.bh * g.n * e;

  load_state(sSt, lde, nullptr, d, e);
  const int64_t ntile = (r.t1 - r.t0 + GB - 1) / GB;
  for (int64_t it = 0; it < ntile; ++it) {
    const int64_t t = r.t0 + (reverse ? (ntile - 1 - it) : it) * GB;
    const int len = (int)((r.t1 - t) < GB ? (r.t1 - t) : GB);
    __syncthreads();
    load_tile(sX, ldd, Xb + t * d, len, d);
    load_tile(sY, lde, Yb + t * e, len, e);
    fill_decay(lamq, lamk, s, len);
    __syncthreads();
    const float blk = expf(-s * (float)len);
    const float *w = reverse ? lamq : lamk;
    for (int idx = threadIdx.x; idx < d * e; idx += NT) {
      const int dd = idx / e, c = idx - dd * e;
      float acc = 0.f;
      for (int j = 0; j < len; ++j) acc = fmaf(w[j] * sX[j * ldd + dd], sY[j * lde + c], acc);
      sSt[dd * lde + c] = fmaf(blk, sSt[dd * lde + c], acc);
    }
  }
  __syncthreads();
  float *out = states + ((int64_t)r.bh * g.n_seg + r.seg) * d * e;
  for (int idx = threadIdx.x; idx < d * e; idx += NT) {
    const int dd = idx / e, c = idx - dd * e;
    out[idx] = sSt[dd * lde + c];
  }
}

// ------------------------------------------------------------------ forward
template <class T>
__global__ void __launch_bounds__(NT)
generic_fwd_apply(const T *__restrict__ Q, const T *__restrict__ K, const T *__restrict__ V,
                  const float *__restrict__ S, const float *__restrict__ states,
                  T *__restrict__ O, Geom g) {
  extern __shared__ float smem[];
  const int d = g.d, e = g.e, ldd = d + 1, lde = e + 1;
  float *sQ = smem;
  float *sK = sQ + GB * ldd;
  float *sV = sK + GB * ldd;
  float *sS = sV + GB * lde;
  float *sKV = sS + GB * LDS_S;
  float *lamq = sKV + d * lde;
  float *lamk = lamq + GB;

  const SegRange r = seg_range(g);
  const float s = S[r.bh % g.h];
  const T *Qb = Q + (int64_t)r.bh * g.n * d;
  const T *Kb = K + (int64_t)r.bh * g.n * d;
  const T *Vb = V + (int64_t)r.bh * g.n * e;
  T *Ob = O + (int64_t)r.bh * g.n * e;

  load_state(sKV, lde, states ? states + ((int64_t)r.bh * g.n_seg + r.seg) * d * e : nullptr, d, e);

  for (int64_t t = r.t0; t < r.t1; t += GB) {
    const int len = (int)((r.t1 - t) < GB ? (r.t1 - t) : GB);
    __syncthreads();
    load_tile(sQ, ldd, Qb + t * d, len, d);
    load_tile(sK, ldd, Kb + t * d, len, d);
    load_tile(sV, lde, Vb + t * e, len, e);
    fill_decay(lamq, lamk, s, len);
    __syncthreads();
    // S_ij = (q_i . k_j) l^(i-j) for j <= i
    tile_mm(GB, GB, d, sQ, ldd, 1, sK, 1, ldd, [&](int i, int j, float acc) {
      sS[i * LDS_S + j] = (j <= i) ? acc * lamq[i - j] : 0.f;
    });
    __syncthreads();
    // O_i = sum_j S_ij v_j + l^i q_i KV
    tile_mm2(GB, e, GB, sS, LDS_S, 1, sV, lde, 1, d, sQ, ldd, 1, sKV, lde, 1,
             [&](int i, int c, float intra, float inter) {
               if (i < len) elem<T>::store(Ob + (t + i) * e + c, fmaf(lamq[i], inter, intra));
             });
    __syncthreads();
    // KV <- l^len KV + sum_j l^(len-j) k_j^T v_j
    const float blk = expf(-s * (float)len);
    for (int idx = threadIdx.x; idx < d * e; idx += NT) {
      const int dd = idx / e, c = idx - dd * e;
      float acc = 0.f;
      for (int j = 0; j < len; ++j) acc = fmaf(lamk[j] * sK[j * ldd + dd], sV[j * lde + c], acc);
      sKV[dd * lde + c] = fmaf(blk, sKV[dd * lde + c], acc);
    }
  }
}

// ------------------------------------------------------------------ backward: dQ
template <class T>
__global__ void __launch_bounds__(NT)
generic_bwd_dq(const T *__restrict__ K, const T *__restrict__ V, const T *__restrict__ DO,
               const float *__restrict__ S, const float *__restrict__ states,
               T *__restrict__ DQ, Geom g) {
  extern __shared__ float smem[];
  const int d = g.d, e = g.e, ldd = d + 1, lde = e + 1;
  float *sDO = smem;
  float *sV = sDO + GB * lde;
  float *sK = sV + GB * lde;
  float *sP = sK + GB * ldd;
  float *sKV = sP + GB * LDS_S;
  float *lamq = sKV + d * lde;
  float *lamk = lamq + GB;

  const SegRange r = seg_range(g);
  const float s = S[r.bh % g.h];
  const T *Kb = K + (int64_t)r.bh * g.n * d;
  const T *Vb = V + (int64_t)r.bh * g.n * e;
  const T *DOb = DO + (int64_t)r.bh * g.n * e;
  T *DQb = DQ + (int64_t)r.bh * g.n * d;

  load_state(sKV, lde, states ? states + ((int64_t)r.bh * g.n_seg + r.seg) * d * e : nullptr, d, e);

  for (int64_t t = r.t0; t < r.t1; t += GB) {
    const int len = (int)((r.t1 - t) < GB ? (r.t1 - t) : GB);
    __syncthreads();
    load_tile(sDO, lde, DOb + t * e, len, e);
    load_tile(sV, lde, Vb + t * e, len, e);
    load_tile(sK, ldd, Kb + t * d, len, d);
    fill_decay(lamq, lamk, s, len);
    __syncthreads();
    // P_ij = (dO_i . v_j) l^(i-j) for j <= i
    tile_mm(GB, GB, e, sDO, lde, 1, sV, 1, lde, [&](int i, int j, float acc) {
      sP[i * LDS_S + j] = (j <= i) ? acc * lamq[i - j] : 0.f;
    });
    __syncthreads();
    // dQ_i = sum_j P_ij k_j + l^i dO_i KV^T
    tile_mm2(GB, d, GB, sP, LDS_S, 1, sK, ldd, 1, e, sDO, lde, 1, sKV, 1, lde,
             [&](int i, int c, float intra, float inter) {
               if (i < len) elem<T>::store(DQb + (t + i) * d + c, fmaf(lamq[i], inter, intra));
             });
    __syncthreads();
    const float blk = expf(-s * (float)len);
    for (int idx = threadIdx.x; idx < d * e; idx += NT) {
      const int dd = idx / e, c = idx - dd * e;
      float acc = 0.f;
      for (int j = 0; j < len; ++j) acc = fmaf(lamk[j] * sK[j * ldd + dd], sV[j * lde + c], acc);
      sKV[dd * lde + c] = fmaf(blk, sKV[dd * lde + c], acc);
    }
  }
}

// ------------------------------------------------------------------ backward: dK, dV
template <class T>
__global__ void __launch_bounds__(NT)
generic_bwd_dkdv(const T *__restrict__ Q, const T *__restrict__ K, const T *__restrict__ V,
                 const T *__restrict__ DO, const float *__restrict__ S,
                 const float *__restrict__ states, T *__restrict__ DK, T *__restrict__ DV, Geom g) {
  extern __shared__ float smem[];
  const int d = g.d, e = g.e, ldd = d + 1, lde = e + 1;
  float *sQ = smem;
  float *sK = sQ + GB * ldd;
  float *sV = sK + GB * ldd;
  float *sDO = sV + GB * lde;
  float *sS = sDO + GB * lde;
  float *sP = sS + GB * LDS_S;
  float *sD = sP + GB * LDS_S;  // dkv state, d x e
  float *lamq = sD + d * lde;
  float *lamk = lamq + GB;

  const SegRange r = seg_range(g);
  const float s = S[r.bh % g.h];
  const T *Qb = Q + (int64_t)r.bh * g.n * d;
  const T *Kb = K + (int64_t)r.bh * g.n * d;
  const T *Vb = V + (int64_t)r.bh * g.n * e;
  const T *DOb = DO + (int64_t)r.bh * g.n * e;
  T *DKb = DK + (int64_t)r.bh * g.n * d;
  T *DVb = DV + (int64_t)r.bh * g.n * e;

  load_state(sD, lde, states ? states + ((int64_t)r.bh * g.n_seg + r.seg) * d * e : nullptr, d, e);

  const int64_t ntile = (r.t1 - r.t0 + GB - 1) / GB;
  for (int64_t it = ntile - 1; it >= 0; --it) {
    const int64_t t = r.t0 + it * GB;
    const int len = (int)((r.t1 - t) < GB ? (r.t1 - t) : GB);
    __syncthreads();
    load_tile(sQ, ldd, Qb + t * d, len, d);
    load_tile(sK, ldd, Kb + t * d, len, d);
    load_tile(sV, lde, Vb + t * e, len, e);
    load_tile(sDO, lde, DOb + t * e, len, e);
    fill_decay(lamq, lamk, s, len);
    __syncthreads();
    tile_mm2(GB, GB, d, sQ, ldd, 1, sK, 1, ldd, e, sDO, lde, 1, sV, 1, lde,
             [&](int i, int j, float qk, float dov) {
               const float m = (j <= i) ? lamq[i - j] : 0.f;
               sS[i * LDS_S + j] = qk * m;
               sP[i * LDS_S + j] = dov * m;
             });
    __syncthreads();
    // dK_j = sum_i P_ij q_i + l^(len-j) v_j DKV^T
    tile_mm2(GB, d, GB, sP, 1, LDS_S, sQ, ldd, 1, e, sV, lde, 1, sD, 1, lde,
             [&](int j, int c, float intra, float inter) {
               if (j < len) elem<T>::store(DKb + (t + j) * d + c, fmaf(lamk[j], inter, intra));
             });
    // dV_j = sum_i S_ij dO_i + l^(len-j) k_j DKV
    tile_mm2(GB, e, GB, sS, 1, LDS_S, sDO, lde, 1, d, sK, ldd, 1, sD, lde, 1,
             [&](int j, int c, float intra, float inter) {
               if (j < len) elem<T>::store(DVb + (t + j) * e + c, fmaf(lamk[j], inter, intra));
             });
    __syncthreads();
    // DKV <- l^len DKV + sum_i l^i q_i^T dO_i
    const float blk = expf(-s * (float)len);
    for (int idx = threadIdx.x; idx < d * e; idx += NT) {
      const int dd = idx / e, c = idx - dd * e;
      float acc = 0.f;
      for (int i = 0; i < len; ++i) acc = fmaf(lamq[i] * sQ[i * ldd + dd], sDO[i * lde + c], acc);
      sD[dd * lde + c] = fmaf(blk, sD[dd * lde + c], acc);
    }
  }
}

// ------------------------------------------------------------------ segment scan
// W consecutive columns of the stored (sd x se) state per thread (the carries are d x e).  W = 4
// moves 16 bytes per lane and needs se % 4 == 0, e % 4 == 0 and 16-byte aligned states.
template <int W>
struct ScanVec {
  float v[W];
  __device__ void load(const float *p) {
    if constexpr (W == 4) {
      const float4 t = *reinterpret_cast<const float4 *>(p);
      v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
    } else {
      v[0] = *p;
    }
  }
  __device__ void store(float *p) const {
    if constexpr (W == 4) {
      *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
      *p = v[0];
    }
  }
};

template <int W>
__global__ void __launch_bounds__(256)
segment_scan_kernel(float *__restrict__ states, const float *carry_in, float *carry_out,
                    const float *__restrict__ S, Geom g, int reverse) {
  const int64_t sde = (int64_t)g.sd * g.se;
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * W;
  const int64_t total = (int64_t)g.b * g.h * sde;
  if (idx >= total) return;
  const int bh = (int)(idx / sde);
  const int64_t el = idx - (int64_t)bh * sde;
  const int row = (int)(el / g.se), col = (int)(el - (int64_t)row * g.se);
  const bool in_carry = row < g.d && col < g.e;  // the padding of a stored state stays zero
  const int64_t cidx = ((int64_t)bh * g.d + row) * g.e + col;
  const float s = S[bh % g.h];
  ScanVec<W> run;
#pragma unroll
  for (int w = 0; w < W; ++w) run.v[w] = (carry_in && in_carry) ? carry_in[cidx + w] : 0.f;
  float *p = states + (int64_t)bh * g.n_seg * sde + el;
  const float full = expf(-s * (float)g.seg_len);
  const int64_t last_len = g.n - (int64_t)(g.n_seg - 1) * g.seg_len;
  const float tail = expf(-s * (float)last_len);
  if (state_dies_in_segment(s, g)) {
    // This head's own states stay as the pre-pass wrote them (the sweeps read the neighbour's).  Only the
    // outgoing carry is formed, from the two segments visited last: anything older has faded below 2^-24.
    const int prev = reverse ? 1 : g.n_seg - 2, end = reverse ? 0 : g.n_seg - 1;
    if (carry_out && in_carry) {
      ScanVec<W> a, b;
      a.load(p + (int64_t)prev * sde);
      b.load(p + (int64_t)end * sde);
      const float f = end == g.n_seg - 1 ? tail : full;
#pragma unroll
      for (int w = 0; w < W; ++w) carry_out[cidx + w] = fmaf(f, a.v[w], b.v[w]);
    }
    // The incoming carry (read above, before the outgoing one was written: the two may be the same memory)
    // moves into the slot of the segment visited last, whose own state nothing reads from here on; the sweep
    // of the segment visited first takes it from there, zero-extended like every state of the workspace.
    if (carry_in) run.store(p + (int64_t)end * sde);
    return;
  }
  // The loads do not depend on the recurrence: a batch of segment states is fetched while the
  // serial chain runs over the batch before it (forward: segments ascending; reverse: descending).
  constexpr int BATCH = 8;
  auto fetch = [&](int done, ScanVec<W> (&local)[BATCH]) {
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int k = done + u < g.n_seg ? done + u : g.n_seg - 1;  // past the end: a harmless repeat
      const int sg = reverse ? g.n_seg - 1 - k : k;
      local[u].load(p + (int64_t)sg * sde);
    }
  };
  ScanVec<W> cur[BATCH], nxt[BATCH];
  fetch(0, cur);
  for (int done = 0; done < g.n_seg; done += BATCH) {
    const bool more = done + BATCH < g.n_seg;
    if (more) fetch(done + BATCH, nxt);
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int k = done + u;
      if (k < g.n_seg) {
        const int sg = reverse ? g.n_seg - 1 - k : k;
        run.store(p + (int64_t)sg * sde);
        const float f = sg == g.n_seg - 1 ? tail : full;
#pragma unroll
        for (int w = 0; w < W; ++w) run.v[w] = fmaf(f, run.v[w], cur[u].v[w]);
      }
    }
    if (more) {
#pragma unroll
      for (int u = 0; u < BATCH; ++u) cur[u] = nxt[u];
    }
  }
  if (carry_out && in_carry) {
#pragma unroll
    for (int w = 0; w < W; ++w) carry_out[cidx + w] = run.v[w];
  }
}

// the largest dynamic LDS any kernel of this family asks for (generic_bwd_dkdv at d = e = 128)
constexpr int GENERIC_MAX_LDS = (int)sizeof(float) * (4 * GB * 129 + 2 * GB * LDS_S + 128 * 129 + 2 * GB);

template <class T>
int fwd_t(const FwdArgs &a, const Geom &g, hipStream_t st) {
  const int d = g.d, e = g.e, ldd = d + 1, lde = e + 1;
  const unsigned grid = (unsigned)((int64_t)g.b * g.h * g.n_seg);
  int rc;
  const bool need_states = g.n_seg > 1 || a.kv_in || a.kv_out;
  if (need_states) {
    const size_t lds = sizeof(float) * (GB * ldd + GB * lde + d * lde + 2 * GB);
    if ((rc = grant_lds<generic_seg_state<T>>(GENERIC_MAX_LDS))) return rc;
    {
      ProfScope prof(KC_GENERIC, st);
      generic_seg_state<T><<<grid, NT, lds, st>>>((const T *)a.k, (const T *)a.v, a.s, a.seg_states, g, 0);
    }
    if ((rc = launch_segment_scan(a.seg_states, a.kv_in, a.kv_out, a.s, g, 0, st))) return rc;
  }
  const size_t lds = sizeof(float) * (2 * GB * ldd + GB * lde + GB * LDS_S + d * lde + 2 * GB);
  if ((rc = grant_lds<generic_fwd_apply<T>>(GENERIC_MAX_LDS))) return rc;
  ProfScope prof(KC_GENERIC, st);
  generic_fwd_apply<T><<<grid, NT, lds, st>>>((const T *)a.q, (const T *)a.k, (const T *)a.v, a.s,
                                              need_states ? a.seg_states : nullptr, (T *)a.o, g);
  return (int)hipGetLastError();
}

template <class T>
int bwd_t(const BwdArgs &a, const Geom &g, hipStream_t st) {
  const int d = g.d, e = g.e, ldd = d + 1, lde = e + 1;
  const unsigned grid = (unsigned)((int64_t)g.b * g.h * g.n_seg);
  int rc;
  const size_t lds_state = sizeof(float) * (GB * ldd + GB * lde + d * lde + 2 * GB);
  if ((rc = grant_lds<generic_seg_state<T>>(GENERIC_MAX_LDS))) return rc;

  const float *kv_states = a.kv_seg_states;
  if (!kv_states && (g.n_seg > 1 || a.kv_in)) {
    {
      ProfScope prof(KC_GENERIC, st);
      generic_seg_state<T><<<grid, NT, lds_state, st>>>((const T *)a.k, (const T *)a.v, a.s, a.ws_kv, g, 0);
    }
    if ((rc = launch_segment_scan(a.ws_kv, a.kv_in, nullptr, a.s, g, 0, st))) return rc;
    kv_states = a.ws_kv;
  }
  const float *dkv_states = nullptr;
  if (g.n_seg > 1 || a.dkv_in || a.dkv_out) {
    {
      ProfScope prof(KC_GENERIC, st);
      generic_seg_state<T><<<grid, NT, lds_state, st>>>((const T *)a.q, (const T *)a.d_o, a.s, a.ws_dkv, g, 1);
    }
    if ((rc = launch_segment_scan(a.ws_dkv, a.dkv_in, a.dkv_out, a.s, g, 1, st))) return rc;
    dkv_states = a.ws_dkv;
  }
  {
    const size_t lds = sizeof(float) * (2 * GB * lde + GB * ldd + GB * LDS_S + d * lde + 2 * GB);
    if ((rc = grant_lds<generic_bwd_dq<T>>(GENERIC_MAX_LDS))) return rc;
    ProfScope prof(KC_GENERIC, st);
    generic_bwd_dq<T><<<grid, NT, lds, st>>>((const T *)a.k, (const T *)a.v, (const T *)a.d_o, a.s,
                                             kv_states, (T *)a.dq, g);
  }
  {
    const size_t lds =
        sizeof(float) * (2 * GB * ldd + 2 * GB * lde + 2 * GB * LDS_S + d * lde + 2 * GB);
    if ((rc = grant_lds<generic_bwd_dkdv<T>>(GENERIC_MAX_LDS))) return rc;
    ProfScope prof(KC_GENERIC, st);
    generic_bwd_dkdv<T><<<grid, NT, lds, st>>>((const T *)a.q, (const T *)a.k, (const T *)a.v,
                                               (const T *)a.d_o, a.s, dkv_states, (T *)a.dk,
                                               (T *)a.dv, g);
  }
  return (int)hipGetLastError();
}

}  // namespace

int launch_segment_scan(float *states, const float *carry_in, float *carry_out, const float *s,
                        const Geom &g, int reverse, hipStream_t st) {
  const int64_t total = (int64_t)g.b * g.h * g.sd * g.se;
  const bool wide = g.se % 4 == 0 && g.e % 4 == 0 && (uintptr_t)states % 16 == 0;
  const int64_t threads = wide ? total / 4 : total;
  const unsigned grid = (unsigned)((threads + 255) / 256);
  ProfScope prof(KC_SCAN, st);
  if (wide)
    segment_scan_kernel<4><<<grid, 256, 0, st>>>(states, carry_in, carry_out, s, g, reverse);
  else
    segment_scan_kernel<1><<<grid, 256, 0, st>>>(states, carry_in, carry_out, s, g, reverse);
  return (int)hipGetLastError();
}

int generic_fwd(const FwdArgs &a, const Geom &g, int dtype, hipStream_t st) {
  switch (dtype) {
    case LASP_DTYPE_F32: return fwd_t<float>(a, g, st);
    case LASP_DTYPE_BF16: return fwd_t<bf16_tag>(a, g, st);
    case LASP_DTYPE_F16: return fwd_t<_Float16>(a, g, st);
  }
  return LASP_E_DTYPE;
}

int generic_bwd(const BwdArgs &a, const Geom &g, int dtype, hipStream_t st) {
  switch (dtype) {
    case LASP_DTYPE_F32: return bwd_t<float>(a, g, st);
    case LASP_DTYPE_BF16: return bwd_t<bf16_tag>(a, g, st);
    case LASP_DTYPE_F16: return bwd_t<_Float16>(a, g, st);
  }
  return LASP_E_DTYPE;
}

}  // namespace lasp
