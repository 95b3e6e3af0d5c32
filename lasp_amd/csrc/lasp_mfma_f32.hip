// fp32 MFMA kernels for d = e = 128 (gfx950, wave64): the same decomposition
// as the 16-bit kernels -- one routine evaluates a causal or anti-causal decayed linear
// attention over a segment given the state entering it, and the four outputs of the
// operator are instances of it (O: x=Q y=K z=V; dQ: x=dO y=V z=K with the state transposed;
// dV: x=K y=Q z=dO anti-causal; dK: x=V y=dO z=Q anti-causal, state transposed) -- but with
// full-precision arithmetic throughout (v_mfma_f32_32x32x2_f32), for inputs whose tolerance
// (1e-3) rules out 16-bit operands.
//
// v_mfma_f32_32x32x2_f32 contracts over two indices per instruction, one per lane half:
// lane (c, hh) supplies A[c][k_hh] and B[k_hh][c], and leaves C[8g+4hh+r][c] in register
// 4g+r.  Choosing (k_0, k_1) = (8g+r, 8g+4+r) makes register 4g+r of an accumulator tile
// exactly the operand element the next product needs, so
//   * the state tiles feed the state-term product straight from registers,
//   * the masked 32x32 score tile feeds the intra-block product straight from registers
//     (every wave computes the whole tile: no LDS round trip, no rounding),
// and the LDS only holds the block's inputs: X and Y token-major, (w (.) Y)^T and Z^T
// feature-major (XOR-swizzled 16-byte granules).  Blocks are 32 tokens.
#include "lasp_common.h"

namespace lasp {
namespace {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int F = 128;
constexpr int BLK = 32;
constexpr int NTHR = 256;
constexpr int LDN = 528;   // bytes per token-major row (512 + 16: consecutive rows shift 4 banks)
constexpr int LDT = 128;   // bytes per feature-major row (32 tokens)
constexpr int OFF_XN = 0;
constexpr int OFF_YN = OFF_XN + BLK * LDN;
constexpr int OFF_YT = OFF_YN + BLK * LDN;
constexpr int OFF_ZT = OFF_YT + F * LDT;
constexpr int APPLY_LDS = OFF_ZT + F * LDT;  // 66560 B: two workgroups per CU
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ float decay(float s_log2e, float x) {
  return __builtin_amdgcn_exp2f(-s_log2e * x);
}
__device__ __forceinline__ f32x4 lds16(const char *p) { return *reinterpret_cast<const f32x4 *>(p); }
__device__ __forceinline__ floatx16 mfma(float a, float b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// byte offset of 16-byte granule g16 (4 tokens) of feature row f.  The XOR term is a bijection
// both of f bits 0-2 (rows read by 8 consecutive lanes) and of f bits 2-4 (rows written by 8
// consecutive loader lanes), so 16-byte reads and writes are bank-conflict free.
__device__ __forceinline__ int tr_off(int f, int g16) {
  const int sw = ((f & 3) ^ ((f >> 3) & 3)) | (f & 4);
  return f * LDT + (((g16 ^ sw) & 7) << 4);
}

struct SegWork {
  int bh, seg;
  int64_t tok0;
  int nblk;  // 32-token blocks, the last one possibly partial
  int tail;  // tokens in the last block (1..32); below 32 only at the end of a ragged chunk
};
__device__ __forceinline__ SegWork seg_work(const Geom &g, int item) {
  SegWork r;
  r.bh = item / g.n_seg;
  r.seg = item - r.bh * g.n_seg;
  r.tok0 = (int64_t)r.seg * g.seg_len;
  int64_t t1 = r.tok0 + g.seg_len;
  if (t1 > g.n) t1 = g.n;
  const int tokens = (int)(t1 - r.tok0);
  r.nblk = (tokens + BLK - 1) / BLK;
  r.tail = tokens - (r.nblk - 1) * BLK;
  return r;
}

// four rows (tokens 4*rq .. +3) x four features (4*cq .. +3), written feature-major:
// one 16-byte store per feature, holding the four tokens scaled by w[r]
__device__ __forceinline__ void store_transposed(char *tile, const f32x4 (&rows)[4], int cq, int rq,
                                                 const float (&w)[4]) {
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    f32x4 out;
    out.x = rows[0][x] * w[0];
    out.y = rows[1][x] * w[1];
    out.z = rows[2][x] * w[2];
    out.w = rows[3][x] * w[3];
    *reinterpret_cast<f32x4 *>(tile + tr_off(4 * cq + x, rq)) = out;
  }
}

// RAGGED: the chunk length is not a multiple of 32, so the last block of the last segment is
// partial (missing rows read as zeros, stores masked, and -- going backwards, where that block
// comes first -- the entering state sits `len` tokens ahead instead of 32).
template <bool REV, bool TRANS, bool RAGGED>
__device__ __forceinline__ void
apply_body(const float *__restrict__ X, const float *__restrict__ Y, const float *__restrict__ Z,
           const float *__restrict__ S, const float *__restrict__ states, float *__restrict__ Out,
           const Geom &g, int item, char *smem) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave index, uniform: keeps it in an SGPR
  const int c = lane & 31, hh = lane >> 5;
  const int cq = tid & 31, rq = tid >> 5;  // loader: 16-byte column, row (X) / group of four rows (Y, Z)

  const SegWork sw = seg_work(g, item);
  const float sl = S[sw.bh % g.h] * LOG2E;
  const int64_t base = ((int64_t)sw.bh * g.n + sw.tok0) * F;
  const f32x4 *Xg = reinterpret_cast<const f32x4 *>(X + base);
  const f32x4 *Yg = reinterpret_cast<const f32x4 *>(Y + base);
  const f32x4 *Zg = reinterpret_cast<const f32x4 *>(Z + base);
  float *Og = Out + base;

  // ---- constants (all exponents <= 0)
  const float blockdec = decay(sl, (float)BLK);
  const float qdec = decay(sl, REV ? (float)(BLK - c) : (float)c);
  float kdec[4], ones[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int b = 4 * rq + r;
    kdec[r] = decay(sl, REV ? (float)b : (float)(BLK - b));
    ones[r] = 1.f;
  }

  // ---- state entering the segment: st[T][4g+r] = St[32T+8g+4hh+r][32w+c]
  floatx16 st[4];
  if (states) {
    const float *sp = states + ((int64_t)sw.bh * g.n_seg + sw.seg) * (F * F);
#pragma unroll
    for (int T = 0; T < 4; ++T)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 32 * T + 8 * (r >> 2) + 4 * hh + (r & 3);
        const int col = 32 * w + c;
        st[T][r] = TRANS ? sp[col * F + row] : sp[row * F + col];
      }
  } else {
#pragma unroll
    for (int T = 0; T < 4; ++T)
#pragma unroll
      for (int r = 0; r < 16; ++r) st[T][r] = 0.f;
  }

  f32x4 nx[4], ny[4], nz[4];
  auto issue_loads = [&](int blk) __attribute__((always_inline)) {
    const int64_t off = (int64_t)blk * (BLK * F / 4);  // 16-byte units, 32 per row
    const int len = RAGGED && blk == sw.nblk - 1 ? sw.tail : BLK;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int row = rq + 8 * it;
      nx[it] = (!RAGGED || row < len) ? Xg[off + row * 32 + cq] : zero;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = 4 * rq + r;
      ny[r] = (!RAGGED || row < len) ? Yg[off + row * 32 + cq] : zero;
      nz[r] = (!RAGGED || row < len) ? Zg[off + row * 32 + cq] : zero;
    }
  };
  auto fill_lds = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int it = 0; it < 4; ++it)
      *reinterpret_cast<f32x4 *>(smem + OFF_XN + (rq + 8 * it) * LDN + cq * 16) = nx[it];
#pragma unroll
    for (int r = 0; r < 4; ++r)
      *reinterpret_cast<f32x4 *>(smem + OFF_YN + (4 * rq + r) * LDN + cq * 16) = ny[r];
    store_transposed(smem + OFF_YT, ny, cq, rq, kdec);
    store_transposed(smem + OFF_ZT, nz, cq, rq, ones);
  };

  const int first = REV ? sw.nblk - 1 : 0;
  const int step = REV ? -1 : 1;
  issue_loads(first);
  fill_lds();
  __syncthreads();

  for (int it = 0, blk = first; it < sw.nblk; ++it, blk += step) {
    const bool more = it + 1 < sw.nblk;
    if (more) issue_loads(blk + step);
    const int len = RAGGED && blk == sw.nblk - 1 ? sw.tail : BLK;
    float qd = qdec, bd = blockdec;
    if (RAGGED && REV && len != BLK) {
      qd = decay(sl, (float)max(len - c, 0));
      bd = decay(sl, (float)len);
    }

    // (1) sweep over the features: state term and score tile from the same X elements
    //     acc[4g+r] = sum_f St[f][32w+8g+4hh+r] x_a[f]      (a = c)
    //     sc[4g+r]  = y_b . x_a,  b = 8g+4hh+r
    floatx16 acc, sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[r] = 0.f;
      sc[r] = 0.f;
    }
    {
      const char *xp = smem + OFF_XN + c * LDN + hh * 16;
      const char *yp = smem + OFF_YN + c * LDN + hh * 16;
#pragma unroll
      for (int m = 0; m < 16; ++m) {  // features 8m + 4hh + {0..3}
        const f32x4 xf = lds16(xp + m * 32);
        const f32x4 yf = lds16(yp + m * 32);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          acc = mfma(st[m >> 2][4 * (m & 3) + r], xf[r], acc);
          sc = mfma(yf[r], xf[r], sc);
        }
      }
    }
    // (2) mask the scores, scale the state term
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int b = 8 * (r >> 2) + 4 * hh + (r & 3);
      const int dist = REV ? b - c : c - b;
      sc[r] = dist >= 0 ? sc[r] * decay(sl, (float)dist) : 0.f;
      acc[r] *= qd;
    }
    // (3) intra-block term and (4) state update share the Z^T elements
    f32x4 zf[4];
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) zf[gq] = lds16(smem + OFF_ZT + tr_off(32 * w + c, 2 * gq + hh));
#pragma unroll
    for (int gq = 0; gq < 4; ++gq)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc = mfma(zf[gq][r], sc[4 * gq + r], acc);
#pragma unroll
    for (int T = 0; T < 4; ++T) {
#pragma unroll
      for (int r = 0; r < 16; ++r) st[T][r] *= bd;
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const f32x4 yt = lds16(smem + OFF_YT + tr_off(32 * T + c, 2 * gq + hh));
#pragma unroll
        for (int r = 0; r < 4; ++r) st[T] = mfma(yt[r], zf[gq][r], st[T]);
      }
    }
    // (5) output: lane (c, hh) holds, for token c, four consecutive columns per g
    if (!RAGGED || c < len) {
      float *orow = Og + ((int64_t)blk * BLK + c) * F + 32 * w + 4 * hh;
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        f32x4 o;
        o.x = acc[4 * gq + 0];
        o.y = acc[4 * gq + 1];
        o.z = acc[4 * gq + 2];
        o.w = acc[4 * gq + 3];
        *reinterpret_cast<f32x4 *>(orow + 8 * gq) = o;
      }
    }
    if (more) {
      __syncthreads();  // every wave is done reading this block's tiles
      fill_lds();
      __syncthreads();  // next block visible
    }
  }
}

template <bool REV, bool TRANS, bool RAGGED>
__global__ void __launch_bounds__(NTHR, 2)
la32_apply(const float *__restrict__ X, const float *__restrict__ Y, const float *__restrict__ Z,
           const float *__restrict__ S, const float *__restrict__ states, float *__restrict__ Out, Geom g) {
  extern __shared__ __align__(16) char smem[];
  apply_body<REV, TRANS, RAGGED>(X, Y, Z, S, states, Out, g, (int)blockIdx.x, smem);
}

// dQ, dV and dK in one launch; the three workgroups of a (b*h, segment) sit 8 block indices
// apart, i.e. on the same XCD
template <bool RAGGED>
__global__ void __launch_bounds__(NTHR, 2)
la32_bwd3(const float *__restrict__ Q, const float *__restrict__ K, const float *__restrict__ V,
          const float *__restrict__ DO, const float *__restrict__ S, const float *__restrict__ kv_states,
          const float *__restrict__ dkv_states, float *__restrict__ DQ, float *__restrict__ DK,
          float *__restrict__ DV, Geom g) {
  extern __shared__ __align__(16) char smem[];
  const int n_items = g.b * g.h * g.n_seg;
  const int grp = blockIdx.x / 24, r = blockIdx.x - grp * 24;
  const int role = r >> 3;
  const int item = n_items - 1 - (grp * 8 + (r & 7));
  if (item < 0) return;
  if (role == 0)
    apply_body<false, true, RAGGED>(DO, V, K, S, kv_states, DQ, g, item, smem);
  else if (role == 1)
    apply_body<true, false, RAGGED>(K, Q, DO, S, dkv_states, DV, g, item, smem);
  else
    apply_body<true, true, RAGGED>(V, DO, Q, S, dkv_states, DK, g, item, smem);
}

// a segment's own state: causal sum_b l^(L-b) y_b^T z_b ; anti-causal sum_b l^b y_b^T z_b
template <bool REV, bool RAGGED>
__global__ void __launch_bounds__(NTHR, 2)
la32_seg_state(const float *__restrict__ Y, const float *__restrict__ Z, const float *__restrict__ S,
               float *__restrict__ states, Geom g, int skip_seg) {
  __shared__ __align__(16) char smem[2][2 * F * LDT];  // double-buffered {(w (.) Y)^T, Z^T}
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave index, uniform: keeps it in an SGPR
  const int c = lane & 31, hh = lane >> 5;
  const int cq = tid & 31, rq = tid >> 5;

  const SegWork sw = seg_work(g, (int)blockIdx.x);
  if (sw.seg == skip_seg) return;
  const float sl = S[sw.bh % g.h] * LOG2E;
  const int64_t base = ((int64_t)sw.bh * g.n + sw.tok0) * F;
  const f32x4 *Yg = reinterpret_cast<const f32x4 *>(Y + base);
  const f32x4 *Zg = reinterpret_cast<const f32x4 *>(Z + base);

  const float blockdec = decay(sl, (float)BLK);
  float kdec[4], ones[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int b = 4 * rq + r;
    kdec[r] = decay(sl, REV ? (float)b : (float)(BLK - b));
    ones[r] = 1.f;
  }
  floatx16 st[4];
#pragma unroll
  for (int T = 0; T < 4; ++T)
#pragma unroll
    for (int r = 0; r < 16; ++r) st[T][r] = 0.f;

  f32x4 ny[4], nz[4];
  auto issue_loads = [&](int blk) __attribute__((always_inline)) {
    const int64_t off = (int64_t)blk * (BLK * F / 4);
    const int len = RAGGED && blk == sw.nblk - 1 ? sw.tail : BLK;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = 4 * rq + r;
      ny[r] = (!RAGGED || row < len) ? Yg[off + row * 32 + cq] : zero;
      nz[r] = (!RAGGED || row < len) ? Zg[off + row * 32 + cq] : zero;
    }
  };
  // going forwards a partial block is the last one: its tokens sit `len - b` before the segment end
  auto fill_lds = [&](int buf, int blk) __attribute__((always_inline)) {
    const int len = RAGGED && blk == sw.nblk - 1 ? sw.tail : BLK;
    if (RAGGED && !REV && len != BLK) {
      float kd[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) kd[r] = decay(sl, (float)max(len - (4 * rq + r), 0));
      store_transposed(smem[buf], ny, cq, rq, kd);
    } else {
      store_transposed(smem[buf], ny, cq, rq, kdec);
    }
    store_transposed(smem[buf] + F * LDT, nz, cq, rq, ones);
  };

  const int first = REV ? sw.nblk - 1 : 0;
  const int step = REV ? -1 : 1;
  issue_loads(first);
  fill_lds(0, first);
  __syncthreads();
  for (int it = 0, blk = first; it < sw.nblk; ++it, blk += step) {
    const bool more = it + 1 < sw.nblk;
    if (more) issue_loads(blk + step);
    const int len = RAGGED && blk == sw.nblk - 1 ? sw.tail : BLK;
    const float bd = RAGGED && len != BLK ? decay(sl, (float)len) : blockdec;
    const char *ytile = smem[it & 1];
    const char *ztile = ytile + F * LDT;
    f32x4 zf[4];
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) zf[gq] = lds16(ztile + tr_off(32 * w + c, 2 * gq + hh));
#pragma unroll
    for (int T = 0; T < 4; ++T) {
#pragma unroll
      for (int r = 0; r < 16; ++r) st[T][r] *= bd;
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const f32x4 yt = lds16(ytile + tr_off(32 * T + c, 2 * gq + hh));
#pragma unroll
        for (int r = 0; r < 4; ++r) st[T] = mfma(yt[r], zf[gq][r], st[T]);
      }
    }
    if (more) fill_lds((it + 1) & 1, blk + step);
    __syncthreads();
  }
  float *sp = states + ((int64_t)sw.bh * g.n_seg + sw.seg) * (F * F);
#pragma unroll
  for (int T = 0; T < 4; ++T)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      sp[(32 * T + 8 * (r >> 2) + 4 * hh + (r & 3)) * F + 32 * w + c] = st[T][r];
}

template <bool REV, bool RAGGED>
int launch_state(const void *y, const void *z, const float *s, float *states, const Geom &g,
                 bool carry_wanted, hipStream_t st) {
  const unsigned grid = (unsigned)((int64_t)g.b * g.h * g.n_seg);
  const int skip_seg = carry_wanted ? -1 : (REV ? 0 : g.n_seg - 1);
  ProfScope prof(KC_STATE, st);
  la32_seg_state<REV, RAGGED><<<grid, NTHR, 0, st>>>((const float *)y, (const float *)z, s, states, g,
                                                     skip_seg);
  return (int)hipGetLastError();
}

template <bool RAGGED>
int fwd_r(const FwdArgs &a, const Geom &g, hipStream_t st) {
  int rc;
  const bool need_states = g.n_seg > 1 || a.kv_in || a.kv_out;
  if (need_states) {
    if ((rc = launch_state<false, RAGGED>(a.k, a.v, a.s, a.seg_states, g, a.kv_out != nullptr, st))) return rc;
    if ((rc = launch_segment_scan(a.seg_states, a.kv_in, a.kv_out, a.s, g, 0, st))) return rc;
  }
  if ((rc = grant_lds<la32_apply<false, false, RAGGED>>(APPLY_LDS))) return rc;
  const unsigned grid = (unsigned)((int64_t)g.b * g.h * g.n_seg);
  ProfScope prof(KC_APPLY, st);
  la32_apply<false, false, RAGGED><<<grid, NTHR, APPLY_LDS, st>>>((const float *)a.q, (const float *)a.k,
                                                                  (const float *)a.v, a.s,
                                                                  need_states ? a.seg_states : nullptr,
                                                                  (float *)a.o, g);
  return (int)hipGetLastError();
}

template <bool RAGGED>
int bwd_r(const BwdArgs &a, const Geom &g, hipStream_t st) {
  int rc;
  const float *kv_states = a.kv_seg_states;
  if (!kv_states && (g.n_seg > 1 || a.kv_in)) {
    if ((rc = launch_state<false, RAGGED>(a.k, a.v, a.s, a.ws_kv, g, false, st))) return rc;
    if ((rc = launch_segment_scan(a.ws_kv, a.kv_in, nullptr, a.s, g, 0, st))) return rc;
    kv_states = a.ws_kv;
  }
  const float *dkv_states = nullptr;
  if (g.n_seg > 1 || a.dkv_in || a.dkv_out) {
    if ((rc = launch_state<true, RAGGED>(a.q, a.d_o, a.s, a.ws_dkv, g, a.dkv_out != nullptr, st))) return rc;
    if ((rc = launch_segment_scan(a.ws_dkv, a.dkv_in, a.dkv_out, a.s, g, 1, st))) return rc;
    dkv_states = a.ws_dkv;
  }
  if ((rc = grant_lds<la32_bwd3<RAGGED>>(APPLY_LDS))) return rc;
  const int64_t n_items = (int64_t)g.b * g.h * g.n_seg;
  const unsigned grid = (unsigned)(((n_items + 7) / 8) * 24);
  ProfScope prof(KC_BWD3, st);
  la32_bwd3<RAGGED><<<grid, NTHR, APPLY_LDS, st>>>((const float *)a.q, (const float *)a.k,
                                                   (const float *)a.v, (const float *)a.d_o, a.s, kv_states,
                                                   dkv_states, (float *)a.dq, (float *)a.dk, (float *)a.dv, g);
  return (int)hipGetLastError();
}

}  // namespace

int mfma_f32_fwd(const FwdArgs &a, const Geom &g, hipStream_t st) {
  return g.n % BLK != 0 ? fwd_r<true>(a, g, st) : fwd_r<false>(a, g, st);
}

int mfma_f32_bwd(const BwdArgs &a, const Geom &g, hipStream_t st) {
  return g.n % BLK != 0 ? bwd_r<true>(a, g, st) : bwd_r<false>(a, g, st);
}

}  // namespace lasp
