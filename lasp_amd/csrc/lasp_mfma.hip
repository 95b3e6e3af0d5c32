// bf16 MFMA kernels for d = e = 128, n % 64 == 0 (gfx950, wave64).
//
// One kernel, `la_apply`, evaluates a causal (or anti-causal) decayed linear
// attention over a segment of 64-token blocks given the state entering it:
//
//   causal       out_a = sum_{b<=a} l^(a-b) (x_a . y_b) z_b + l^a      x_a St
//                St   <- l^64 St + sum_b l^(64-b) y_b^T z_b           (blocks ascending)
//   anti-causal  out_a = sum_{b>=a} l^(b-a) (x_a . y_b) z_b + l^(64-a) x_a St
//                St   <- l^64 St + sum_b l^b      y_b^T z_b           (blocks descending)
//
// (a, b: token index inside the block; St is 128 x 128, rows = features of y,
// columns = features of z.)  The four outputs of the operator are instances:
//   O  : x=Q  y=K  z=V   causal       St = KV            lasp/lasp_fuse.py:104-124
//   dQ : x=dO y=V  z=K   causal       St = KV^T          lasp/lasp_fuse.py:237-260
//   dV : x=K  y=Q  z=dO  anti-causal  St = DKV           lasp/lasp_fuse.py:340-350
//   dK : x=V  y=dO z=Q   anti-causal  St = DKV^T         lasp/lasp_fuse.py:333-350
// `la_seg_state` computes a segment's own contribution to St (the pre-pass whose
// results the decayed scan stitches together).
//
// Work split inside a 256-thread workgroup (4 waves): wave w owns columns
// [32w, 32w+32) of St and of the output, as four 32x32 fp32 MFMA accumulator
// tiles that never leave registers; the 64x64 score tile is computed once,
// cooperatively (one 32x32 quadrant per wave), masked, rounded to bf16 and shared
// through LDS.  All products are arranged so that an accumulator tile can be fed
// back as an MFMA operand without a shuffle: v_mfma_f32_32x32x16_bf16 leaves
// C[8g+4hh+r][c] in register 4g+r of lane (c, hh) -- four consecutive rows per
// lane -- and the contraction index of the following product is permuted to
// match on both operands.
#include "lasp_common.h"

namespace lasp {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));

constexpr int F = 128;      // feature size (d = e)
constexpr int BLK = 64;     // tokens per block
constexpr int NTHR = 256;
constexpr int LDN = 272;    // bytes per row of a token-major tile (256 + 16: rows shift 4 banks)
constexpr int LDT = 128;    // bytes per row of a feature-major tile (64 tokens), XOR-swizzled
constexpr int LDSC = 144;   // bytes per row of the score tile (128 + 16)
constexpr int OFF_XN = 0;
constexpr int OFF_YN = OFF_XN + BLK * LDN;
constexpr int OFF_YT = OFF_YN + BLK * LDN;
constexpr int OFF_ZT = OFF_YT + F * LDT;
constexpr int OFF_SC = OFF_ZT + F * LDT;
constexpr int APPLY_LDS = OFF_SC + BLK * LDSC;  // 76800 B: two workgroups per CU
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  float2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

union Frag {
  bf16x8 v;
  uint4 q;
  uint2 h[2];
  uint32_t w[4];
};

__device__ __forceinline__ bf16x8 lds16(const char *p) { return *reinterpret_cast<const bf16x8 *>(p); }

// element x (0..7) of a 16-byte group of bf16, widened to fp32
__device__ __forceinline__ float bf_elem(const uint4 &q, int x) {
  const uint32_t w = (x >> 1) == 0 ? q.x : (x >> 1) == 1 ? q.y : (x >> 1) == 2 ? q.z : q.w;
  return __uint_as_float((x & 1) ? (w & 0xffff0000u) : (w << 16));
}
__device__ __forceinline__ uint32_t bf_bits(const uint4 &q, int x) {
  const uint32_t w = (x >> 1) == 0 ? q.x : (x >> 1) == 1 ? q.y : (x >> 1) == 2 ? q.z : q.w;
  return (x & 1) ? (w >> 16) : (w & 0xffffu);
}

// byte offset of 16-byte granule g16 (8 tokens) of feature row f in a feature-major tile
__device__ __forceinline__ int tr_off(int f, int g16) {
  return f * LDT + (((g16 ^ f ^ (f >> 3)) & 7) << 4);
}

// l^x for x >= 0
__device__ __forceinline__ float decay(float s_log2e, float x) {
  return __builtin_amdgcn_exp2f(-s_log2e * x);
}

// Writes four rows (tokens 4*rowgrp .. +3) x eight features (8*dchunk .. +7) into a
// feature-major tile: eight 8-byte stores, one per feature, each holding the four
// tokens; `w[r]` scales token r before rounding (SCALE), else bits are moved as is.
template <bool SCALE>
__device__ __forceinline__ void store_transposed(char *tile, const uint4 (&rows)[4], int dchunk,
                                                 int rowgrp, const float (&w)[4]) {
#pragma unroll
  for (int x = 0; x < 8; ++x) {
    const int f = 8 * dchunk + x;
    uint2 out;
    if (SCALE) {
      out.x = pack_bf16(bf_elem(rows[0], x) * w[0], bf_elem(rows[1], x) * w[1]);
      out.y = pack_bf16(bf_elem(rows[2], x) * w[2], bf_elem(rows[3], x) * w[3]);
    } else {
      out.x = bf_bits(rows[0], x) | (bf_bits(rows[1], x) << 16);
      out.y = bf_bits(rows[2], x) | (bf_bits(rows[3], x) << 16);
    }
    *reinterpret_cast<uint2 *>(tile + tr_off(f, rowgrp >> 1) + ((rowgrp & 1) << 3)) = out;
  }
}

struct SegWork {
  int bh, seg;
  int64_t tok0;  // first token of the segment
  int nblk;      // 64-token blocks in it
};
__device__ __forceinline__ SegWork seg_work(const Geom &g) {
  SegWork r;
  r.bh = blockIdx.x / g.n_seg;
  r.seg = blockIdx.x - r.bh * g.n_seg;
  r.tok0 = (int64_t)r.seg * g.seg_len;
  int64_t t1 = r.tok0 + g.seg_len;
  if (t1 > g.n) t1 = g.n;
  r.nblk = (int)((t1 - r.tok0) / BLK);
  return r;
}

// ------------------------------------------------------------------------------
template <bool REV, bool TRANS>
__global__ void __launch_bounds__(NTHR, 2)
la_apply(const bf16_t *__restrict__ X, const bf16_t *__restrict__ Y, const bf16_t *__restrict__ Z,
         const float *__restrict__ S, const float *__restrict__ states, bf16_t *__restrict__ Out,
         Geom g) {
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, w = tid >> 6;
  const int c = lane & 31, hh = lane >> 5;
  const int chunk = tid & 15, rowq = tid >> 4;  // loader roles: 16-byte column, row / row group

  const SegWork sw = seg_work(g);
  const float sl = S[sw.bh % g.h] * LOG2E;
  const int64_t base = ((int64_t)sw.bh * g.n + sw.tok0) * F;
  const uint4 *Xg = reinterpret_cast<const uint4 *>(X + base);
  const uint4 *Yg = reinterpret_cast<const uint4 *>(Y + base);
  const uint4 *Zg = reinterpret_cast<const uint4 *>(Z + base);
  uint4 *Og = reinterpret_cast<uint4 *>(Out + base);

  // ---- constants (all exponents <= 0)
  const float blockdec = decay(sl, (float)BLK);
  float qdec[2];
#pragma unroll
  for (int I = 0; I < 2; ++I) {
    const int a = 32 * I + c;
    qdec[I] = decay(sl, REV ? (float)(BLK - a) : (float)a);
  }
  float kdec[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int b = 4 * rowq + r;
    kdec[r] = decay(sl, REV ? (float)b : (float)(BLK - b));
  }
  const int qI = w >> 1, qJ = w & 1;  // score quadrant of this wave: queries 32*qI.., keys 32*qJ..
  const bool q_active = REV ? !(qI == 1 && qJ == 0) : !(qI == 0 && qJ == 1);

  // ---- state entering the segment, as accumulator tiles: st[T][4g+r] = St[32T+8g+4hh+r][32w+c]
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

  // ---- block loader: registers <- global, LDS <- registers
  uint4 nx[4], ny[4], nz[4];
  auto issue_loads = [&](int blk) {
    const int64_t off = (int64_t)blk * (BLK * F / 8);  // in 16-byte units
#pragma unroll
    for (int it = 0; it < 4; ++it) nx[it] = Xg[off + (rowq + 16 * it) * 16 + chunk];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      ny[r] = Yg[off + (4 * rowq + r) * 16 + chunk];
      nz[r] = Zg[off + (4 * rowq + r) * 16 + chunk];
    }
  };
  auto fill_lds = [&]() {
#pragma unroll
    for (int it = 0; it < 4; ++it)
      *reinterpret_cast<uint4 *>(smem + OFF_XN + (rowq + 16 * it) * LDN + chunk * 16) = nx[it];
#pragma unroll
    for (int r = 0; r < 4; ++r)
      *reinterpret_cast<uint4 *>(smem + OFF_YN + (4 * rowq + r) * LDN + chunk * 16) = ny[r];
    store_transposed<true>(smem + OFF_YT, ny, chunk, rowq, kdec);
    store_transposed<false>(smem + OFF_ZT, nz, chunk, rowq, kdec);
  };

  const int first = REV ? sw.nblk - 1 : 0;
  const int step = REV ? -1 : 1;
  issue_loads(first);
  fill_lds();
  __syncthreads();

  for (int it = 0, blk = first; it < sw.nblk; ++it, blk += step) {
    const bool more = it + 1 < sw.nblk;
    if (more) issue_loads(blk + step);

    // (1) score quadrant, transposed: sc[4g+r] = y_b . x_a, b = 32qJ+8g+4hh+r, a = 32qI+c
    if (q_active) {
      floatx16 sc;
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[r] = 0.f;
      const char *ya = smem + OFF_YN + (32 * qJ + c) * LDN + hh * 16;
      const char *xb = smem + OFF_XN + (32 * qI + c) * LDN + hh * 16;
#pragma unroll
      for (int u = 0; u < 8; ++u)
        sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds16(ya + u * 32), lds16(xb + u * 32), sc, 0, 0, 0);
      const int a = 32 * qI + c;
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        float m[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int b = 32 * qJ + 8 * gq + 4 * hh + r;
          const int dist = REV ? b - a : a - b;
          m[r] = dist >= 0 ? sc[4 * gq + r] * decay(sl, (float)dist) : 0.f;
        }
        uint2 o;
        o.x = pack_bf16(m[0], m[1]);
        o.y = pack_bf16(m[2], m[3]);
        *reinterpret_cast<uint2 *>(smem + OFF_SC + a * LDSC + (32 * qJ + 8 * gq + 4 * hh) * 2) = o;
      }
    }

    // (2) state term, transposed: acc[I][4g+r] = sum_f St[f][32w+8g+4hh+r] x_a[f], a = 32I+c
    floatx16 acc[2];
#pragma unroll
    for (int I = 0; I < 2; ++I)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[I][r] = 0.f;
#pragma unroll
    for (int T = 0; T < 4; ++T)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        Frag a;
#pragma unroll
        for (int p = 0; p < 4; ++p) a.w[p] = pack_bf16(st[T][8 * u + 2 * p], st[T][8 * u + 2 * p + 1]);
#pragma unroll
        for (int I = 0; I < 2; ++I) {
          const char *xp = smem + OFF_XN + (32 * I + c) * LDN + (32 * T + 16 * u + 4 * hh) * 2;
          Frag b;
          b.h[0] = *reinterpret_cast<const uint2 *>(xp);
          b.h[1] = *reinterpret_cast<const uint2 *>(xp + 16);
          acc[I] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, acc[I], 0, 0, 0);
        }
      }
#pragma unroll
    for (int I = 0; I < 2; ++I)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[I][r] *= qdec[I];

    __syncthreads();  // A: score tile complete; XN / YN no longer read

    // (3) intra-block term: acc[I] += Z^T[32w.., tokens] * score[a][tokens]
    bf16x8 zf[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) zf[u] = lds16(smem + OFF_ZT + tr_off(32 * w + c, 2 * u + hh));
#pragma unroll
    for (int I = 0; I < 2; ++I)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const bool needed = REV ? (I == 0 || u >= 2) : (I == 1 || u < 2);
        if (needed) {
          const bf16x8 b = lds16(smem + OFF_SC + (32 * I + c) * LDSC + (16 * u + 8 * hh) * 2);
          acc[I] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(zf[u], b, acc[I], 0, 0, 0);
        }
      }

    // (4) state update: St <- l^64 St + (scaled Y)^T Z
#pragma unroll
    for (int T = 0; T < 4; ++T) {
#pragma unroll
      for (int r = 0; r < 16; ++r) st[T][r] *= blockdec;
#pragma unroll
      for (int u = 0; u < 4; ++u)
        st[T] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            lds16(smem + OFF_YT + tr_off(32 * T + c, 2 * u + hh)), zf[u], st[T], 0, 0, 0);
    }

    // (5) stage the output tile (token-major, in the YN region) for coalesced stores
#pragma unroll
    for (int I = 0; I < 2; ++I)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        uint2 o;
        o.x = pack_bf16(acc[I][4 * gq + 0], acc[I][4 * gq + 1]);
        o.y = pack_bf16(acc[I][4 * gq + 2], acc[I][4 * gq + 3]);
        *reinterpret_cast<uint2 *>(smem + OFF_YN + (32 * I + c) * LDN + (32 * w + 8 * gq + 4 * hh) * 2) = o;
      }
    __syncthreads();  // B: staged output complete; YT / ZT / score no longer read
    {
      const int64_t off = (int64_t)blk * (BLK * F / 8);
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int row = rowq + 16 * r4;
        Og[off + row * 16 + chunk] = *reinterpret_cast<const uint4 *>(smem + OFF_YN + row * LDN + chunk * 16);
      }
    }
    if (more) {
      __syncthreads();  // C: staged output consumed
      fill_lds();
      __syncthreads();  // D: next block visible
    }
  }
}

// ------------------------------------------------------------------------------
// A segment's own state:  causal  sum_b l^(L-b) y_b^T z_b ;  anti-causal  sum_b l^b y_b^T z_b
// (b from the segment start, L its length), written token-free as 128 x 128 fp32.
template <bool REV>
__global__ void __launch_bounds__(NTHR, 2)
la_seg_state(const bf16_t *__restrict__ Y, const bf16_t *__restrict__ Z, const float *__restrict__ S,
             float *__restrict__ states, Geom g) {
  __shared__ __align__(16) char smem[2][2 * F * LDT];  // double-buffered {Y^T scaled, Z^T}
  const int tid = threadIdx.x;
  const int lane = tid & 63, w = tid >> 6;
  const int c = lane & 31, hh = lane >> 5;
  const int chunk = tid & 15, rowq = tid >> 4;

  const SegWork sw = seg_work(g);
  const float sl = S[sw.bh % g.h] * LOG2E;
  const int64_t base = ((int64_t)sw.bh * g.n + sw.tok0) * F;
  const uint4 *Yg = reinterpret_cast<const uint4 *>(Y + base);
  const uint4 *Zg = reinterpret_cast<const uint4 *>(Z + base);

  const float blockdec = decay(sl, (float)BLK);
  float kdec[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int b = 4 * rowq + r;
    kdec[r] = decay(sl, REV ? (float)b : (float)(BLK - b));
  }

  floatx16 st[4];
#pragma unroll
  for (int T = 0; T < 4; ++T)
#pragma unroll
    for (int r = 0; r < 16; ++r) st[T][r] = 0.f;

  uint4 ny[4], nz[4];
  auto issue_loads = [&](int blk) {
    const int64_t off = (int64_t)blk * (BLK * F / 8);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      ny[r] = Yg[off + (4 * rowq + r) * 16 + chunk];
      nz[r] = Zg[off + (4 * rowq + r) * 16 + chunk];
    }
  };
  auto fill_lds = [&](int buf) {
    store_transposed<true>(smem[buf], ny, chunk, rowq, kdec);
    store_transposed<false>(smem[buf] + F * LDT, nz, chunk, rowq, kdec);
  };

  const int first = REV ? sw.nblk - 1 : 0;
  const int step = REV ? -1 : 1;
  issue_loads(first);
  fill_lds(0);
  __syncthreads();
  for (int it = 0, blk = first; it < sw.nblk; ++it, blk += step) {
    const bool more = it + 1 < sw.nblk;
    if (more) issue_loads(blk + step);
    const char *yt = smem[it & 1];
    const char *zt = yt + F * LDT;
    bf16x8 zf[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) zf[u] = lds16(zt + tr_off(32 * w + c, 2 * u + hh));
#pragma unroll
    for (int T = 0; T < 4; ++T) {
#pragma unroll
      for (int r = 0; r < 16; ++r) st[T][r] *= blockdec;
#pragma unroll
      for (int u = 0; u < 4; ++u)
        st[T] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds16(yt + tr_off(32 * T + c, 2 * u + hh)), zf[u],
                                                        st[T], 0, 0, 0);
    }
    if (more) fill_lds((it + 1) & 1);
    __syncthreads();
  }

  float *sp = states + ((int64_t)sw.bh * g.n_seg + sw.seg) * (F * F);
#pragma unroll
  for (int T = 0; T < 4; ++T)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      sp[(32 * T + 8 * (r >> 2) + 4 * hh + (r & 3)) * F + 32 * w + c] = st[T][r];
}

template <class K>
int raise_lds(K kernel) {
  return (int)hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  APPLY_LDS);
}

template <bool REV, bool TRANS>
int launch_apply(const void *x, const void *y, const void *z, const float *s, const float *states,
                 void *out, const Geom &g, hipStream_t st) {
  int rc = raise_lds(la_apply<REV, TRANS>);
  if (rc) return rc;
  const unsigned grid = (unsigned)((int64_t)g.b * g.h * g.n_seg);
  ProfScope prof(KC_APPLY, st);
  la_apply<REV, TRANS><<<grid, NTHR, APPLY_LDS, st>>>((const bf16_t *)x, (const bf16_t *)y,
                                                      (const bf16_t *)z, s, states, (bf16_t *)out, g);
  return (int)hipGetLastError();
}

template <bool REV>
int launch_state(const void *y, const void *z, const float *s, float *states, const Geom &g,
                 hipStream_t st) {
  const unsigned grid = (unsigned)((int64_t)g.b * g.h * g.n_seg);
  ProfScope prof(KC_STATE, st);
  la_seg_state<REV><<<grid, NTHR, 0, st>>>((const bf16_t *)y, (const bf16_t *)z, s, states, g);
  return (int)hipGetLastError();
}

}  // namespace

int mfma_fwd(const FwdArgs &a, const Geom &g, hipStream_t st) {
  int rc;
  const bool need_states = g.n_seg > 1 || a.kv_in || a.kv_out;
  if (need_states) {
    if ((rc = launch_state<false>(a.k, a.v, a.s, a.seg_states, g, st))) return rc;
    if ((rc = launch_segment_scan(a.seg_states, a.kv_in, a.kv_out, a.s, g, 0, st))) return rc;
  }
  return launch_apply<false, false>(a.q, a.k, a.v, a.s, need_states ? a.seg_states : nullptr, a.o, g, st);
}

int mfma_bwd(const BwdArgs &a, const Geom &g, hipStream_t st) {
  int rc;
  const float *kv_states = a.kv_seg_states;
  if (!kv_states && (g.n_seg > 1 || a.kv_in)) {
    if ((rc = launch_state<false>(a.k, a.v, a.s, a.ws_kv, g, st))) return rc;
    if ((rc = launch_segment_scan(a.ws_kv, a.kv_in, nullptr, a.s, g, 0, st))) return rc;
    kv_states = a.ws_kv;
  }
  const float *dkv_states = nullptr;
  if (g.n_seg > 1 || a.dkv_in || a.dkv_out) {
    if ((rc = launch_state<true>(a.q, a.d_o, a.s, a.ws_dkv, g, st))) return rc;
    if ((rc = launch_segment_scan(a.ws_dkv, a.dkv_in, a.dkv_out, a.s, g, 1, st))) return rc;
    dkv_states = a.ws_dkv;
  }
  if ((rc = launch_apply<false, true>(a.d_o, a.v, a.k, a.s, kv_states, a.dq, g, st))) return rc;
  if ((rc = launch_apply<true, false>(a.k, a.q, a.d_o, a.s, dkv_states, a.dv, g, st))) return rc;
  return launch_apply<true, true>(a.v, a.d_o, a.q, a.s, dkv_states, a.dk, g, st);
}

}  // namespace lasp
