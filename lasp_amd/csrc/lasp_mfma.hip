// bf16 / fp16 MFMA kernels (gfx950, wave64).  The arithmetic is laid out for d = e = 128.
// Three instantiations of every kernel: M_ALIGNED (chunk length a multiple of 64), M_RAGGED
// (one partial last block) and M_NARROW (rows of d, e < 128 features, multiples of 8, read
// zero-extended to 128 and written back at their own width; any chunk length).
//
// One device routine, `ws_body`, evaluates a causal (or anti-causal) decayed linear
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
// Work split inside a 512-thread workgroup (8 waves, one workgroup per CU): four "math"
// waves own the state and the output -- wave w columns [32w, 32w+32), as four 32x32 fp32
// MFMA accumulator tiles that never leave registers -- and four "feed" waves fetch and
// transpose the next block, compute the 64x64 score tile (one 32x32 quadrant per wave;
// masked, rounded to 16 bits and shared through LDS) and store the outputs.  All products are arranged so that an accumulator tile can be fed
// back as an MFMA operand without a shuffle: v_mfma_f32_32x32x16_bf16 leaves
// C[8g+4hh+r][c] in register 4g+r of lane (c, hh) -- four consecutive rows per
// lane -- and the contraction index of the following product is permuted to
// match on both operands.
#include "lasp_common.h"

namespace lasp {
namespace {

// native vector types (HIP's uint4 / uint2 structs copy through memcpy, which can pin
// a register array to scratch memory)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef uint16_t elem16_t;  // raw bits of one bf16 or fp16 element

constexpr int F = 128;      // feature size (d = e)
constexpr int BLK = 64;     // tokens per block
constexpr int LDN = 272;    // bytes per row of a token-major tile (256 + 16: rows shift 4 banks)
constexpr int LDT = 128;    // bytes per row of a feature-major tile (64 tokens), XOR-swizzled
constexpr int LDSC = 144;   // bytes per row of the score tile (128 + 16)
constexpr float LOG2E = kLog2e;
constexpr float SKIP_LOG2 = kSkipLog2;  // decay weights below 2^-SKIP_LOG2 are treated as zero (see la_seg_state)
enum Mode { M_ALIGNED = 0, M_RAGGED = 1, M_NARROW = 2 };
// where a sweep takes the state entering its segment from (see ws_body)
enum Source { SRC_SCANNED = 0, SRC_WALK = 1, SRC_COMBINE = 2 };

// Element policies: the kernels move 16-bit elements as raw bits and only touch their value
// in three places -- widening one element, rounding two floats into a packed pair, and the
// MFMA itself.
struct ElemBF16 {
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    float2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  }
  // `word` holds the element in its low (odd = false) or high (odd = true) half
  static __device__ __forceinline__ float widen(uint32_t word, bool odd) {
    return __uint_as_float(odd ? (word & 0xffff0000u) : (word << 16));
  }
  static __device__ __forceinline__ floatx16 mfma(u32x4 a, u32x4 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                   c, 0, 0, 0);
  }
};
struct ElemF16 {
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    float2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
  }
  static __device__ __forceinline__ float widen(uint32_t word, bool odd) {
    const f16x2_t h = __builtin_bit_cast(f16x2_t, word);
    return (float)(odd ? h.y : h.x);
  }
  static __device__ __forceinline__ floatx16 mfma(u32x4 a, u32x4 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                  0, 0, 0);
  }
};

// A pointer that is the same for every lane, moved to scalar registers: loads through it then take
// the form scalar base + 32-bit lane offset + immediate, instead of a 64-bit address per lane that
// the loop optimiser would otherwise carry (and increment) in vector registers.  The result is
// typed as a global-memory pointer, which the round trip through integers would otherwise lose.
typedef const __attribute__((address_space(1))) char *gmem_ptr;
__device__ __forceinline__ gmem_ptr uniform_ptr(const char *p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (gmem_ptr)(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ u32x4 lds16(const char *p) { return *reinterpret_cast<const u32x4 *>(p); }

// element x (0..7) of a 16-byte group of 16-bit elements, widened to fp32
template <class E>
__device__ __forceinline__ float elem_f32(const u32x4 &q, int x) {
  const uint32_t w = (x >> 1) == 0 ? q.x : (x >> 1) == 1 ? q.y : (x >> 1) == 2 ? q.z : q.w;
  return E::widen(w, x & 1);
}
__device__ __forceinline__ uint32_t elem_bits(const u32x4 &q, int x) {
  const uint32_t w = (x >> 1) == 0 ? q.x : (x >> 1) == 1 ? q.y : (x >> 1) == 2 ? q.z : q.w;
  return (x & 1) ? (w >> 16) : (w & 0xffffu);
}

// Feature order inside LDS rows and registers.  A thread never holds eight consecutive
// features: its 16 bytes are features {16G+4j .. +3} and {16G+8+4j .. +3} (G = 0..7,
// j = 0..1), fetched as two 8-byte loads.  Token-major rows store these 16-byte units at
// index 2G+j, so that lane half hh of an MFMA operand, reading unit 2k+hh, receives
// features {16k+4hh .. +3, 16k+8+4hh .. +3}: exactly the rows 8g+4hh+r (g = 2u, 2u+1)
// that the same lane holds of a 32x32 accumulator tile.  Accumulators can therefore be
// multiplied against LDS rows with single 16-byte reads, and one set of X fragments
// serves both the score product and the state product.
struct LoaderRole {
  int G, j;    // feature group and half handled by this thread
  int rowq;    // X: row within a 16-row band; Y/Z: group of four rows
};
// X tile: 16 consecutive lanes fetch one 256-byte row
__device__ __forceinline__ LoaderRole x_role(int tid) {
  LoaderRole r;
  r.G = (tid >> 1) & 7;
  r.j = tid & 1;
  r.rowq = tid >> 4;
  return r;
}
// Y / Z tiles (also stored transposed): lane bits are dealt so that any 16 consecutive
// lanes cover 8 feature units x 2 row groups -- 16 distinct 8-byte slots of the
// feature-major tile, i.e. conflict-free ds_write_b64
__device__ __forceinline__ LoaderRole yz_role(int tid) {
  LoaderRole r;
  r.j = tid & 1;
  r.G = ((tid >> 1) & 3) | (((tid >> 4) & 1) << 2);
  r.rowq = ((tid >> 3) & 1) | ((tid >> 5) << 1);
  return r;
}

// byte offset of 16-byte granule g16 (8 tokens) of feature row f in a feature-major tile.
// The XOR term varies with f bits 0-2 (consecutive rows read by consecutive lanes) and
// with bits 2,4,5 (the rows written by 16 consecutive loader lanes).
__device__ __forceinline__ int tr_off(int f, int g16) {
  return f * LDT + (((g16 ^ (f & 7) ^ ((f >> 4) & 3)) & 7) << 4);
}

// l^x for x >= 0
__device__ __forceinline__ float decay(float s_log2e, float x) {
  return __builtin_amdgcn_exp2f(-s_log2e * x);
}

// Writes four rows (tokens 4*rowq .. +3) x the thread's eight features into a
// feature-major tile: eight 8-byte stores, one per feature, each holding the four
// tokens; `w[r]` scales token r before rounding (SCALE), else bits are moved as is.
template <class E, bool SCALE>
__device__ __forceinline__ void store_transposed(char *tile, const u32x4 (&rows)[4],
                                                 const LoaderRole &role, const float (&w)[4]) {
#pragma unroll
  for (int x = 0; x < 8; ++x) {
    const int f = 16 * role.G + 8 * (x >> 2) + 4 * role.j + (x & 3);
    u32x2 out;
    if (SCALE) {
      out.x = E::pack(elem_f32<E>(rows[0], x) * w[0], elem_f32<E>(rows[1], x) * w[1]);
      out.y = E::pack(elem_f32<E>(rows[2], x) * w[2], elem_f32<E>(rows[3], x) * w[3]);
    } else {
      out.x = elem_bits(rows[0], x) | (elem_bits(rows[1], x) << 16);
      out.y = elem_bits(rows[2], x) | (elem_bits(rows[3], x) << 16);
    }
    *reinterpret_cast<u32x2 *>(tile + tr_off(f, role.rowq >> 1) + ((role.rowq & 1) << 3)) = out;
  }
}

// A thread's two 8-byte pieces of the row that starts `row_bytes` (uniform across the workgroup) past
// the block pointer `tile` (scalar, see uniform_ptr), at the thread's own byte offset `lane_off` (32 bits,
// loop-invariant); a piece that lies beyond the row width, or the whole row, reads as zeros.
struct PieceMask {
  bool lo, hi;
};
__device__ __forceinline__ u32x4 load_row_pieces(gmem_ptr tile, int row_bytes, uint32_t lane_off, PieceMask ok,
                                                 bool row_ok) {
  typedef const __attribute__((address_space(1))) u32x2 *gmem_u32x2;
  gmem_ptr p = tile + row_bytes;
  const u32x2 zero = {0u, 0u};
  const u32x2 lo = (row_ok && ok.lo) ? *reinterpret_cast<gmem_u32x2>(p + lane_off) : zero;
  const u32x2 hi = (row_ok && ok.hi) ? *reinterpret_cast<gmem_u32x2>(p + lane_off + 16) : zero;
  u32x4 r;
  r.x = lo.x;
  r.y = lo.y;
  r.z = hi.x;
  r.w = hi.y;
  return r;
}
// thread-own part of the address: `row` rows down, then the thread's first piece
__device__ __forceinline__ uint32_t lane_offset(const LoaderRole &role, int row, int units) {
  return (uint32_t)((row * units + 4 * role.G + role.j) * 8);
}
__device__ __forceinline__ PieceMask piece_mask(const LoaderRole &role, int units) {
  PieceMask m;
  m.lo = 4 * role.G + role.j < units;
  m.hi = 4 * role.G + 2 + role.j < units;
  return m;
}

struct SegWork {
  int bh, seg;
  int64_t tok0;  // first token of the segment
  int nblk;      // 64-token blocks in it, the last one possibly partial
  int tail;      // tokens in its last block (1..64); below 64 only at the end of a ragged chunk
};
// `item` enumerates (b*h, segment) pairs
__device__ __forceinline__ SegWork seg_work(const Geom &g, int item) {
  SegWork r;
  // the division runs on the vector unit; its (uniform) result goes back to a scalar register
  r.bh = __builtin_amdgcn_readfirstlane(item / g.n_seg);
  r.seg = item - r.bh * g.n_seg;
  r.tok0 = (int64_t)r.seg * g.seg_len;
  int64_t t1 = r.tok0 + g.seg_len;
  if (t1 > g.n) t1 = g.n;
  const int tokens = (int)(t1 - r.tok0);
  r.nblk = (tokens + BLK - 1) / BLK;
  r.tail = tokens - (r.nblk - 1) * BLK;
  return r;
}

// ------------------------------------------------------------------------------
// Every sweep kernel below is an instance of ws_body<E, REV, TRANS, SRC, MODE>.
//
// MODE.  M_RAGGED: the chunk length is not a multiple of 64, so the last block of the last segment is
// partial (rows past its end read as zeros, stores are masked, and the decay factors of that one block use
// its true length).  M_NARROW: in addition X and Y rows hold `fa` features, Z and Out rows `fb`
// (multiples of 8, at most 128), read zero-extended to 128 and written back at their own width; the upper
// half of the feature steps and state tiles, and waves whose columns lie in the zero extension, are skipped
// when they would only see zeros.  M_ALIGNED carries none of that bookkeeping; fa and fb are read in
// M_NARROW only.
//
// SRC says where the state entering the segment comes from.
// SRC_SCANNED: `states` holds it, left there by the decayed scan over the segments' own states.
// SRC_COMBINE: `states` holds the segments' OWN states as the pre-pass wrote them, and the
//   workgroup runs the scan's recurrence itself over the segments before (after) its own,
//   starting from the chunk's incoming state `carry_in` (d x e floats per (b, h), may be NULL):
//   St <- l^len_j St + own_j.  With few segments that is cheaper than a scan launch.
// SRC_WALK: no workspace at all: the state is rebuilt by first walking the blocks that precede the
//   segment (follow it, going backwards) and only updating the state: no X tile, no score, no
//   output.  The walk starts from `carry_in`, or from zero as many blocks back as the head's decay
//   reaches (weights below 2^-SKIP_LOG2 are dropped).  One launch then does a whole chunk; the
//   repeated walks make it a tool for short chunks.
// In the last two the workgroup of the segment visited last writes the state it ends with to
// `carry_out` (non-transposed roles only).
// ------------------------------------------------------------------------------
// The sweep, with the work of a block split between two groups of waves.  A workgroup whose waves all run
// fill -> products -> store one after the other spends most of a block waiting for its own LDS round trips
// (measured on such a form of this kernel: 5806 against 3700 clock ticks per block alone on a CU); here 512
// threads form one workgroup per CU:
//   waves 0-3 ("feed"): global loads, the LDS tiles of the NEXT block (transposes and decay scaling
//     included), the masked score tile of the current block, the coalesced output stores;
//   waves 4-7 ("math"): own the state and the output accumulators (wave 4 + w: columns [32w, 32w + 32)):
//     state term, intra-block term, state update, output staging.
// The tiles are double-buffered (two sets of X, Y token-major and Y^T, Z^T feature-major, 144 384 B
// with the score tile), and a block takes two barriers:
//     feed: store O(t-1), score(t)    | math: state term(t)
//   ---- barrier ----
//     feed: fill(t+1),                | math: intra(t) from the score tile, state update(t), stage O(t) into
//           issue loads(t+2)          |       the X tile of block t (no longer read)
//   ---- barrier ----
// O(t-1) waits in the X tile of the set that fill(t+1) overwrites after the first barrier.
// Both groups run their own loop; each executes exactly 1 + 2 * nblk barriers.
constexpr int WS_THREADS = 512;
constexpr int WS_XN = 0, WS_YN = BLK * LDN, WS_YT = 2 * BLK * LDN, WS_ZT = WS_YT + F * LDT;
constexpr int WS_SET = WS_ZT + F * LDT;        // one block's tiles
constexpr int WS_SC = 2 * WS_SET;              // the score tile
constexpr int WS_LDS = WS_SC + BLK * LDSC;     // 144 384 B: one workgroup per CU

template <class E, bool REV, bool TRANS, int SRC, int MODE>
__device__ __forceinline__ void
ws_body(const elem16_t *__restrict__ X, const elem16_t *__restrict__ Y, const elem16_t *__restrict__ Z,
        const float *__restrict__ S, const float *__restrict__ states, elem16_t *__restrict__ Out, const Geom &g,
        int fa, int fb, int item, char *smem, const float *__restrict__ carry_in,
        float *__restrict__ carry_out = nullptr) {
  constexpr bool RAGGED = MODE != M_ALIGNED, NARROW = MODE == M_NARROW;
  constexpr bool LEAVES_STATE = SRC != SRC_SCANNED;  // the sweep's final state is the chunk's outgoing one
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w8 = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int w = w8 & 3;  // feed: score quadrant; math: column block
  const int c = lane & 31, hh = lane >> 5;

  const SegWork sw = seg_work(g, item);
  const float sl = S[sw.bh % g.h] * LOG2E;
  const int64_t row0 = (int64_t)sw.bh * g.n + sw.tok0;
  const int nblk = sw.nblk;
  const int step = REV ? -1 : 1;
  const int blk0 = REV ? nblk - 1 : 0;
  const float blockdec = decay(sl, (float)BLK);

  // SRC_WALK: the state entering the segment is rebuilt by walking `runup` blocks outside it first (before it,
  // or after it going backwards), as far as the head's decay reaches, from the chunk's incoming state if the
  // walk gets to the chunk's end, else from zero.  Blocks are numbered relative to the segment; walk and sweep
  // form one run of runup + nblk blocks, first_blk, first_blk + step, ..., of which the first `runup` only
  // update the state (one barrier each, both groups).
  const int total_blk = (int)((g.n + BLK - 1) / BLK);  // blocks in the chunk
  const int seg_blk0 = (int)(sw.tok0 / BLK);           // the segment's first block
  const int chunk_tail = (int)(g.n - (int64_t)(total_blk - 1) * BLK);
  // tokens in a block (numbered relative to the segment): a partial block is the chunk's last one
  auto len_of = [&](int blk) __attribute__((always_inline)) {
    if (!RAGGED) return BLK;
    return seg_blk0 + blk == total_blk - 1 ? chunk_tail : BLK;
  };
  int runup = 0;
  bool take_carry = false;
  if (SRC == SRC_WALK) {
    const int avail = REV ? total_blk - (seg_blk0 + nblk) : seg_blk0;
    int reach = avail;
    if (sl > 0.f) {
      const float x = SKIP_LOG2 / (sl * (float)BLK);  // blocks over which a weight falls to 2^-SKIP_LOG2
      if (x < (float)avail) reach = (int)x + 1;
    }
    runup = __builtin_amdgcn_readfirstlane(min(reach, avail));
    take_carry = carry_in != nullptr && runup == avail;
  }
  const int first_blk = blk0 - runup * step;
  const int run = runup + nblk;  // blocks in the whole run

  if (w8 < 4) {
    // ================================ feed waves ================================
    const int ftid = tid;  // 0..255
    const LoaderRole xr = x_role(ftid), yr = yz_role(ftid);
    const int chunk = ftid & 15, rowq = ftid >> 4;
    const int xw = NARROW ? fa : F, zw = NARROW ? fb : F;  // row widths in elements
    const u32x2 *Xg = reinterpret_cast<const u32x2 *>(X + row0 * xw);
    const u32x2 *Yg = reinterpret_cast<const u32x2 *>(Y + row0 * xw);
    const u32x2 *Zg = reinterpret_cast<const u32x2 *>(Z + row0 * zw);
    u32x4 *Og = reinterpret_cast<u32x4 *>(Out + row0 * zw);
    const int xu = xw / 4, zu = zw / 4;  // 8-byte units per row
    const int ou = zw / 8;               // 16-byte units per output row
    float kdec[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int b = 4 * yr.rowq + r;
      kdec[r] = decay(sl, REV ? (float)b : (float)(BLK - b));
    }
    const int qI = w >> 1, qJ = w & 1;
    const bool q_active = REV ? !(qI == 1 && qJ == 0) : !(qI == 0 && qJ == 1);
    const uint32_t x_off = lane_offset(xr, xr.rowq, xu), y_off = lane_offset(yr, 4 * yr.rowq, xu),
                   z_off = lane_offset(yr, 4 * yr.rowq, zu);
    const PieceMask all = {true, true};
    const PieceMask x_ok = piece_mask(xr, xu), y_ok = piece_mask(yr, xu), z_ok = piece_mask(yr, zu);

    // the block in flight, two 8-byte pieces per row (see LoaderRole)
    u32x4 nx[4], ny[4], nz[4];
    // k: position in the run; walk blocks (k < runup) need no X tile
    auto issue_loads = [&](int k) __attribute__((always_inline)) {
      const int blk = first_blk + k * step;
      const int len = len_of(blk);  // rows past a partial block's end and pieces past a narrow row's width read as zeros
      const gmem_ptr xblk = uniform_ptr(reinterpret_cast<const char *>(Xg) + (int64_t)blk * BLK * xu * 8);
      const gmem_ptr yblk = uniform_ptr(reinterpret_cast<const char *>(Yg) + (int64_t)blk * BLK * xu * 8);
      const gmem_ptr zblk = uniform_ptr(reinterpret_cast<const char *>(Zg) + (int64_t)blk * BLK * zu * 8);
      if (SRC != SRC_WALK || k >= runup) {
#pragma unroll
        for (int it = 0; it < 4; ++it)
          nx[it] = load_row_pieces(xblk, 16 * it * xu * 8, x_off, NARROW ? x_ok : all,
                                   !RAGGED || xr.rowq + 16 * it < len);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bool row_ok = !RAGGED || 4 * yr.rowq + r < len;
        ny[r] = load_row_pieces(yblk, r * xu * 8, y_off, NARROW ? y_ok : all, row_ok);
        nz[r] = load_row_pieces(zblk, r * zu * 8, z_off, NARROW ? z_ok : all, row_ok);
      }
    };
    // writes the block held in nx / ny / nz into a tile set: token-major X and Y, feature-major Y (scaled by the
    // key decay) and Z
    auto fill = [&](char *set, int k) __attribute__((always_inline)) {
      if (SRC != SRC_WALK || k >= runup) {  // a walk block is only multiplied into the state
#pragma unroll
        for (int it = 0; it < 4; ++it)
          *reinterpret_cast<u32x4 *>(set + WS_XN + (xr.rowq + 16 * it) * LDN + (2 * xr.G + xr.j) * 16) = nx[it];
#pragma unroll
        for (int r = 0; r < 4; ++r)
          *reinterpret_cast<u32x4 *>(set + WS_YN + (4 * yr.rowq + r) * LDN + (2 * yr.G + yr.j) * 16) = ny[r];
      }
      const int len = len_of(first_blk + k * step);
      if (LEAVES_STATE && RAGGED && !REV && len != BLK) {
        // the chunk's partial last block, going forwards: its tokens sit `len - b` before the chunk end, which
        // matters here because the state it leaves is the outgoing one
        float kd[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) kd[r] = decay(sl, (float)max(len - (4 * yr.rowq + r), 0));
        store_transposed<E, true>(set + WS_YT, ny, yr, kd);
      } else {
        store_transposed<E, true>(set + WS_YT, ny, yr, kdec);
      }
      store_transposed<E, false>(set + WS_ZT, nz, yr, kdec);
    };
    // the output tile staged in `set`'s X region -> global rows of block `blk`
    auto store_out = [&](const char *set, int blk) __attribute__((always_inline)) {
      const int64_t brow = (int64_t)blk * BLK;
      const int len = len_of(blk);
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int row = rowq + 16 * r4;
        if (!RAGGED || (row < len && (!NARROW || chunk < ou)))
          __builtin_nontemporal_store(*reinterpret_cast<const u32x4 *>(set + WS_XN + row * LDN + chunk * 16),
                                      &Og[(brow + row) * (NARROW ? ou : F / 8) + chunk]);
      }
    };
    // this wave's quadrant of the transposed score tile: sc[4g+r] = y_b . x_a, b = 32qJ+8g+4hh+r, a = 32qI+c
    auto score = [&](const char *set) __attribute__((always_inline)) {
      if (!q_active) return;
      floatx16 sc;
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[r] = 0.f;
      const char *xa = set + WS_XN + (32 * qI + c) * LDN + hh * 16;
      const char *ya = set + WS_YN + (32 * qJ + c) * LDN + hh * 16;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) sc = E::mfma(lds16(ya + ks * 32), lds16(xa + ks * 32), sc);
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
        u32x2 o;
        o.x = E::pack(m[0], m[1]);
        o.y = E::pack(m[2], m[3]);
        *reinterpret_cast<u32x2 *>(smem + WS_SC + a * LDSC + (32 * qJ + 8 * gq + 4 * hh) * 2) = o;
      }
    };

    issue_loads(0);
    fill(smem, 0);
    if (run > 1) issue_loads(1);
    __syncthreads();  // barrier 0: block 0 of the run visible
    int k = 0;
    for (; k < runup; ++k) {  // walk: the math waves multiply block k into the state meanwhile
      fill(smem + ((k + 1) & 1) * WS_SET, k + 1);  // k + 1 < run: a sweep block follows the walk
      if (k + 2 < run) issue_loads(k + 2);
      __syncthreads();  // walk barrier k
    }
    for (; k < run; ++k) {
      char *cur = smem + (k & 1) * WS_SET, *nxt = smem + ((k + 1) & 1) * WS_SET;
      // the stores go first: by the time the fill below waits for its loads (loads and stores share one
      // counter, so that wait drains both) they have long left
      if (k > runup) store_out(nxt, first_blk + (k - 1) * step);
      score(cur);
      __syncthreads();  // first barrier of a sweep block: score tile complete; X / Y of `cur` and the output staged in `nxt` no longer read
      if (k + 1 < run) {
        fill(nxt, k + 1);
        if (k + 2 < run) issue_loads(k + 2);
      }
      __syncthreads();  // second barrier: next block visible; output of this block staged
    }
    store_out(smem + ((run - 1) & 1) * WS_SET, first_blk + (run - 1) * step);
    return;
  }

  // ================================== math waves ==================================
  float qdec[2];
#pragma unroll
  for (int I = 0; I < 2; ++I) {
    const int a = 32 * I + c;
    qdec[I] = decay(sl, REV ? (float)(BLK - a) : (float)a);
  }
  // state entering the segment: st[T][4g+r] = St[32T+8g+4hh+r][32w+c]
  floatx16 st[4];
#pragma unroll
  for (int T = 0; T < 4; ++T)
#pragma unroll
    for (int r = 0; r < 16; ++r) st[T][r] = 0.f;
  // M_NARROW: a wave whose 32 columns all lie past the width of Z has nothing to compute (it still takes part in
  // every barrier); the upper 64 features are skipped as a whole when the rows are no wider
  const bool wave_active = !NARROW || 32 * w < fb;
  const bool upper_half = !NARROW || fa > 64;
  // st <- f * st + M, M being the 128 x 128 fp32 tile whose element (row, col) is src[row * ld + col], or for a
  // transposed role src[col * ld + row]; `bounded`: src holds only fa x fb (transposed: fb x fa) elements
  auto add_state_ld = [&](const float *src, int ld, float f, bool bounded) __attribute__((always_inline)) {
    typedef const __attribute__((address_space(1))) float *gmem_f32;
    const uint32_t lane_off =
        (uint32_t)(TRANS ? (32 * w + c) * ld + 4 * hh : 4 * hh * ld + 32 * w + c) * (uint32_t)sizeof(float);
    const bool col_ok = !bounded || 32 * w + c < fb;
#pragma unroll
    for (int T = 0; T < 4; ++T)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const int band = 32 * T + 8 * gq;
        const gmem_ptr bp = uniform_ptr(reinterpret_cast<const char *>(src + (TRANS ? band : (int64_t)band * ld)));
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const bool ok = col_ok && (!bounded || band + 4 * hh + r < fa);
          const float own =
              ok ? *reinterpret_cast<gmem_f32>(bp + lane_off + (uint32_t)(TRANS ? r : r * ld) * sizeof(float)) : 0.f;
          st[T][4 * gq + r] = fmaf(f, st[T][4 * gq + r], own);
        }
      }
  };
  // a state of the workspace (128 x 128, zero beyond fa x fb) / the chunk's incoming state (fa x fb, unpadded)
  auto add_state = [&](const float *src, float f) __attribute__((always_inline)) { add_state_ld(src, F, f, false); };
  auto add_carry = [&]() __attribute__((always_inline)) {
    add_state_ld(carry_in + (int64_t)sw.bh * fa * fb, NARROW ? (TRANS ? fa : fb) : F, 0.f, NARROW);
  };
  if (SRC == SRC_WALK) {
    if (take_carry) add_carry();
  } else if (SRC == SRC_SCANNED) {
    if (states) {
      // the scanned state of this segment, or for a head the scan leaves out (state_dies_in_segment), whose
      // own states are still where the pre-pass put them, the own state of the segment visited before it
      // (the chunk's incoming state for the first one)
      // The workspace holds one state per segment of the pre-pass, of which this sweep segment spans
      // `sub` (a power of two; 1 unless the plan cut long segments finer for the pre-pass): the state that
      // enters it is the one entering its first piece in sweep order.
      const int sub = g.seg_len / g.pre_len;
      const int piece = REV ? min(sw.seg * sub + sub, g.pre_n) - 1 : sw.seg * sub;
      const float *src = states + ((int64_t)sw.bh * g.pre_n + piece) * (F * F);
      bool from_carry = false;
      if (state_dies_in_segment(S[sw.bh % g.h], g)) {
        const int nb = REV ? piece + 1 : piece - 1;
        if (nb < 0 || nb >= g.pre_n)
          from_carry = true;
        else
          src = states + ((int64_t)sw.bh * g.pre_n + nb) * (F * F);
      }
      // (for such a head the scan kernel has parked the chunk's incoming state in the slot of the piece it
      // visits last, so that nothing reads `carry_in`'s memory once the outgoing state may have replaced it)
      if (from_carry) src = states + ((int64_t)sw.bh * g.pre_n + (REV ? 0 : g.pre_n - 1)) * (F * F);
      if (!from_carry || carry_in != nullptr) add_state(src, 0.f);
    }
  } else {
    // `states` holds the segments' OWN states.  The scan's recurrence, St <- l^len_j St + own_j over the
    // segments visited before this one, is run here -- over as many of them as the head's decay reaches:
    // an own state further back arrives weighted below 2^-SKIP_LOG2 (everything between it and this
    // segment is a full-length segment) and is left out, and so is the chunk's incoming state unless the
    // walk starts at the chunk's end.  These waves have the time: the feed waves are fetching block 0.
    const int n_before = REV ? g.n_seg - 1 - sw.seg : sw.seg;
    int first = 0;
    if (sl > 0.f) {
      const float segs = SKIP_LOG2 / (sl * (float)g.seg_len);  // full segments over which a weight falls to 2^-SKIP_LOG2
      if (segs < (float)n_before) first = n_before - ((int)segs + 1);
    }
    first = __builtin_amdgcn_readfirstlane(first);
    if (first == 0 && carry_in) add_carry();
    if (states) {
      const float *base = states + (int64_t)sw.bh * g.n_seg * (F * F);
      const float full = decay(sl, (float)g.seg_len);
      const float last = decay(sl, (float)(g.n - (int64_t)(g.n_seg - 1) * g.seg_len));
      for (int i = first; i < n_before; ++i) {
        const int j = REV ? g.n_seg - 1 - i : i;
        add_state(base + (int64_t)j * (F * F), j == g.n_seg - 1 ? last : full);
      }
    }
  }
  // St <- l^64 St + (scaled Y)^T Z from the feature-major tiles of `set`
  auto update_state = [&](const char *set, const u32x4 (&zf)[4], float bd) __attribute__((always_inline)) {
#pragma unroll
    for (int T = 0; T < 4; ++T)
#pragma unroll
      for (int r = 0; r < 16; ++r) st[T][r] *= bd;
    u32x4 yf[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int T = 0; T < 4; ++T)
        if (T < 2 || upper_half) yf[u][T] = lds16(set + WS_YT + tr_off(32 * T + c, 2 * u + hh));
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int T = 0; T < 4; ++T)
        if (T < 2 || upper_half) st[T] = E::mfma(yf[u][T], zf[u], st[T]);  // state rows past the width of Y stay zero
  };
  __syncthreads();  // barrier 0
  for (int k = 0; k < runup; ++k) {  // walk
    const char *set = smem + (k & 1) * WS_SET;
    if (wave_active) {
      const int len = len_of(first_blk + k * step);
      u32x4 zf[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) zf[u] = lds16(set + WS_ZT + tr_off(32 * w + c, 2 * u + hh));
      update_state(set, zf, RAGGED && len != BLK ? decay(sl, (float)len) : blockdec);
    }
    __syncthreads();  // walk barrier k
  }
  for (int it = 0; it < nblk; ++it) {
    char *cur = smem + ((runup + it) & 1) * WS_SET;
    // A partial block is the chunk's last one.  Going forwards nothing after it uses the state (but the outgoing
    // state where the sweep leaves it); going backwards it comes first and the entering state sits `len` (not 64)
    // tokens ahead.
    const int len = len_of(blk0 + it * step);
    float qd[2] = {qdec[0], qdec[1]};
    float bd = blockdec;
    if (RAGGED && REV && len != BLK) {
      qd[0] = decay(sl, (float)max(len - c, 0));
      qd[1] = decay(sl, (float)max(len - 32 - c, 0));
      bd = decay(sl, (float)len);
    }
    if (LEAVES_STATE && RAGGED && !REV && len != BLK) bd = decay(sl, (float)len);
    // state term, transposed: acc[I][4g+r] = sum_f St[f][32w+8g+4hh+r] x_a[f], a = 32I+c
    floatx16 acc[2];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[0][r] = 0.f;
      acc[1][r] = 0.f;
    }
    if (wave_active) {
      // all sixteen X fragments are requested before the first product (these waves have the registers for it)
      const char *x0 = cur + WS_XN + c * LDN + hh * 16;
      const char *x1 = x0 + 32 * LDN;
      u32x4 xf[8][2];
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        if (ks >= 4 && !upper_half) continue;
        xf[ks][0] = lds16(x0 + ks * 32);
        xf[ks][1] = lds16(x1 + ks * 32);
      }
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        if (ks >= 4 && !upper_half) continue;
        const int T = ks >> 1, u = ks & 1;
        u32x4 a;
        a.x = E::pack(st[T][8 * u + 0], st[T][8 * u + 1]);
        a.y = E::pack(st[T][8 * u + 2], st[T][8 * u + 3]);
        a.z = E::pack(st[T][8 * u + 4], st[T][8 * u + 5]);
        a.w = E::pack(st[T][8 * u + 6], st[T][8 * u + 7]);
        acc[0] = E::mfma(a, xf[ks][0], acc[0]);
        acc[1] = E::mfma(a, xf[ks][1], acc[1]);
      }
    }
#pragma unroll
    for (int I = 0; I < 2; ++I)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[I][r] *= qd[I];
    __syncthreads();  // barrier 2 it + 1: score tile complete
    if (wave_active) {
      u32x4 zf[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) zf[u] = lds16(cur + WS_ZT + tr_off(32 * w + c, 2 * u + hh));
      // intra-block term: acc[I] += Z^T[32w.., tokens] * score[a][tokens]
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int I = 0; I < 2; ++I) {
          const bool needed = REV ? (I == 0 || u >= 2) : (I == 1 || u < 2);
          if (needed)
            acc[I] = E::mfma(zf[u], lds16(smem + WS_SC + (32 * I + c) * LDSC + (16 * u + 8 * hh) * 2), acc[I]);
        }
      update_state(cur, zf, bd);
    }
    // stage the output tile (token-major) in the X region of this block
    if (wave_active)
#pragma unroll
    for (int I = 0; I < 2; ++I)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        u32x2 o;
        o.x = E::pack(acc[I][4 * gq + 0], acc[I][4 * gq + 1]);
        o.y = E::pack(acc[I][4 * gq + 2], acc[I][4 * gq + 3]);
        *reinterpret_cast<u32x2 *>(cur + WS_XN + (32 * I + c) * LDN + (32 * w + 8 * gq + 4 * hh) * 2) = o;
      }
    __syncthreads();  // barrier 2 it + 2
  }
  // the segment visited last leaves the chunk's outgoing state
  if (SRC != SRC_SCANNED && !TRANS && carry_out != nullptr && sw.seg == (REV ? 0 : g.n_seg - 1)) {
    float *cp = carry_out + (int64_t)sw.bh * fa * fb;
    const int col = 32 * w + c;
#pragma unroll
    for (int T = 0; T < 4; ++T)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 32 * T + 8 * (r >> 2) + 4 * hh + (r & 3);
        if (!NARROW || (row < fa && col < fb)) cp[row * (NARROW ? fb : F) + col] = st[T][r];
      }
  }
}

template <class E, bool REV, bool TRANS, int SRC, int MODE>
__global__ void __launch_bounds__(WS_THREADS, 1)
la_apply(const elem16_t *__restrict__ X, const elem16_t *__restrict__ Y, const elem16_t *__restrict__ Z,
            const float *__restrict__ S, const float *__restrict__ states, const float *__restrict__ carry_in,
            float *__restrict__ carry_out, elem16_t *__restrict__ Out, Geom g) {
  extern __shared__ __align__(16) char smem[];
  // SRC_COMBINE: later segments have more states to gather first, so they are started first
  const int item = SRC == SRC_COMBINE ? g.b * g.h * g.n_seg - 1 - (int)blockIdx.x : (int)blockIdx.x;
  ws_body<E, REV, TRANS, SRC, MODE>(X, Y, Z, S, states, Out, g, g.d, g.e, item, smem, carry_in, carry_out);
}

// A whole short chunk in one launch: every workgroup rebuilds the state entering its segment (SRC_WALK), so
// there is no pre-pass, no scan and no workspace.  Workgroups are dealt to the 8 XCDs round-robin: all
// segments of one (b, h) go to the same XCD, whose L2 then serves the repeated walks over that (b, h)'s K
// and V; later segments, which walk over more blocks first, are started first.
template <class E, int MODE>
__global__ void __launch_bounds__(WS_THREADS, 1)
la_fused_fwd(const elem16_t *__restrict__ Q, const elem16_t *__restrict__ K, const elem16_t *__restrict__ V,
                const float *__restrict__ S, const float *__restrict__ kv_in, float *__restrict__ kv_out,
                elem16_t *__restrict__ O, Geom g) {
  extern __shared__ __align__(16) char smem[];
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int bh = (slot / g.n_seg) * 8 + xcd;
  if (bh >= g.b * g.h) return;
  const int item = bh * g.n_seg + (g.n_seg - 1 - slot % g.n_seg);
  ws_body<E, false, false, SRC_WALK, MODE>(Q, K, V, S, nullptr, O, g, g.d, g.e, item, smem, kv_in, kv_out);
}

// roles as in la_bwd3 (the dV role leaves dKV_out); all roles and segments of one (b, h) on one XCD
template <class E, int MODE>
__global__ void __launch_bounds__(WS_THREADS, 1)
la_fused_bwd(const elem16_t *__restrict__ Q, const elem16_t *__restrict__ K, const elem16_t *__restrict__ V,
                const elem16_t *__restrict__ DO, const float *__restrict__ S, const float *__restrict__ kv_in,
                const float *__restrict__ dkv_in, float *__restrict__ dkv_out, elem16_t *__restrict__ DQ,
                elem16_t *__restrict__ DK, elem16_t *__restrict__ DV, Geom g) {
  extern __shared__ __align__(16) char smem[];
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int per_bh = 3 * g.n_seg;
  const int bh = (slot / per_bh) * 8 + xcd;
  if (bh >= g.b * g.h) return;
  const int rem = slot % per_bh;
  const int role = rem % 3, k = rem / 3;  // k-th longest walk of its role
  if (role == 0)
    ws_body<E, false, true, SRC_WALK, MODE>(DO, V, K, S, nullptr, DQ, g, g.e, g.d, bh * g.n_seg + g.n_seg - 1 - k, smem,
                                            kv_in);
  else if (role == 1)
    ws_body<E, true, false, SRC_WALK, MODE>(K, Q, DO, S, nullptr, DV, g, g.d, g.e, bh * g.n_seg + k, smem, dkv_in,
                                            dkv_out);
  else
    ws_body<E, true, true, SRC_WALK, MODE>(V, DO, Q, S, nullptr, DK, g, g.e, g.d, bh * g.n_seg + k, smem, dkv_in);
}

// The three gradients in one launch.  Workgroups come in triples (dQ, dV, dK) that work on the same
// (b*h, segment) and therefore read the same Q, K, V, dO blocks; the triple is spread over block indices 8
// apart so that all three land on the same XCD (workgroups are dealt to the 8 XCDs round-robin) and share
// its L2.
template <class E, int SRC, int MODE>
__global__ void __launch_bounds__(WS_THREADS, 1)
la_bwd3(const elem16_t *__restrict__ Q, const elem16_t *__restrict__ K, const elem16_t *__restrict__ V,
           const elem16_t *__restrict__ DO, const float *__restrict__ S, const float *__restrict__ kv_states,
           const float *__restrict__ dkv_states, const float *__restrict__ kv_in, const float *__restrict__ dkv_in,
           float *__restrict__ dkv_out, elem16_t *__restrict__ DQ, elem16_t *__restrict__ DK,
           elem16_t *__restrict__ DV, Geom g) {
  extern __shared__ __align__(16) char smem[];
  const int n_items = g.b * g.h * g.n_seg;
  const int grp = blockIdx.x / 24, r = blockIdx.x - grp * 24;
  const int role = r >> 3;
  const int item = n_items - 1 - (grp * 8 + (r & 7));
  if (item < 0) return;
  if (role == 0)
    ws_body<E, false, true, SRC, MODE>(DO, V, K, S, kv_states, DQ, g, g.e, g.d, item, smem, kv_in);
  else if (role == 1)
    ws_body<E, true, false, SRC, MODE>(K, Q, DO, S, dkv_states, DV, g, g.d, g.e, item, smem, dkv_in, dkv_out);
  else
    ws_body<E, true, true, SRC, MODE>(V, DO, Q, S, dkv_states, DK, g, g.e, g.d, item, smem, dkv_in);
}

// ------------------------------------------------------------------------------
// A segment's own state:  causal  sum_b l^(L-b) y_b^T z_b ;  anti-causal  sum_b l^b y_b^T z_b
// (b from the segment start, L its length), written token-free as 128 x 128 fp32.  Y rows hold
// g.d features and Z rows g.e (M_NARROW; 128 otherwise).
//
// Blocks whose every token carries a weight below 2^-SKIP_LOG2 are neither read nor multiplied:
// with slope s a token that lies x tokens from the segment's far end weighs exp(-s x), so a
// fast-decaying head only needs the last (causal) or first (anti-causal) SKIP_LOG2 ln2 / s tokens
// of each segment.  What is dropped is below 2^-24 of a full-weight term, i.e. under the fp32
// rounding (2^-24) of the sum it would be added to.  s = 0 skips nothing.
//
// That leaves the workgroups unevenly loaded -- those of slow-decaying heads still read whole
// segments -- so one workgroup has to be able to pull more than an even share of the memory
// bandwidth.  512 threads (8 waves): threads 0-255 fetch the Y tile, 256-511 the Z tile, each
// keeping D blocks in flight in registers (16 registers per block) on top of the two LDS
// buffers; wave (wc, rh) owns rows [64 rh, 64 rh + 64) x columns [32 wc, 32 wc + 32) of the state
// as two accumulator tiles.
//
// Both tiles stay token-major in LDS, as they are in memory (16-byte copies, Y scaled by the decay
// weights on the way); the products contract over tokens, so the MFMA operands are fetched with
// the transposing LDS read.
constexpr int STATE_THREADS = 512;
constexpr int LDR = 320;  // bytes per token row (256 + 64: the four rows that one transposing read
                          // touches per half-wave fall on disjoint banks)
constexpr int STATE_TILE = BLK * LDR;
constexpr int STATE_LDS = 2 * 2 * STATE_TILE;  // double-buffered {Y scaled, Z}: 80 KiB
// Blocks in flight per thread in registers (even).  Long walks gain from the deeper pipeline (b*h = 16,
// n = 65536, 2048-token pieces: 46 us per launch against 49); on short ones the longer start-up costs more
// than it gains (320-token segments: 13.1 us against 12.4).  The shallow form stays within 128 registers, so two
// workgroups share a CU; the deep one runs one per CU (squeezed into 128 registers it spills and measured slower).
constexpr int STATE_DEPTH_LONG = 4, STATE_DEPTH_SHORT = 2;
constexpr int STATE_LONG_WALK = 1024;  // tokens per segment from which the deeper pipeline is used

typedef short v4i16 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4i16 *lds_v4i16;
// The transposing 8-byte read works in groups of 16 lanes: lane i of a group receives, as element j,
// element (i % 4) of what lane (4 j + i / 4) of the group addressed.  With lane s of a group addressing
// token T + s / 4, features f + 4 (s % 4) .. + 3, lane i ends up with feature f + i of tokens T .. T + 3.
__device__ __forceinline__ u32x2 lds_tr8(const char *p) {
  const v4i16 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16)(p));
  return __builtin_bit_cast(u32x2, r);
}
// MFMA operand of lane (c, hh): feature f0 + c, tokens t0 + 8 hh .. + 7 (`lane_part` holds the lane's share
// of the address, see la_seg_state)
__device__ __forceinline__ u32x4 token_fragment(const char *tile, int lane_part, int f0, int t0) {
  const char *p = tile + lane_part + t0 * LDR + f0 * 2;
  const u32x2 lo = lds_tr8(p), hi = lds_tr8(p + 4 * LDR);
  u32x4 r;
  r.x = lo.x;
  r.y = lo.y;
  r.z = hi.x;
  r.w = hi.y;
  return r;
}

template <class E, bool REV, int MODE, int D>
__global__ void __launch_bounds__(STATE_THREADS, 1)
la_seg_state(const elem16_t *__restrict__ Y, const elem16_t *__restrict__ Z, const float *__restrict__ S,
             float *__restrict__ states, Geom g, int skip_seg, int sub) {
  constexpr bool RAGGED = MODE != M_ALIGNED, NARROW = MODE == M_NARROW;
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w8 = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave index, uniform: keeps it in an SGPR
  const int wc = w8 & 3, rh = w8 >> 2;                      // column block and row half of this wave's tiles
  const bool zgrp = w8 >= 4;                                // this wave fetches Z (else Y)
  const int c = lane & 31, hh = lane >> 5;
  // loader: 16 consecutive threads copy one row, the thread's 16 bytes are features 8 cq .. + 7 of rows
  // rq, rq + 16, rq + 32, rq + 48
  const int cq = tid & 15, rq = (tid & 255) >> 4;

  // slow-decaying heads (the later ones in the usual slope schedules) have the most to read: first
  const int n_items = g.b * g.h * g.n_seg;
  const SegWork sw = seg_work(g, n_items - 1 - (int)blockIdx.x);
  if (sw.seg == skip_seg) return;  // the scan's final segment feeds only the outgoing carry
  const float slope = S[sw.bh % g.h];
  // Where sweep segments span `sub` > 1 of these segments, a head that takes no part in the scan
  // (state_dies_in_segment) has readers for one state in `sub` only: a sweep reads the own state of the piece
  // next to its segment -- the last piece of the segment before it, or going backwards the first piece of the
  // segment after it -- and the outgoing state, if one is wanted (skip_seg < 0), is formed from the two pieces
  // visited last.  The other pieces are left out, and their slots in `states` unwritten.
  if (sub > 1 && state_dies_in_segment(slope, g)) {
    const int p = sw.seg;
    bool read = REV ? (p % sub == 0 && p >= sub) : (p % sub == sub - 1 && p + 1 < g.n_seg);
    if (skip_seg < 0) read = read || (REV ? p <= 1 : p >= g.n_seg - 2);
    if (!read) return;
  }
  const float sl = slope * LOG2E;
  const int64_t row0 = (int64_t)sw.bh * g.n + sw.tok0;
  const int yw = NARROW ? g.d : F, zw = NARROW ? g.e : F;  // row widths in elements
  const int tw = zgrp ? zw : yw;                           // of the tile this thread fetches
  const char *Tg = reinterpret_cast<const char *>(zgrp ? Z + row0 * zw : Y + row0 * yw);
  const int row_bytes = tw * 2;

  const float blockdec = decay(sl, (float)BLK);
  float kdec[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int b = rq + 16 * r;
    kdec[r] = decay(sl, REV ? (float)b : (float)(BLK - b));
  }

  // blocks lo..hi of the segment are processed (uniform across the workgroup)
  int lo = 0, hi = sw.nblk - 1;
  if (sl > 0.f) {
    const float keep = SKIP_LOG2 / sl;  // tokens whose weight is at least 2^-SKIP_LOG2
    if (!REV) {
      // the last token of block t lies (tokens - 64 t - 63) tokens before the segment end
      const float x = ((float)((sw.nblk - 1) * BLK + sw.tail) - 63.f - keep) * (1.f / BLK);
      if (x > 0.f) lo = min((int)ceilf(x), hi);
    } else {
      // the first token of block t lies 64 t tokens after the segment start
      const float x = keep * (1.f / BLK);
      if (x < (float)hi) hi = (int)x;
    }
  }
  // the float arithmetic above ran on the vector unit; put the (uniform) results back in scalar
  // registers so that the block addresses stay scalar
  lo = __builtin_amdgcn_readfirstlane(lo);
  hi = __builtin_amdgcn_readfirstlane(hi);
  const int cnt = hi - lo + 1;

  floatx16 st[2];
#pragma unroll
  for (int T = 0; T < 2; ++T)
#pragma unroll
    for (int r = 0; r < 16; ++r) st[T][r] = 0.f;

  // A partial block (the end of a ragged chunk) reads its missing rows as zeros; going
  // forwards it is the last block, and its tokens sit `len - b` (not 64 - b) before the
  // segment end.
  const uint32_t t_off = (uint32_t)(rq * row_bytes + cq * 16);
  const bool col_ok = !NARROW || cq * 8 < tw;  // chunks past the row width read as zeros
  // every address is a workgroup-uniform block pointer plus one per-thread 32-bit offset
  auto issue_loads = [&](u32x4 (&nt)[4], int blk) __attribute__((always_inline)) {
    typedef const __attribute__((address_space(1))) u32x4 *gmem_u32x4;
    const int len = RAGGED && blk == sw.nblk - 1 ? sw.tail : BLK;
    const gmem_ptr tblk = uniform_ptr(Tg + (int64_t)blk * BLK * row_bytes);
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const bool ok = col_ok && (!RAGGED || rq + 16 * r < len);
      nt[r] = ok ? *reinterpret_cast<gmem_u32x4>(tblk + 16 * r * row_bytes + t_off) : zero;
    }
  };
  auto scaled = [&](const u32x4 &q, float w) __attribute__((always_inline)) {
    u32x4 o;
    o.x = E::pack(elem_f32<E>(q, 0) * w, elem_f32<E>(q, 1) * w);
    o.y = E::pack(elem_f32<E>(q, 2) * w, elem_f32<E>(q, 3) * w);
    o.z = E::pack(elem_f32<E>(q, 4) * w, elem_f32<E>(q, 5) * w);
    o.w = E::pack(elem_f32<E>(q, 6) * w, elem_f32<E>(q, 7) * w);
    return o;
  };
  char *const my_rows = smem + (zgrp ? STATE_TILE : 0) + rq * LDR + cq * 16;
  auto fill_lds = [&](int buf, const u32x4 (&nt)[4], int blk) __attribute__((always_inline)) {
    const int len = RAGGED && blk == sw.nblk - 1 ? sw.tail : BLK;
    char *dst = my_rows + buf * (2 * STATE_TILE);
    const bool partial = RAGGED && !REV && len != BLK;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      u32x4 v = nt[r];
      if (!zgrp) v = scaled(v, partial ? decay(sl, (float)max(len - (rq + 16 * r), 0)) : kdec[r]);
      *reinterpret_cast<u32x4 *>(dst + 16 * r * LDR) = v;
    }
  };
  // M_NARROW: columns past the width of Z stay zero, as do rows past Y's
  const bool wave_active = !NARROW || (32 * wc < g.e && (rh == 0 || g.d > 64));
  // the lane's share of a fragment address: token 8 hh + (lane % 16) / 4, feature 16 ((lane / 16) % 2) + 4 (lane % 4)
  const int lane_part = (8 * hh + ((lane & 15) >> 2)) * LDR + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  auto accumulate = [&](int buf, int blk) __attribute__((always_inline)) {
    const int len = RAGGED && blk == sw.nblk - 1 ? sw.tail : BLK;
    const float bd = RAGGED && len != BLK ? decay(sl, (float)len) : blockdec;
    const char *yt = smem + buf * (2 * STATE_TILE);
    const char *zt = yt + STATE_TILE;
    if (wave_active) {
      u32x4 zf[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) zf[u] = token_fragment(zt, lane_part, 32 * wc, 16 * u);
#pragma unroll
      for (int T = 0; T < 2; ++T) {
#pragma unroll
        for (int r = 0; r < 16; ++r) st[T][r] *= bd;
#pragma unroll
        for (int u = 0; u < 4; ++u)
          st[T] = E::mfma(token_fragment(yt, lane_part, 64 * rh + 32 * T, 16 * u), zf[u], st[T]);
      }
    }
  };

  // Block i of the walk (0 <= i < cnt) travels through register set i mod D.  Loads and LDS fills
  // past the end of the walk are not skipped but repeat its last block (served by the cache, never
  // used): with the same number of loads in flight on every path, the wait before a fill covers
  // exactly the oldest register set.
  const int first = REV ? hi : lo;
  const int step = REV ? -1 : 1;
  auto block_of = [&](int i) __attribute__((always_inline)) { return first + min(i, cnt - 1) * step; };
  u32x4 set[D][4];
#pragma unroll
  for (int k = 0; k < D; ++k) issue_loads(set[k], block_of(k));
  fill_lds(0, set[0], block_of(0));
  issue_loads(set[0], block_of(D));
  __syncthreads();
  // The walk leaves the loop from the middle of the unrolled body.  Were the exit test left to the loop
  // head, the compiler would have to assume that any of the D positions can precede the first one, could
  // no longer tell which register set holds the oldest loads there, and would wait for all of them.
  for (int i = 0;; i += D) {
    bool last = false;
#pragma unroll
    for (int k = 0; k < D; ++k) {  // D is even: LDS buffer (i + k) & 1 == k & 1
      accumulate(k & 1, block_of(i + k));
      __builtin_amdgcn_sched_barrier(0);
      fill_lds((k + 1) & 1, set[(k + 1) % D], block_of(i + k + 1));
      __builtin_amdgcn_sched_barrier(0);
      issue_loads(set[(k + 1) % D], block_of(i + k + 1 + D));
      __syncthreads();
      if (i + k + 1 >= cnt) {
        last = true;
        break;
      }
    }
    if (last) break;
  }

  {
    float *sp = states + ((int64_t)sw.bh * g.n_seg + sw.seg) * (F * F);
#pragma unroll
    for (int T = 0; T < 2; ++T)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        sp[(64 * rh + 32 * T + 8 * (r >> 2) + 4 * hh + (r & 3)) * F + 32 * wc + c] = st[T][r];
  }
}

template <class E, bool REV, bool TRANS, int SRC, int MODE>
int launch_apply(const void *x, const void *y, const void *z, const float *s, const float *states,
                    const float *carry_in, float *carry_out, void *out, const Geom &g, hipStream_t st) {
  int rc = grant_lds<la_apply<E, REV, TRANS, SRC, MODE>>(WS_LDS);
  if (rc) return rc;
  const unsigned grid = (unsigned)((int64_t)g.b * g.h * g.n_seg);
  ProfScope prof(KC_APPLY, st);
  la_apply<E, REV, TRANS, SRC, MODE><<<grid, WS_THREADS, WS_LDS, st>>>(
      (const elem16_t *)x, (const elem16_t *)y, (const elem16_t *)z, s, states, carry_in, carry_out, (elem16_t *)out, g);
  return (int)hipGetLastError();
}

template <class E, int SRC, int MODE>
int launch_bwd3(const BwdArgs &a, const float *kv_states, const float *dkv_states, const Geom &g,
                   hipStream_t st) {
  int rc = grant_lds<la_bwd3<E, SRC, MODE>>(WS_LDS);
  if (rc) return rc;
  const int64_t n_items = (int64_t)g.b * g.h * g.n_seg;
  const unsigned grid = (unsigned)(((n_items + 7) / 8) * 24);
  ProfScope prof(KC_BWD3, st);
  la_bwd3<E, SRC, MODE><<<grid, WS_THREADS, WS_LDS, st>>>((const elem16_t *)a.q, (const elem16_t *)a.k,
                                                         (const elem16_t *)a.v, (const elem16_t *)a.d_o, a.s,
                                                         kv_states, dkv_states, a.kv_in, a.dkv_in, a.dkv_out,
                                                         (elem16_t *)a.dq, (elem16_t *)a.dk, (elem16_t *)a.dv, g);
  return (int)hipGetLastError();
}

template <class E, bool REV, int MODE, int D>
int launch_state_depth(const void *y, const void *z, const float *s, float *states, const Geom &g, int skip_seg,
                       int sub, hipStream_t st) {
  int rc = grant_lds<la_seg_state<E, REV, MODE, D>>(STATE_LDS);
  if (rc) return rc;
  const unsigned grid = (unsigned)((int64_t)g.b * g.h * g.n_seg);
  ProfScope prof(KC_STATE, st);
  la_seg_state<E, REV, MODE, D><<<grid, STATE_THREADS, STATE_LDS, st>>>((const elem16_t *)y, (const elem16_t *)z, s,
                                                                        states, g, skip_seg, sub);
  return (int)hipGetLastError();
}

// skip_seg: the segment whose own state nothing reads (-1: none); its workgroups leave at once.
// sub: segments of `g` per sweep segment (1 unless the plan cut the sweep segments finer for the pre-pass).
template <class E, bool REV, int MODE>
int launch_state_skipping(const void *y, const void *z, const float *s, float *states, const Geom &g, int skip_seg,
                          hipStream_t st, int sub = 1) {
  return g.seg_len >= STATE_LONG_WALK
             ? launch_state_depth<E, REV, MODE, STATE_DEPTH_LONG>(y, z, s, states, g, skip_seg, sub, st)
             : launch_state_depth<E, REV, MODE, STATE_DEPTH_SHORT>(y, z, s, states, g, skip_seg, sub, st);
}

// carry_wanted: whether the scan that follows has to produce the outgoing carry; if not, the
// segment it visits last (whose own state feeds nothing else) is skipped.
template <class E, bool REV, int MODE>
int launch_state(const void *y, const void *z, const float *s, float *states, const Geom &g,
                 bool carry_wanted, int sub, hipStream_t st) {
  return launch_state_skipping<E, REV, MODE>(y, z, s, states, g, carry_wanted ? -1 : (REV ? 0 : g.n_seg - 1), st, sub);
}

template <class E, int MODE>
int launch_fused_fwd(const FwdArgs &a, const Geom &g, hipStream_t st) {
  int rc = grant_lds<la_fused_fwd<E, MODE>>(WS_LDS);
  if (rc) return rc;
  const unsigned grid = (unsigned)((((int64_t)g.b * g.h + 7) / 8) * 8 * g.n_seg);  // whole groups of 8 (b, h)
  ProfScope prof(KC_FUSED, st);
  la_fused_fwd<E, MODE><<<grid, WS_THREADS, WS_LDS, st>>>((const elem16_t *)a.q, (const elem16_t *)a.k,
                                                         (const elem16_t *)a.v, a.s, a.kv_in, a.kv_out,
                                                         (elem16_t *)a.o, g);
  return (int)hipGetLastError();
}

// The backward's three workgroups per segment should fit the chip in one round (one workgroup per CU), and
// nothing ties its segments to the forward's: no states are handed over on this path.
Geom fused_bwd_geom(const Geom &g) {
  Geom gb = g;
  const int64_t bh = (int64_t)g.b * g.h;
  int64_t fit = 256 / (3 * bh);  // segments per (b, h) in one round
  if (fit < 1) fit = 1;
  if (fit < g.n_seg) {
    int64_t len = (g.n + fit - 1) / fit;
    len = ((len + BLK - 1) / BLK) * BLK;
    gb.seg_len = (int)len;
    gb.n_seg = (int)((g.n + len - 1) / len);
  }
  return gb;
}

template <class E, int MODE>
int launch_fused_bwd(const BwdArgs &a, const Geom &g_fwd, hipStream_t st) {
  int rc = grant_lds<la_fused_bwd<E, MODE>>(WS_LDS);
  if (rc) return rc;
  const Geom g = fused_bwd_geom(g_fwd);
  const unsigned grid = (unsigned)((((int64_t)g.b * g.h + 7) / 8) * 8 * 3 * g.n_seg);
  ProfScope prof(KC_FUSED, st);
  la_fused_bwd<E, MODE><<<grid, WS_THREADS, WS_LDS, st>>>((const elem16_t *)a.q, (const elem16_t *)a.k,
                                                         (const elem16_t *)a.v, (const elem16_t *)a.d_o, a.s,
                                                         a.kv_in, a.dkv_in, a.dkv_out, (elem16_t *)a.dq,
                                                         (elem16_t *)a.dk, (elem16_t *)a.dv, g);
  return (int)hipGetLastError();
}

// The geometry the pre-pass and the scan work on: the chunk cut into g.pre_n segments of g.pre_len tokens
// (the sweeps' own segments unless the plan cut those finer for the pre-pass).
Geom pre_pass_geom(const Geom &g) {
  Geom gp = g;
  gp.seg_len = g.pre_len;
  gp.n_seg = g.pre_n;
  return gp;
}

template <class E, int MODE>
int fwd_e(const FwdArgs &a, const Geom &g, hipStream_t st) {
  if (g.fused) return launch_fused_fwd<E, MODE>(a, g, st);
  int rc;
  if constexpr (MODE != M_NARROW) if (g.combine) {  // (the plan combines full-width heads only)
    // few segments: the pre-pass leaves every segment's own state (the last one's is never read), each
    // sweep workgroup gathers the ones before it, and the last segment's sweep ends with KV_out
    if (g.n_seg > 1 &&
        (rc = launch_state_skipping<E, false, MODE>(a.k, a.v, a.s, a.seg_states, g, g.n_seg - 1, st)))
      return rc;
    return launch_apply<E, false, false, SRC_COMBINE, MODE>(a.q, a.k, a.v, a.s, g.n_seg > 1 ? a.seg_states : nullptr,
                                                               a.kv_in, a.kv_out, a.o, g, st);
  }
  const bool need_states = g.n_seg > 1 || a.kv_in || a.kv_out;
  const Geom gp = pre_pass_geom(g);
  const int sub = g.seg_len / g.pre_len;  // pre-pass segments per sweep segment
  if (need_states) {
    if ((rc = launch_state<E, false, MODE>(a.k, a.v, a.s, a.seg_states, gp, a.kv_out != nullptr, sub, st))) return rc;
    if ((rc = launch_segment_scan(a.seg_states, a.kv_in, a.kv_out, a.s, gp, 0, st))) return rc;
  }
  return launch_apply<E, false, false, SRC_SCANNED, MODE>(a.q, a.k, a.v, a.s, need_states ? a.seg_states : nullptr,
                                                             a.kv_in, nullptr, a.o, g, st);
}

template <class E, int MODE>
int bwd_e(const BwdArgs &a, const Geom &g, hipStream_t st) {
  if (g.fused) return launch_fused_bwd<E, MODE>(a, g, st);
  int rc;
  if constexpr (MODE != M_NARROW) if (g.combine) {
    const float *kv_states = a.kv_seg_states;
    if (!kv_states && g.n_seg > 1) {
      if ((rc = launch_state_skipping<E, false, MODE>(a.k, a.v, a.s, a.ws_kv, g, g.n_seg - 1, st))) return rc;
      kv_states = a.ws_kv;
    }
    if (g.n_seg > 1 && (rc = launch_state_skipping<E, true, MODE>(a.q, a.d_o, a.s, a.ws_dkv, g, 0, st))) return rc;
    return launch_bwd3<E, SRC_COMBINE, MODE>(a, g.n_seg > 1 ? kv_states : nullptr,
                                                g.n_seg > 1 ? a.ws_dkv : nullptr, g, st);
  }
  const Geom gp = pre_pass_geom(g);
  const int sub = g.seg_len / g.pre_len;  // pre-pass segments per sweep segment
  const float *kv_states = a.kv_seg_states;
  if (!kv_states && (g.n_seg > 1 || a.kv_in)) {
    if ((rc = launch_state<E, false, MODE>(a.k, a.v, a.s, a.ws_kv, gp, false, sub, st))) return rc;
    if ((rc = launch_segment_scan(a.ws_kv, a.kv_in, nullptr, a.s, gp, 0, st))) return rc;
    kv_states = a.ws_kv;
  }
  const float *dkv_states = nullptr;
  if (g.n_seg > 1 || a.dkv_in || a.dkv_out) {
    if ((rc = launch_state<E, true, MODE>(a.q, a.d_o, a.s, a.ws_dkv, gp, a.dkv_out != nullptr, sub, st))) return rc;
    if ((rc = launch_segment_scan(a.ws_dkv, a.dkv_in, a.dkv_out, a.s, gp, 1, st))) return rc;
    dkv_states = a.ws_dkv;
  }
  return launch_bwd3<E, SRC_SCANNED, MODE>(a, kv_states, dkv_states, g, st);
}


int mode_of(const Geom &g) {
  if (g.d != F || g.e != F) return M_NARROW;
  return g.n % BLK != 0 ? M_RAGGED : M_ALIGNED;
}

template <class E>
int fwd_m(const FwdArgs &a, const Geom &g, hipStream_t st) {
  switch (mode_of(g)) {
    case M_ALIGNED: return fwd_e<E, M_ALIGNED>(a, g, st);
    case M_RAGGED: return fwd_e<E, M_RAGGED>(a, g, st);
    default: return fwd_e<E, M_NARROW>(a, g, st);
  }
}
template <class E>
int bwd_m(const BwdArgs &a, const Geom &g, hipStream_t st) {
  switch (mode_of(g)) {
    case M_ALIGNED: return bwd_e<E, M_ALIGNED>(a, g, st);
    case M_RAGGED: return bwd_e<E, M_RAGGED>(a, g, st);
    default: return bwd_e<E, M_NARROW>(a, g, st);
  }
}

}  // namespace

int mfma_fwd(const FwdArgs &a, const Geom &g, int dtype, hipStream_t st) {
  return dtype == LASP_DTYPE_F16 ? fwd_m<ElemF16>(a, g, st) : fwd_m<ElemBF16>(a, g, st);
}

int mfma_bwd(const BwdArgs &a, const Geom &g, int dtype, hipStream_t st) {
  return dtype == LASP_DTYPE_F16 ? bwd_m<ElemF16>(a, g, st) : bwd_m<ElemBF16>(a, g, st);
}

}  // namespace lasp
