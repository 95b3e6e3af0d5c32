// C ABI of liblasp_hip.so: argument validation, segment planning and dispatch to
// the kernel families.  Declarations and the tensor contract: include/lasp_hip.h.
#include <stdarg.h>
#include <stdio.h>

#include <atomic>

#include "lasp_common.h"

namespace lasp {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// ---- per-kernel timing -------------------------------------------------------
struct ProfEntry {
  int cls;
  hipEvent_t start, stop;
};
// Launches may come from several threads (PyTorch runs backward on its own thread): a launch
// claims its slot with one atomic increment, and lasp_profile_end only reads slots after the
// profile has been closed to new launches and the claimed ones have recorded their events.
static std::atomic<ProfEntry *> g_prof{nullptr};  // non-NULL while a profile is open
static std::atomic<int> g_prof_used{0};           // slots claimed (may run past the capacity)
static std::atomic<int> g_prof_busy{0};           // launches between claiming a slot and recording its stop event
static int g_prof_cap = 0;

ProfScope::ProfScope(int kernel_class, hipStream_t st) : slot(-1), entry(nullptr), stream(st) {
  if (!g_prof.load(std::memory_order_acquire)) return;
  g_prof_busy.fetch_add(1, std::memory_order_acq_rel);
  ProfEntry *p = g_prof.load(std::memory_order_acquire);  // re-read: the profile may have closed meanwhile
  const int claimed = p ? g_prof_used.fetch_add(1, std::memory_order_acq_rel) : -1;
  if (!p || claimed >= g_prof_cap) {
    g_prof_busy.fetch_sub(1, std::memory_order_acq_rel);
    return;
  }
  slot = claimed;
  entry = p + slot;
  entry->cls = kernel_class;
  (void)hipEventRecord(entry->start, stream);
}
ProfScope::~ProfScope() {
  if (slot < 0) return;
  (void)hipEventRecord(entry->stop, stream);
  g_prof_busy.fetch_sub(1, std::memory_order_acq_rel);
}

namespace {

constexpr int kMaxFeature = 128;     // d and e of one launch (the Python wrappers slice d, as
                                     // lasp/lightning_attention.py:513-519 does)
constexpr int kSegQuantum = 64;      // segment lengths are multiples of this
constexpr int64_t kTargetGroups = 512;  // workgroups wanted per launch (2 per CU on 256 CUs)
constexpr int kMinSeg = 256;
constexpr int kPreferredSeg = 1024;     // preferred lower bound while kMinGroups workgroups remain
constexpr int64_t kMinGroups = 256;     // one workgroup per CU
constexpr int64_t kMaxSeg = 1 << 24;    // offsets inside a segment stay within 32 bits
constexpr int kLongestPlanned = 4352;   // longest segment the refined default plan picks (4096 tokens and a little more)
constexpr int kPreMaxSeg = 2304;        // longest segment the pre-pass walks in one workgroup (see make_geom):
                                        // 2048 tokens and a little more, so that lengths just above 4096, 8192, ...
                                        // are still cut in 2, 4, ... and not in twice as many pieces

int check_shape(int b, int h, int64_t n, int d, int e, int dtype) {
  if (dtype != LASP_DTYPE_F32 && dtype != LASP_DTYPE_BF16 && dtype != LASP_DTYPE_F16) {
    set_error("unknown dtype code %d", dtype);
    return LASP_E_DTYPE;
  }
  if (b <= 0 || h <= 0 || n <= 0 || d <= 0 || e <= 0 || d > kMaxFeature || e > kMaxFeature) {
    set_error("unsupported shape b=%d h=%d n=%lld d=%d e=%d (need b,h,n >= 1 and 1 <= d,e <= %d)", b,
              h, (long long)n, d, e, kMaxFeature);
    return LASP_E_SHAPE;
  }
  if ((int64_t)b * h > (int64_t)1 << 24) {
    set_error("b*h = %lld is too large", (long long)b * h);
    return LASP_E_SHAPE;
  }
  return 0;
}

int default_seg_len(int b, int h, int64_t n) {
  const int64_t bh = (int64_t)b * h;
  const int64_t want = (kTargetGroups + bh - 1) / bh;  // segments per (b, h)
  // rounded up, so that no more than `want` segments result: one workgroup more than the chip
  // holds at once would cost a second pass over the CUs
  int64_t len = (n + want - 1) / want;
  len = ((len + kMinSeg - 1) / kMinSeg) * kMinSeg;
  // Segments shorter than kPreferredSeg spend a visible share of their time on the 64 KiB
  // state each one loads and the scan has to carry; one workgroup per CU of longer
  // segments measured faster than two of shorter ones.
  if (len < kPreferredSeg && bh * ((n + kPreferredSeg - 1) / kPreferredSeg) >= kMinGroups)
    len = kPreferredSeg;
  // Small problems that leave the chip under-filled even in the backward sweep (three workgroups per
  // segment) run 5-13 % faster on 3-block segments than on 4-block ones: more workgroups, each with a
  // shorter serial walk (b*h = 12, n = 2048: 60 against 67 us forward + backward; b*h = 6, n = 4096:
  // 62 against 71).  Not for one or two (b, h) pairs, where the longer scan costs more than that, and
  // not for chunks short enough for the single-launch kernels, whose choice this must not disturb.
  // Only where the shorter segments do not cost the backward sweep (one workgroup per CU) another round:
  // b*h = 4, n = 4096: 22 segments of 192 tokens are 264 workgroups, 56 us against 51 for 16 of 256; b*h = 8,
  // n = 2048: 52 against 49; b*h = 6, n = 3072: 54 against 52 -- and the other way round wherever the rounds
  // stay the same (b*h = 3 ... 14, n = 2048 ... 4096: 2-6 us faster on 192).
  constexpr int kShortSeg = 3 * kSegQuantum;
  auto bwd_rounds = [&](int64_t l) { return (3 * bh * ((n + l - 1) / l) + kMinGroups - 1) / kMinGroups; };
  if (len == kMinSeg && bh >= 3 && n > 3 * kMinSeg && 3 * bh * ((n + kShortSeg - 1) / kShortSeg) <= kTargetGroups &&
      bwd_rounds(kShortSeg) <= bwd_rounds(kMinSeg))
    len = kShortSeg;
  // The backward sweep runs three workgroups per segment.  When those exceed what the chip holds at
  // once by a little (up to a quarter), the stragglers cost it a second round; segments up to two
  // blocks longer that bring the count back within one round measured 6 % faster (b*h = 24, n = 2048:
  // 7 segments of 320 tokens, 80 us forward + backward, against 8 of 256, 85 us).
  if (len < kPreferredSeg) {
    const int64_t groups = 3 * bh * ((n + len - 1) / len);
    const int64_t fit = kTargetGroups / (3 * bh);  // segments per (b, h) that fit in one round
    if (groups > kTargetGroups && groups <= kTargetGroups + kTargetGroups / 4 && fit >= 1) {
      int64_t longer = (n + fit - 1) / fit;
      longer = ((longer + kSegQuantum - 1) / kSegQuantum) * kSegQuantum;
      if (longer <= len + 2 * kSegQuantum) len = longer;
    }
  }
  // One or two (b, h) pairs cannot fill the chip with segments of 256 tokens and more; there the sweeps (serial in
  // the blocks of a segment) are traded against the scan (serial in the segments): about 2 sqrt(n) tokens per
  // segment.  Forward + backward, b*h = 1: n = 32768, 64 segments of 512 tokens 81 us against 93 for 128 of 256;
  // n = 65536: 120 for 128 of 512 against 148; n = 131072: 177 for 128 of 1024 against 190 for 256 of 512 and 203
  // for 64 of 2048; n = 262144: 291 for 256 of 1024 against 307 for 128 of 2048; b*h = 2, n = 32768: 104 against 117.
  int64_t balanced = kMinSeg;
  while (balanced * balanced < 4 * n) balanced *= 2;
  if (balanced > kMinSeg && balanced > len && bh * ((n + balanced - 1) / balanced) <= kMinGroups) len = balanced;
  if (len > kMaxSeg) len = kMaxSeg;
  return (int)len;
}

// The 16-bit MFMA kernels work on 128 features and read narrower rows zero-extended; their
// 8-byte loads and 16-byte stores need every row to start on such a boundary.
bool mfma_eligible(int d, int e, int dtype) {
  return (dtype == LASP_DTYPE_BF16 || dtype == LASP_DTYPE_F16) && d % 8 == 0 && e % 8 == 0;
}
bool mfma_f32_eligible(int d, int e, int dtype) {
  return dtype == LASP_DTYPE_F32 && d == kMaxFeature && e == kMaxFeature;
}

// Short chunks given to the library with the default plan run as ONE launch per direction: every
// workgroup rebuilds the state entering its segment by walking the blocks before it, which saves
// the pre-pass, its launch and the workspace.  The walk is serial work on the critical path (0.7 us
// per 64-token block: the math waves multiply a block into the state while the feed waves fetch and
// transpose the next one), and the single launch wins up to walks of about 16 blocks.  Forward +
// backward replayed from a graph over rotating inputs, scan path against single launch: b*h = 24:
// n = 512 44 / 33 us, 768 48 / 40, 1024 59 / 46, 1536 70 / 69, 2048 81 / 87; b*h = 128, n = 1024:
// 172 / 133; b*h = 16, n = 2048: 66 / 76; b*h = 4, n = 2048: 45 / 70.  An explicit seg_len always
// selects the pre-pass / sweep kernels.
constexpr int64_t kFusedMaxTokens = 2048;
constexpr int kFusedMaxWalk = 16;  // blocks
// With few segments the 16-bit sweeps of full-width heads gather the segments' own states themselves
// (each workgroup re-runs the scan's recurrence over at most kCombineMaxSeg - 1 states of 64 KiB)
// and the scan launch is dropped; with one segment the pre-pass goes too.  Measured at b*h = 24,
// n = 2048: 4 segments 84 against 88 us forward + backward, 8 segments 137 against 100 us (the
// gathers grow with the square of the segment count), hence the limit.  The sweeps gather only as far back as a
// head's decay reaches, and while their feed waves fetch the first block; at 7 segments that still
// costs what the scan launch saves (b*h = 24, n = 2048: 67 against 69 us per chunk in kernels, 691 against 677 us
// for the 8-chunk chain replayed from a graph), so the limit stays.
constexpr int64_t kCombineMaxSeg = 4;
bool fused_eligible(int64_t n, int d, int e, int dtype, int seg_len_arg, int seg_len, int64_t n_seg) {
  if (seg_len_arg != 0 || !mfma_eligible(d, e, dtype) || n > kFusedMaxTokens) return false;
  const int per_seg = seg_len / kSegQuantum;  // blocks in one segment's sweep
  return (n_seg - 1) * per_seg <= kFusedMaxWalk;
}

// Default segment length of the fp32 MFMA kernels and the generic kernels, which run two (or more) workgroups
// per CU and are bound by arithmetic: what counts is that every CU gets the same number of workgroups.  Of the
// power-of-two lengths that give the forward sweep at least one workgroup per CU, the one with the smallest
// load per CU -- ceil(workgroups / 256) x (seg_len + 64 tokens for the state each workgroup loads and leaves) --
// is taken, longer segments (fewer states to scan) winning ties; a single segment of 1024 tokens or more is
// then cut in two when the chunk has more than one, because two workgroups on a CU fill each other's waits.
// Measured forward + backward in fp32, d = e = 128, this rule against the one of the 16-bit sweeps:
// b*h = 24, n = 16384: 512 tokens, 1555 us against 1783 (1024: 384 workgroups, half the CUs with two);
// b*h = 4, n = 8192: 128 tokens, 181 against 231; b*h = 8, n = 4096: 128, 173 against 228; b*h = 16, n = 1024:
// 64, 108 against 176; b*h = 1, n = 8192: 64, 109 against 179; b*h = 24, n = 2048: 128, 272 against 280; equal
// within 3 % on the other shapes tried (b*h = 1 ... 256, n = 1024 ... 262144).
int two_per_cu_seg_len(int b, int h, int64_t n) {
  const int64_t bh = (int64_t)b * h;
  auto groups = [&](int64_t len) { return bh * ((n + len - 1) / len); };
  int64_t best = kSegQuantum, best_load = -1;
  for (int64_t len = kSegQuantum; len <= kMaxSeg; len *= 2) {
    if (groups(len) < kMinGroups && len > kSegQuantum) break;  // (the shortest length stands where nothing fills the chip)
    const int64_t load = ((groups(len) + kMinGroups - 1) / kMinGroups) * (len + kSegQuantum);
    if (best_load < 0 || load <= best_load) {
      best = len;
      best_load = load;
    }
    if (len >= n) break;
  }
  if (best >= kPreferredSeg && best < n && groups(best) <= kMinGroups) best /= 2;
  return (int)best;
}

int make_geom(int b, int h, int64_t n, int d, int e, int dtype, int seg_len, Geom *g) {
  int rc = check_shape(b, h, n, d, e, dtype);
  if (rc) return rc;
  const int seg_len_arg = seg_len;
  if (seg_len == 0) seg_len = mfma_eligible(d, e, dtype) ? default_seg_len(b, h, n) : two_per_cu_seg_len(b, h, n);
  if (seg_len < 0 || seg_len % kSegQuantum != 0) {
    set_error("seg_len=%d must be a positive multiple of %d (or 0 for the default)", seg_len,
              kSegQuantum);
    return LASP_E_SEGMENT;
  }
  const int64_t n_seg = (n + seg_len - 1) / seg_len;
  if (n_seg > (1 << 20) || (int64_t)b * h * n_seg > (int64_t)1 << 30) {
    set_error("too many segments (%lld) for seg_len=%d", (long long)n_seg, seg_len);
    return LASP_E_SEGMENT;
  }
  const bool sweeps16 = mfma_eligible(d, e, dtype) && !fused_eligible(n, d, e, dtype, seg_len_arg, seg_len, n_seg);
  if (sweeps16 && seg_len_arg == 0) {
    // The 16-bit sweeps hold a CU each, so the default plan aims at one round of 256 workgroups in the
    // forward sweep rather than two per CU: longer segments mean fewer states to load and carry (b*h = 16,
    // n = 65536: 4096-token segments, sweeps 193 + 496 us against 201 + 513 with 2048; b*h = 32, n = 16384:
    // 2048 against 1024, 97 + 248 against 102 + 256).
    while (n_seg > kCombineMaxSeg && (int64_t)b * h * ((n + 2 * seg_len - 1) / (2 * seg_len)) >= kMinGroups &&
           (n + 2 * seg_len - 1) / (2 * seg_len) > kCombineMaxSeg)
      seg_len *= 2;
    // That leaves between one and two rounds of workgroups, and a round that is only part full costs a whole
    // round's time.  So the plan is refined: of the segment counts that fill r = 1, 2, ... rounds of the forward
    // sweep (floor(256 r / (b*h)) segments per (b, h), the segments stretched to cover the chunk) and give
    // segments of 1024 to about 4096 tokens, the one that keeps the most CUs busy -- fill of the last round,
    // times the share of a full segment that the chunk's last segment has, times the share of a workgroup's time
    // that goes into blocks -- is taken, fewer rounds winning ties.  Measured forward + backward, this plan
    // against the power-of-two one: b*h = 24, n = 16384: 10 segments of 1664 tokens, 334 us against 356;
    // b*h = 24, n = 32768: 647 against 742 (11 segments of 3072 = 264 workgroups); b*h = 28, n = 65536: 18 of
    // 3648, 1444 against 1493; b*h = 48, n = 65536: 16 of 4096, 2386 against 2715; b*h = 100, n = 8192: 5 of
    // 1664, 663 against 733.  In a one-round plan lengths beyond 2048 tokens stay a multiple of 64 * 2^k with
    // seg_len / 2^k <= kPreMaxSeg, so that the pre-pass can work on equal pieces of that length.
    const int64_t bh = (int64_t)b * h;
    double best = 0.0;
    int best_len = 0;
    const bool over_one_round = bh * ((n + seg_len - 1) / seg_len) > kMinGroups;
    for (int r = 1; r <= 16 && over_one_round; ++r) {
      const int64_t fit = kMinGroups * r / bh;  // segments per (b, h) in r rounds
      // With many (b, h) pairs one round means 2 to 4 segments, which full-width heads sweep without a scan
      // launch; taken while the segments stay within 1024 tokens, i.e. while the pre-pass's walks stay short
      // (b*h = 56, n = 2048: 4 segments of 512 tokens, 114 us forward + backward against 151 for 8 of 256;
      // b*h = 64, n = 3072: 4 of 768, 161 against 200; b*h = 60, n = 4096: 4 of 1024, 203 against 234; but
      // b*h = 52, n = 8192: 4 of 2048, 384 against 363 for 8 of 1024).
      // Where such a plan fills the chip to 7/8 and more it is taken up to 2048 tokens and over two rounds as well
      // (b*h = 64, n = 8192: 4 of 2048, 413 us against 438 for 8 of 1024; b*h = 128, n = 4096: 2 of 2048, 408
      // against 430; b*h = 128, n = 8192: 4 of 2048 in two rounds, 808 against 860 for 6 of 1408 in three; b*h = 120, n = 4096: 2 of 2048, 394 against 411; but b*h = 52, n = 8192,
      // 208 of 256 CUs: 380 against 360).
      const bool few = fit <= kCombineMaxSeg;
      const bool few_fills = few && bh * fit * 8 >= kMinGroups * r * 7;
      if (few && (fit < 2 || r > (few_fills ? 2 : 1) || d != kMaxFeature || e != kMaxFeature)) continue;
      const int64_t len = (n + fit - 1) / fit;
      int64_t stretched = 0;
      if (r > 1) {  // (more than one round: the pre-pass takes whole segments, see pre_len below)
        stretched = ((len + kSegQuantum - 1) / kSegQuantum) * kSegQuantum;
      } else {
        for (int k = 0; k < 16 && !stretched; ++k) {
          const int64_t gran = (int64_t)kSegQuantum << k;
          const int64_t cand = ((len + gran - 1) / gran) * gran;
          if ((cand >> k) <= kPreMaxSeg) stretched = cand;
        }
      }
      // one round may be had with segments as short as any plan's (b*h = 24, n = 4096: 10 of 448 tokens, 118 us
      // forward + backward against 138 for 16 of 256; n = 8192: 10 of 832, 172 against 199; b*h = 40, n = 4096:
      // 6 of 704, 151 against 166); several rounds only pay with long segments
      if (stretched < (r == 1 ? kMinSeg : kPreferredSeg)) break;  // more rounds only make the segments shorter
      if (stretched > (few ? (few_fills ? 2 * kPreferredSeg : kPreferredSeg) : kLongestPlanned)) continue;
      const int64_t segs = (n + stretched - 1) / stretched;
      const int64_t groups = bh * segs;
      const double fill = (double)groups / (double)(kMinGroups * ((groups + kMinGroups - 1) / kMinGroups));
      const double blocks = (double)stretched / kSegQuantum;
      // (a workgroup spends about two blocks' time on its start-up and the state it loads)
      const double score = fill * (double)n / (double)(segs * stretched) * blocks / (blocks + 2.0);
      if (score > best + 0.02) {
        best = score;
        best_len = (int)stretched;
      }
    }
    if (best_len) seg_len = best_len;
    // The backward sweep runs three workgroups per segment.  With short segments in one forward round that is at least three quarters full, a few
    // longer ones that save the backward a round are worth it: (1 + rounds) x (blocks + 3) is what a chunk costs,
    // 3 blocks standing for a workgroup's start-up and state traffic (b*h = 24, n = 4096: 7 segments of 640
    // tokens, 106 us forward + backward against 112 for 10 of 448; b*h = 12, n = 8192: 13 of 640, 108 against 112).
    // The longer segments win while they stay below about 10 blocks; beyond that the rounds saved cost more in
    // the forward sweep than they bring (b*h = 24, n = 8192: 10 of 832, 168 against 179 for 7 of 1216).
    // With the forward round less than three quarters full the outcome is mixed (half full: b*h = 2, n = 16384, 70 us
    // against 78, but b*h = 6, n = 6144, 79 against 67), so those plans stay.
    {
      const int64_t segs = (n + seg_len - 1) / seg_len;
      const int64_t rounds = (3 * bh * segs + kMinGroups - 1) / kMinGroups;
      const int64_t fewer = rounds >= 2 ? kMinGroups * (rounds - 1) / (3 * bh) : 0;  // segments per (b, h)
      if (bh * segs <= kMinGroups && bh * segs * 4 >= kMinGroups * 3 && fewer > kCombineMaxSeg && fewer < segs) {
        int64_t longer = (n + fewer - 1) / fewer;
        longer = ((longer + kSegQuantum - 1) / kSegQuantum) * kSegQuantum;
        const int64_t cost_now = (1 + rounds) * (seg_len / kSegQuantum + 3);
        const int64_t cost_longer = rounds * (longer / kSegQuantum + 3);
        if (longer <= kPreMaxSeg && cost_longer < cost_now) seg_len = (int)longer;
      }
    }
  }
  const int64_t n_seg_final = (n + seg_len - 1) / seg_len;
  g->b = b;
  g->h = h;
  g->n = n;
  g->d = d;
  g->e = e;
  g->seg_len = seg_len;
  g->n_seg = (int)n_seg_final;
  g->fused = fused_eligible(n, d, e, dtype, seg_len_arg, seg_len, n_seg_final) ? 1 : 0;
  g->combine = (!g->fused && mfma_eligible(d, e, dtype) && d == kMaxFeature && e == kMaxFeature &&
                n_seg_final <= kCombineMaxSeg) ? 1 : 0;
  // heads whose state dies within a segment skip the scan (16-bit MFMA kernels on the pre-pass / scan / sweep path)
  g->bypass = (mfma_eligible(d, e, dtype) && !g->fused && !g->combine && n_seg_final >= 2) ? 1 : 0;
  // The pre-pass walks a segment serially, and its slow-decay heads walk all of it: beyond 2048 tokens that
  // walk outlasts everything else in the launch (b*h = 16, n = 65536: 71 us at 4096 tokens against 51 at
  // 2048; at 1024 the extra states cost more again, 62 us and a longer scan).  Long sweep segments are
  // therefore cut in halves (quarters, ...) for the pre-pass and the scan, and a sweep takes the state that
  // enters its first piece.  A pure function of the shape and seg_len, so that a backward call given the
  // forward's seg_len finds the states where the forward left them.
  g->pre_len = seg_len;
  // Only while the chip is not full, though: with more pre-pass workgroups than CUs the long walks overlap with
  // other workgroups, and whole segments measured 1-3 % faster in all (b*h = 28, n = 65536, 18 segments of 3648
  // tokens: 1440 us forward + backward against 1484 with halves; b*h = 48, 16 of 4096: 2377 against 2423; at
  // b*h = 16 and 24, 256 and 240 workgroups, the halves win: 838 against 856, 653 against 663).
  if (mfma_eligible(d, e, dtype) && !g->combine && !g->fused && (int64_t)b * h * n_seg_final <= kMinGroups) {
    int pre = seg_len;
    while (pre > kPreMaxSeg && pre % (2 * kSegQuantum) == 0) pre /= 2;
    if (pre <= kPreMaxSeg) g->pre_len = pre;
  }
  g->pre_n = (int)((n + g->pre_len - 1) / g->pre_len);
  const bool padded_states = mfma_eligible(d, e, dtype) || mfma_f32_eligible(d, e, dtype);
  g->sd = padded_states ? kMaxFeature : d;
  g->se = padded_states ? kMaxFeature : e;
  return 0;
}

// The kernels fetch rows of q/k/v/do with 8-byte loads and store o/dq/dk/dv with 16-byte stores,
// and read states as floats: tensors must start on a 16-byte boundary, states on a 4-byte one.
int check_aligned(const char *call, const char *name, const void *p, size_t align) {
  if (p && ((uintptr_t)p % align) != 0) {
    set_error("%s: %s = %p is not aligned to %zu bytes", call, name, p, align);
    return LASP_E_ALIGN;
  }
  return 0;
}

// The calling thread's current device must be the one that owns the tensors (checked on q).
int check_device(const char *call, const void *q) {
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, q);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // the failed query must not be reported by a later launch
    set_error("%s: q = %p is not a device pointer known to HIP (%s)", call, q, hipGetErrorString(e));
    return LASP_E_DEVICE;
  }
  int dev = -1;
  e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (attr.type != hipMemoryTypeDevice || attr.device != dev) {
    set_error("%s: q = %p lives on device %d (memory type %d) but the calling thread's current device is %d",
              call, q, attr.device, (int)attr.type, dev);
    return LASP_E_DEVICE;
  }
  return 0;
}

// In-place state update (out == in).  The scan kernel reads the incoming carry and writes the
// outgoing one from the same thread, and for the heads it leaves out it parks the incoming carry in
// the workspace, where the sweeps take it from; so the pre-pass / scan / sweep path takes it.  On the paths
// where the sweeps combine the states themselves every workgroup of a (b, h) reads the incoming
// state when it starts and one of them writes the outgoing state when it ends; nothing orders a
// late starter against an early finisher, so in place is only safe when one workgroup does both.
bool inplace_ok(const Geom &g, bool backward) {
  if (!g.fused && !g.combine) return true;
  return !backward && g.n_seg == 1;  // backward: the dV workgroup writes what the dK workgroup reads
}

// `in` and `out` are states of `bytes` bytes each.
int check_alias(const char *call, const char *what, const float *in, const float *out, size_t bytes, const Geom &g,
                bool backward) {
  if (!in || !out) return 0;
  const uintptr_t a = (uintptr_t)in, b = (uintptr_t)out;
  if (a + bytes <= b || b + bytes <= a) return 0;  // disjoint
  if (a != b) {
    set_error("%s: %s_out = %p overlaps %s_in = %p without being the same buffer", call, what, (const void *)out,
              what, (const void *)in);
    return LASP_E_ALIAS;
  }
  if (!inplace_ok(g, backward)) {
    set_error("%s: %s_out is %s_in, but this shape runs kernels in which one workgroup writes the outgoing state "
              "while others may still have to read the incoming one (see lasp_inplace_ok); pass a copy as %s_in",
              call, what, what, what);
    return LASP_E_ALIAS;
  }
  return 0;
}

// ---- segment-state scratch owned by the library (lasp_chunk_fwd_static) ------------------------
// Lives in the code object: every device the library runs on holds its own copy, at its own
// address, until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress -- the device address it returns (kept per device below) is what goes
// into kernel arguments.
static __device__ __align__(256) __attribute__((used)) float scratch[LASP_STATIC_SCRATCH_BYTES / sizeof(float)];

constexpr int kMaxDevices = 64;
static std::atomic<float *> g_scratch_ptr[kMaxDevices];  // zero-initialised: not looked up yet

// Device address of `scratch` on the calling thread's current device (looked up once per device).
int static_scratch(float **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("lasp_chunk_fwd_static: hipGetDevice failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    set_error("lasp_chunk_fwd_static: device ordinal %d is outside the supported range 0..%d", dev, kMaxDevices - 1);
    return LASP_E_DEVICE;
  }
  float *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    void *sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !sym) {
      set_error("lasp_chunk_fwd_static: hipGetSymbolAddress(scratch) failed on device %d: %s", dev,
                hipGetErrorString(e));
      return e != hipSuccess ? (int)e : LASP_E_DEVICE;
    }
    p = (float *)sym;
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing threads store the same address
  }
  *out = p;
  return 0;
}

size_t state_bytes_of(const Geom &g) {
  return sizeof(float) * (size_t)g.b * g.h * g.pre_n * g.sd * g.se;
}

}  // namespace
}  // namespace lasp

using namespace lasp;

extern "C" {

int lasp_abi_version(void) { return LASP_ABI_VERSION; }

const char *lasp_last_error(void) { return g_err; }

int lasp_profile_begin(int max_launches) {
  if (g_prof.load()) {
    set_error("lasp_profile_begin: a profile is already open");
    return LASP_E_SHAPE;
  }
  if (max_launches <= 0 || max_launches > (1 << 20)) {
    set_error("lasp_profile_begin: max_launches=%d out of range", max_launches);
    return LASP_E_SHAPE;
  }
  ProfEntry *p = new ProfEntry[max_launches];
  for (int i = 0; i < max_launches; ++i) {
    hipError_t e1 = hipEventCreate(&p[i].start), e2 = hipEventCreate(&p[i].stop);
    if (e1 != hipSuccess || e2 != hipSuccess) {
      if (e1 == hipSuccess) (void)hipEventDestroy(p[i].start);
      if (e2 == hipSuccess) (void)hipEventDestroy(p[i].stop);
      for (int j = 0; j < i; ++j) {
        (void)hipEventDestroy(p[j].start);
        (void)hipEventDestroy(p[j].stop);
      }
      delete[] p;
      set_error("lasp_profile_begin: hipEventCreate failed");
      return (int)(e1 != hipSuccess ? e1 : e2);
    }
  }
  g_prof_cap = max_launches;
  g_prof_used.store(0);
  g_prof.store(p, std::memory_order_release);
  return 0;
}

int lasp_profile_end(double *ms_per_class, int *launches_per_class) {
  ProfEntry *p = g_prof.exchange(nullptr, std::memory_order_acq_rel);
  if (!p) {
    set_error("lasp_profile_end: no profile is open");
    return LASP_E_SHAPE;
  }
  while (g_prof_busy.load(std::memory_order_acquire) > 0) {
  }  // a launch on another thread is between its two event records
  const int used = g_prof_used.load() < g_prof_cap ? g_prof_used.load() : g_prof_cap;
  for (int c = 0; c < KC_COUNT; ++c) {
    if (ms_per_class) ms_per_class[c] = 0.0;
    if (launches_per_class) launches_per_class[c] = 0;
  }
  int rc = 0;
  for (int i = 0; i < used; ++i) {
    float ms = 0.f;
    hipError_t e = hipEventSynchronize(p[i].stop);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, p[i].start, p[i].stop);
    if (e != hipSuccess) rc = (int)e;
    if (ms_per_class) ms_per_class[p[i].cls] += ms;
    if (launches_per_class) launches_per_class[p[i].cls] += 1;
  }
  for (int i = 0; i < g_prof_cap; ++i) {
    (void)hipEventDestroy(p[i].start);
    (void)hipEventDestroy(p[i].stop);
  }
  delete[] p;
  g_prof_cap = 0;
  g_prof_used.store(0);
  if (rc) set_error("lasp_profile_end: HIP error %d: %s", rc, hipGetErrorString((hipError_t)rc));
  return rc;
}

int lasp_plan(int b, int h, int64_t n, int d, int e, int dtype, int seg_len_or_0, int *seg_len,
              int *n_seg, size_t *state_bytes) {
  Geom g;
  int rc = make_geom(b, h, n, d, e, dtype, seg_len_or_0, &g);
  if (rc) return rc;
  if (seg_len) *seg_len = g.seg_len;
  if (n_seg) *n_seg = g.n_seg;
  if (state_bytes) *state_bytes = state_bytes_of(g);
  return 0;
}

int lasp_kernel_path(int b, int h, int64_t n, int d, int e, int dtype) {
  Geom g;
  int rc = make_geom(b, h, n, d, e, dtype, 0, &g);
  if (rc) return rc;
  if (g.fused) return LASP_PATH_MFMA_FUSED;
  return (mfma_eligible(d, e, dtype) || mfma_f32_eligible(d, e, dtype)) ? LASP_PATH_MFMA : LASP_PATH_GENERIC;
}

int lasp_inplace_ok(int b, int h, int64_t n, int d, int e, int dtype, int seg_len, int backward) {
  Geom g;
  int rc = make_geom(b, h, n, d, e, dtype, seg_len, &g);
  if (rc) return rc;
  return inplace_ok(g, backward != 0) ? 1 : 0;
}

static int chunk_fwd_impl(const char *me, const void *q, const void *k, const void *v, const float *s,
                          const float *kv_in, float *kv_out, void *o, float *seg_states, const Geom &g,
                          int dtype, void *stream) {
  int rc;
  if ((rc = check_alias(me, "kv", kv_in, kv_out, sizeof(float) * (size_t)g.b * g.h * g.d * g.e, g, false))) return rc;
  if ((rc = check_aligned(me, "q", q, 16)) || (rc = check_aligned(me, "k", k, 16)) ||
      (rc = check_aligned(me, "v", v, 16)) || (rc = check_aligned(me, "o", o, 16)) ||
      (rc = check_aligned(me, "s", s, 4)) || (rc = check_aligned(me, "kv_in", kv_in, 4)) ||
      (rc = check_aligned(me, "kv_out", kv_out, 4)) || (rc = check_aligned(me, "seg_states", seg_states, 4)))
    return rc;
  if ((rc = check_device(me, q))) return rc;
  (void)hipGetLastError();  // an earlier, unrelated error of this thread is not this call's
  FwdArgs a{q, k, v, s, kv_in, kv_out, o, seg_states};
  hipStream_t st = (hipStream_t)stream;
  rc = mfma_eligible(g.d, g.e, dtype)       ? mfma_fwd(a, g, dtype, st)
       : mfma_f32_eligible(g.d, g.e, dtype) ? mfma_f32_fwd(a, g, st)
                                            : generic_fwd(a, g, dtype, st);
  if (rc > 0) set_error("%s: HIP error %d: %s", me, rc, hipGetErrorString((hipError_t)rc));
  return rc;
}

int lasp_chunk_fwd(const void *q, const void *k, const void *v, const float *s, const float *kv_in,
                   float *kv_out, void *o, float *seg_states, int b, int h, int64_t n, int d, int e,
                   int dtype, int seg_len, void *stream) {
  Geom g;
  int rc = make_geom(b, h, n, d, e, dtype, seg_len, &g);
  if (rc) return rc;
  if (!q || !k || !v || !s || !o) {
    set_error("lasp_chunk_fwd: q, k, v, s and o must not be NULL");
    return LASP_E_NULL;
  }
  if (!g.fused && !seg_states && (g.n_seg > 1 || (!g.combine && (kv_in || kv_out)))) {
    set_error("lasp_chunk_fwd: seg_states workspace (%zu bytes) is required for n_seg=%d%s",
              state_bytes_of(g), g.n_seg, (kv_in || kv_out) ? " with KV in/out" : "");
    return LASP_E_WORKSPACE;
  }
  return chunk_fwd_impl("lasp_chunk_fwd", q, k, v, s, kv_in, kv_out, o, seg_states, g, dtype, stream);
}

int lasp_chunk_fwd_static(const void *q, const void *k, const void *v, const float *s, const float *kv_in,
                          float *kv_out, void *o, int b, int h, int64_t n, int d, int e, int dtype,
                          int seg_len, void *stream) {
  Geom g;
  int rc = make_geom(b, h, n, d, e, dtype, seg_len, &g);
  if (rc) return rc;
  if (!q || !k || !v || !s || !o) {
    set_error("lasp_chunk_fwd_static: q, k, v, s and o must not be NULL");
    return LASP_E_NULL;
  }
  if (!g.fused && state_bytes_of(g) > (size_t)LASP_STATIC_SCRATCH_BYTES) {
    set_error("lasp_chunk_fwd_static: the segment states of this call take %zu bytes (b*h*n_seg = %lld states), "
              "the library's scratch holds %zu; pass a larger seg_len or use lasp_chunk_fwd with a workspace",
              state_bytes_of(g), (long long)g.b * g.h * g.n_seg, (size_t)LASP_STATIC_SCRATCH_BYTES);
    return LASP_E_WORKSPACE;
  }
  float *states = nullptr;
  if ((rc = static_scratch(&states))) return rc;
  // every state the kernels read from the scratch is one they wrote earlier in this same call, so
  // nothing needs clearing between calls
  return chunk_fwd_impl("lasp_chunk_fwd_static", q, k, v, s, kv_in, kv_out, o, states, g, dtype, stream);
}

int lasp_chunk_bwd(const void *q, const void *k, const void *v, const float *s, const void *d_o,
                   const float *kv_in, const float *dkv_in, void *dq, void *dk, void *dv,
                   float *dkv_out, const float *kv_seg_states, float *workspace,
                   size_t workspace_bytes, int b, int h, int64_t n, int d, int e, int dtype,
                   int seg_len, void *stream) {
  Geom g;
  int rc = make_geom(b, h, n, d, e, dtype, seg_len, &g);
  if (rc) return rc;
  if (!q || !k || !v || !s || !d_o || !dq || !dk || !dv) {
    set_error("lasp_chunk_bwd: q, k, v, s, do, dq, dk and dv must not be NULL");
    return LASP_E_NULL;
  }
  const size_t one = state_bytes_of(g);
  const bool need_kv = !g.fused && !kv_seg_states && (g.n_seg > 1 || (!g.combine && kv_in));
  const bool need_dkv = !g.fused && (g.n_seg > 1 || (!g.combine && (dkv_in || dkv_out)));
  const size_t need = one * ((need_kv ? 1 : 0) + (need_dkv ? 1 : 0));
  if (need && (!workspace || workspace_bytes < need)) {
    set_error("lasp_chunk_bwd: workspace of %zu bytes required, got %zu", need,
              workspace ? workspace_bytes : (size_t)0);
    return LASP_E_WORKSPACE;
  }
  const char *me = "lasp_chunk_bwd";
  if ((rc = check_alias(me, "dkv", dkv_in, dkv_out, sizeof(float) * (size_t)b * h * d * e, g, true))) return rc;
  if ((rc = check_aligned(me, "q", q, 16)) || (rc = check_aligned(me, "k", k, 16)) ||
      (rc = check_aligned(me, "v", v, 16)) || (rc = check_aligned(me, "do", d_o, 16)) ||
      (rc = check_aligned(me, "dq", dq, 16)) || (rc = check_aligned(me, "dk", dk, 16)) ||
      (rc = check_aligned(me, "dv", dv, 16)) || (rc = check_aligned(me, "s", s, 4)) ||
      (rc = check_aligned(me, "kv_in", kv_in, 4)) || (rc = check_aligned(me, "dkv_in", dkv_in, 4)) ||
      (rc = check_aligned(me, "dkv_out", dkv_out, 4)) ||
      (rc = check_aligned(me, "kv_seg_states", kv_seg_states, 4)) ||
      (rc = check_aligned(me, "workspace", workspace, 4)))
    return rc;
  if ((rc = check_device(me, q))) return rc;
  (void)hipGetLastError();  // an earlier, unrelated error of this thread is not this call's
  BwdArgs a{q,  k,  v,       s,
            d_o, kv_in, dkv_in, dq,
            dk, dv, dkv_out, kv_seg_states,
            nullptr, nullptr};
  float *wp = workspace;
  if (need_dkv) {
    a.ws_dkv = wp;
    wp += one / sizeof(float);
  }
  if (need_kv) a.ws_kv = wp;
  hipStream_t st = (hipStream_t)stream;
  rc = mfma_eligible(d, e, dtype)       ? mfma_bwd(a, g, dtype, st)
       : mfma_f32_eligible(d, e, dtype) ? mfma_f32_bwd(a, g, st)
                                        : generic_bwd(a, g, dtype, st);
  if (rc > 0) set_error("lasp_chunk_bwd: HIP error %d: %s", rc, hipGetErrorString((hipError_t)rc));
  return rc;
}

}  // extern "C"
