// Shared definitions for the gfx950 kernels behind the C ABI in include/lasp_hip.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "lasp_hip.h"

namespace lasp {

typedef uint16_t bf16_t;  // raw bfloat16 bits

__device__ __forceinline__ float bf16_bits_to_f32(bf16_t x) {
  return __uint_as_float(((uint32_t)x) << 16);
}

// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ bf16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}

struct bf16_tag {
  bf16_t bits;
};

template <class T>
struct elem;
template <>
struct elem<float> {
  static __device__ __forceinline__ float load(const float *p) { return *p; }
  static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
};
template <>
struct elem<bf16_tag> {
  static __device__ __forceinline__ float load(const bf16_tag *p) {
    return bf16_bits_to_f32(p->bits);
  }
  static __device__ __forceinline__ void store(bf16_tag *p, float v) {
    p->bits = f32_to_bf16_bits(v);
  }
};
template <>
struct elem<_Float16> {
  static __device__ __forceinline__ float load(const _Float16 *p) { return (float)*p; }
  static __device__ __forceinline__ void store(_Float16 *p, float v) { *p = (_Float16)v; }
};

// One chunk's geometry, passed by value to every kernel.
struct Geom {
  int b, h;
  int64_t n;    // tokens in the chunk
  int d, e;     // feature sizes of q/k and v/o
  int seg_len;  // tokens per segment (multiple of 64)
  int n_seg;    // ceil(n / seg_len)
  int sd, se;   // rows and columns of one segment state as stored in the workspace: d x e for the
                // generic kernels, 128 x 128 (zero beyond d, e) for the MFMA kernels
  int fused;    // the chunk is served by the single-launch kernels, which use no workspace
  int combine;  // few segments: no scan launch, the sweep workgroups gather the segments' own states
  int bypass;   // the scan leaves out heads whose state dies within one segment (see state_dies_in_segment)
  int pre_len;  // tokens per segment of the pre-pass and the scan: seg_len, or seg_len / 2^k where long sweep
                // segments are cut finer for the pre-pass (16-bit scan path only)
  int pre_n;    // ceil(n / pre_len): states per (b, h) in the workspace
};

// Decay weights below 2^-kSkipLog2 are treated as zero by the 16-bit MFMA kernels.  A state is an fp32 sum
// whose largest terms carry weights near 1 (the tokens next to the segment's far end), so what is dropped
// lies below the rounding of that sum itself -- and the kernels round every state to 16 bits (2^-9 for
// bf16) before they multiply with it.
constexpr float kSkipLog2 = 24.f;
constexpr float kLog2e = 1.4426950408889634f;

// With g.bypass set, a head whose decay over the shortest segment of the pre-pass (the last one) is below
// 2^-kSkipLog2 takes no part in the scan: whatever enters a segment has faded to nothing at its far
// end, so the state entering segment j is the OWN state of the segment before it (after it, going
// backwards) and, for the first segment visited, the chunk's incoming state.  The scan kernel
// leaves those heads' own states in place and only forms their outgoing carry; the sweeps read the
// neighbour's own state.  Both sides must take the same decision, hence this one function.
__device__ __forceinline__ bool state_dies_in_segment(float slope, const Geom &g) {
  const int64_t last_len = g.n - (int64_t)(g.pre_n - 1) * g.pre_len;  // segments of the pre-pass and the scan
  return g.bypass != 0 && slope * kLog2e * (float)last_len > kSkipLog2;
}

// Host-side launchers (each returns a hipError_t as int, or a negative LASP_E_*).
struct FwdArgs {
  const void *q, *k, *v;
  const float *s;
  const float *kv_in;
  float *kv_out;
  void *o;
  float *seg_states;
};
struct BwdArgs {
  const void *q, *k, *v;
  const float *s;
  const void *d_o;
  const float *kv_in, *dkv_in;
  void *dq, *dk, *dv;
  float *dkv_out;
  const float *kv_seg_states;  // may be NULL
  float *ws_kv;                // used when kv_seg_states is NULL
  float *ws_dkv;
};

int generic_fwd(const FwdArgs &a, const Geom &g, int dtype, hipStream_t st);
int generic_bwd(const BwdArgs &a, const Geom &g, int dtype, hipStream_t st);
int mfma_fwd(const FwdArgs &a, const Geom &g, int dtype, hipStream_t st);  // bf16 or fp16
int mfma_bwd(const BwdArgs &a, const Geom &g, int dtype, hipStream_t st);
int mfma_f32_fwd(const FwdArgs &a, const Geom &g, hipStream_t st);
int mfma_f32_bwd(const BwdArgs &a, const Geom &g, hipStream_t st);

// The decayed scan over segment states is shared by both kernel families.
//   forward  (reverse = 0): states[seg] <- state entering segment seg from the
//             left (segment 0: carry_in or 0); carry_out <- state after the chunk
//   reverse  (reverse = 1): states[seg] <- state entering segment seg from the
//             right (last segment: carry_in or 0); carry_out <- state before the chunk
int launch_segment_scan(float *states, const float *carry_in, float *carry_out,
                        const float *s, const Geom &g, int reverse, hipStream_t st);

void set_error(const char *fmt, ...);

// Dynamic LDS above the default limit has to be granted once per kernel and device.  The grant is
// always for the kernel's maximum (so callers with different shapes cannot lower each other's
// limit between the grant and the launch) and is remembered per kernel, thread and device.
template <auto Kernel>
int grant_lds(int max_bytes) {
  static thread_local uint64_t granted = 0;  // one bit per device ordinal below 64
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev >= 0 && dev < 64 && ((granted >> dev) & 1u)) return 0;
  e = hipFuncSetAttribute((const void *)Kernel, hipFuncAttributeMaxDynamicSharedMemorySize, max_bytes);
  if (e == hipSuccess && dev >= 0 && dev < 64) granted |= (uint64_t)1 << dev;
  return (int)e;
}

// Optional per-kernel timing (lasp_profile_begin / lasp_profile_end): while a
// profile is open every kernel launch is bracketed by two events on its stream.
enum KernelClass { KC_APPLY = 0, KC_STATE = 1, KC_SCAN = 2, KC_GENERIC = 3, KC_BWD3 = 4, KC_FUSED = 5, KC_COUNT = 6 };
struct ProfEntry;
struct ProfScope {
  ProfScope(int kernel_class, hipStream_t st);
  ~ProfScope();
  int slot;
  ProfEntry *entry;
  hipStream_t stream;
};

}  // namespace lasp
