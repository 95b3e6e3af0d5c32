// lasp_stream_probe: what the memory system sustains for the sweeps' access pattern without their
// arithmetic.  R read streams and W write streams of the same size; a workgroup of 256 threads walks
// pieces of 16 KiB (one 64-token block of 128 16-bit features), 16 bytes per lane per access, the
// pieces dealt to the workgroups round-robin; writes are non-temporal like the kernels' output stores.
// A measurement hook: nothing in the operator path calls it.
#include "lasp_common.h"

namespace lasp {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kPieceVec = 16384 / 16;  // 16-byte vectors per piece
constexpr int kMaxStreams = 8;

struct Streams {
  const u32x4 *rd[kMaxStreams];
  u32x4 *wr[kMaxStreams];
};

template <int R, int W>
__global__ void __launch_bounds__(256) stream_probe_kernel(Streams p, int64_t n_piece) {
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (int64_t piece = blockIdx.x; piece < n_piece; piece += gridDim.x) {
    const int64_t base = piece * kPieceVec + threadIdx.x;
    u32x4 v[R > 0 ? R : 1][4];
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
      for (int u = 0; u < 4; ++u) v[i][u] = p.rd[i][base + u * 256];
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
      for (int u = 0; u < 4; ++u) acc ^= v[i][u];
#pragma unroll
    for (int i = 0; i < W; ++i)
#pragma unroll
      for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(acc, &p.wr[i][base + u * 256]);
  }
  // a store the compiler cannot rule out keeps the loads of a read-only mix alive
  if (W == 0 && acc.x == 0x12345678u && acc.y == 0x9abcdef0u) const_cast<u32x4 *>(p.rd[0])[0] = acc;
}

template <int R, int W>
int launch(const Streams &p, int64_t n_piece, int grid, hipStream_t st) {
  stream_probe_kernel<R, W><<<(unsigned)grid, 256, 0, st>>>(p, n_piece);
  return (int)hipGetLastError();
}

}  // namespace
}  // namespace lasp

using namespace lasp;

extern "C" int lasp_stream_probe(const void *const *rd, int n_rd, void *const *wr, int n_wr, size_t bytes_each,
                                 int grid, void *stream) {
  if (n_rd < 0 || n_wr < 0 || n_rd > kMaxStreams || n_wr > kMaxStreams || (n_rd && !rd) || (n_wr && !wr) || grid <= 0 ||
      bytes_each == 0 || bytes_each % 16384 != 0) {
    set_error("lasp_stream_probe: need 0..%d read and write streams, a positive grid and a size that is a multiple "
              "of 16384 bytes", kMaxStreams);
    return LASP_E_SHAPE;
  }
  Streams p = {};
  for (int i = 0; i < n_rd; ++i) {
    if (!rd[i] || (uintptr_t)rd[i] % 16) {
      set_error("lasp_stream_probe: read stream %d is NULL or not 16-byte aligned", i);
      return LASP_E_ALIGN;
    }
    p.rd[i] = (const u32x4 *)rd[i];
  }
  for (int i = 0; i < n_wr; ++i) {
    if (!wr[i] || (uintptr_t)wr[i] % 16) {
      set_error("lasp_stream_probe: write stream %d is NULL or not 16-byte aligned", i);
      return LASP_E_ALIGN;
    }
    p.wr[i] = (u32x4 *)wr[i];
  }
  const int64_t n_piece = (int64_t)(bytes_each / 16384);
  hipStream_t st = (hipStream_t)stream;
  int rc;
  const int mix = n_rd * 16 + n_wr;
  switch (mix) {
    case 1 * 16 + 0: rc = launch<1, 0>(p, n_piece, grid, st); break;
    case 2 * 16 + 0: rc = launch<2, 0>(p, n_piece, grid, st); break;
    case 4 * 16 + 0: rc = launch<4, 0>(p, n_piece, grid, st); break;
    case 1 * 16 + 1: rc = launch<1, 1>(p, n_piece, grid, st); break;
    case 3 * 16 + 1: rc = launch<3, 1>(p, n_piece, grid, st); break;
    case 4 * 16 + 3: rc = launch<4, 3>(p, n_piece, grid, st); break;
    case 7 * 16 + 3: rc = launch<7, 3>(p, n_piece, grid, st); break;
    case 0 * 16 + 1: rc = launch<0, 1>(p, n_piece, grid, st); break;
    default:
      set_error("lasp_stream_probe: the mix %d reads : %d writes is not built (1:0, 2:0, 4:0, 0:1, 1:1, 3:1, 4:3, 7:3 are)",
                n_rd, n_wr);
      return LASP_E_SHAPE;
  }
  if (rc > 0) set_error("lasp_stream_probe: HIP error %d: %s", rc, hipGetErrorString((hipError_t)rc));
  return rc;
}
