// Row blocks, tile counts and the tile table of the large-M kernel (k_ring.hip), shared with
// the kernels that prepare a grouped launch on the device (k_moe.hip).
#pragma once
#include "zmi_device.h"

// Row blocks of one problem for a launch whose largest tile has `top` rows:
// floor(M / top) full blocks (handled by the BM == top kernel) and one remainder
// block handled by the smallest of {64, 128, 256} that holds it.  `top` may carry
// ZMI_RING_PAD: the remainder then stays with the BM == top kernel as a partly
// filled block, so that the weights of a problem are streamed by one launch only
// (the choice when the launch is bound by weight traffic, not by MFMA work).
#define ZMI_RING_PAD 0x10000
// Problems with at most 16 rows get no tiles: the decode-shaped grouped kernel (k_group_decode.hip) takes them.
#define ZMI_RING_SKIP_SMALL 0x20000
template <int BM>
__device__ __host__ __forceinline__ void zmi_ring_rows(int M, int top_flags, int &full, bool &has_rem) {
  const int top = top_flags & 0xffff;
  if ((top_flags & ZMI_RING_SKIP_SMALL) && M <= 16) { full = 0; has_rem = false; return; }
  full = BM == top ? M / top : 0;
  const int r = M % top;
  if (top_flags & ZMI_RING_PAD) has_rem = BM == top && r > 0;
  else has_rem = r > 0 && r <= BM && (BM == 64 || r > BM / 2);
}

template <int BM>
__host__ __device__ __forceinline__ int zmi_ring_items(int M, int N, int top, bool gated) {
  int full; bool rem;
  zmi_ring_rows<BM>(M, top, full, rem);
  const int ncols = gated ? N / 2 : N;
  const int per = gated ? 128 : 256;
  return (full + (rem ? 1 : 0)) * ((ncols + per - 1) / per);
}

// Tile table of a problem set, computed where the row counts live: tab[0..2] = number of
// tiles of the 256 / 128 / 64 row kernels, tab[4 + b * n_prob + e] = index of the first
// tile of problem e in kernel b.  One wavefront (all 64 lanes call it together), 64 problems per step.
__device__ __forceinline__ void zmi_ring_fill_table(const ZmiProblem *probs, int n_prob, int top, int gated, int *tab,
                                                    int lane) {
  int run[3] = {0, 0, 0};
  for (int e0 = 0; e0 < n_prob; e0 += 64) {
    const int e = e0 + lane;
    int c[3] = {0, 0, 0};
    if (e < n_prob) {
      const int M = probs[e].M, N = probs[e].N;
      if (M > 0) {
        if ((top & 0xffff) == 256) c[0] = zmi_ring_items<256>(M, N, top, gated != 0);
        c[1] = zmi_ring_items<128>(M, N, top, gated != 0);
        c[2] = zmi_ring_items<64>(M, N, top, gated != 0);
      }
    }
#pragma unroll
    for (int b = 0; b < 3; ++b) {
      // inclusive prefix over the wavefront
      int x = c[b];
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int y = __shfl_up(x, o);
        if (lane >= o) x += y;
      }
      if (e < n_prob) tab[4 + b * n_prob + e] = run[b] + x - c[b];
      run[b] += __shfl(x, 63);
    }
  }
  if (lane == 0) { tab[0] = run[0]; tab[1] = run[1]; tab[2] = run[2]; }
}
