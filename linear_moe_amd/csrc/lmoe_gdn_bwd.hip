// Instantiation and launch of the chunk-parallel backward kernel of the gated delta rule.
#include "lmoe_launch.hpp"
#include "lmoe_gdn_bwd_chunk.hpp"

namespace lmoe {

template <typename T, int K, int V> struct GdnBwdChunk {
  static void run(const lmoe_args& a, hipStream_t st) {
    constexpr int BVH = 32;                            // V-slice of stage 1
    constexpr int NBUF = sizeof(T) == 2 ? 3 : 1;       // slice buffers: three where LDS has the room
    // register sets of the loaders' prefetch rotation: a divisor of the V / BVH + 2 units of an item (three sets
    // against two: 368 -> 362 us at B = 4, T = 8192, H = 16, K = V = 128)
    constexpr int DEPTH = sizeof(T) == 2 ? ((V / BVH + 2) % 3 == 0 ? 3 : 2) : 1;
    static_assert(GdnBwdChunkLds<T, K, BVH, NBUF>::BYTES <= 160 * 1024, "LDS budget of k_gdn_bwd_chunk");
    const int grid = persistent_grid(a.NT * a.H, 1);
    if constexpr (sizeof(T) == 2 && V <= 128) {      // (the entry point rejects q_raw with V = 256)
      if (a.q_raw.ptr) {       // dq, dk with respect to the rows behind q = l2norm(silu(.)), k likewise
        // (two register sets: the raw rows of the item take the room of the third)
        hipLaunchKernelGGL((k_gdn_bwd_chunk<T, K, V, BVH, NBUF, 2, true>), dim3(grid), dim3(3 * NTHR), 0, st, a);
        return;
      }
    }
    hipLaunchKernelGGL((k_gdn_bwd_chunk<T, K, V, BVH, NBUF, DEPTH>), dim3(grid), dim3(3 * NTHR), 0, st, a);
  }
};
void launch_gdn_bwd_chunk(const lmoe_args& a, hipStream_t st) { dispatch_gdn<GdnBwdChunk>(a, st); }

}  // namespace lmoe
