// Measurement behind the choice of a split backward (dQ kernel + dK/dV kernel, seven block
// contractions) over a fused kv-stationary one (five): a fused kernel has to add every
// 64 x 128 fp32 dQ tile it produces into a global buffer shared by all kv work-groups of the
// document.  This program issues exactly those tile additions - 8 GQA groups x 4 query heads, 256 kv
// work-groups per group, documents of `doc_tiles` kv tiles (128 rows each, i.e. 2 * doc_tiles query
// tiles of 64 rows), each kv work-group walking its document's query tiles from the last one back
// to its own diagonal, as the dK/dV kernel does - and nothing else, in four ways:
//   mode 0  atomicAdd, agent scope              (what a fused kernel would have to use)
//   mode 1  atomic add, work-group scope        (not sufficient for correctness; a lower bound on cost)
//   mode 2  plain read-modify-write, no atomicity (wrong results; the memory system's bound)
//   mode 3  plain store                         (the same traffic without the read)
// each with the kv work-groups of a group spread over the XCDs (xcd_local 0) or kept on one XCD
// (xcd_local 1).  It prints the time of one pass and the rate in bytes of accumulated tiles.
//
//   usage: dq_accumulate_probe [doc_tiles = 16]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CHECK(x)                                                   \
  do {                                                             \
    hipError_t e_ = (x);                                           \
    if (e_ != hipSuccess) {                                        \
      printf("%s: %s\n", #x, hipGetErrorString(e_));               \
      exit(1);                                                     \
    }                                                              \
  } while (0)

constexpr int kTileFloats = 64 * 128;

template <int MODE>
__global__ __launch_bounds__(512) void dq_accumulate_kernel(float* acc, int groups, int heads_per_group,
                                                            int n_kv_tiles, int doc_tiles, int xcd_local) {
  // work-group -> (group, kv tile); xcd_local: work-group ids of one group are congruent modulo 8,
  // which is how work-groups are dealt to the 8 XCDs
  const int wg = blockIdx.x;
  int group, j;
  if (xcd_local) {
    const int rounds = (groups + 7) / 8;
    group = wg % 8 + 8 * ((wg / 8) % rounds);
    j = wg / (8 * rounds);
  } else {
    j = wg % n_kv_tiles;
    group = wg / n_kv_tiles;
  }
  if (group >= groups || j >= n_kv_tiles) return;
  const int doc = j / doc_tiles, jd = j % doc_tiles;
  const int q_per_doc = 2 * doc_tiles;  // 64-row query tiles per document
  const int n_q_tiles = 2 * n_kv_tiles;
  const int tid = threadIdx.x;
  float v = 1.0f + tid * 1e-6f;
  for (int h = 0; h < heads_per_group; h++) {
    const int head = group * heads_per_group + h;
    for (int i = q_per_doc - 1; i >= 2 * jd; i--) {
      float* tile = acc + ((size_t)head * n_q_tiles + (size_t)doc * q_per_doc + i) * kTileFloats;
      // 512 threads x 16 floats, neighbouring lanes on neighbouring addresses
#pragma unroll
      for (int r = 0; r < 16; r++) {
        float* p = tile + r * 512 + tid;
        if (MODE == 0) atomicAdd(p, v);
        else if (MODE == 1) __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else if (MODE == 2) *p += v;
        else *p = v;
      }
      v += 1e-3f;
    }
  }
}

int main(int argc, char** argv) {
  const int groups = 8, heads_per_group = 4, n_kv = 256;
  const int doc_tiles = argc > 1 ? atoi(argv[1]) : 16;
  if (doc_tiles < 1 || doc_tiles > n_kv || n_kv % doc_tiles) {
    printf("doc_tiles must divide %d\n", n_kv);
    return 2;
  }
  const size_t n = (size_t)groups * heads_per_group * 2 * n_kv * kTileFloats;
  float* acc = nullptr;
  CHECK(hipMalloc(&acc, n * sizeof(float)));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  double adds = 0;  // tile additions of one pass
  for (int j = 0; j < n_kv; j++) adds += 2 * doc_tiles - 2 * (j % doc_tiles);
  adds *= groups * heads_per_group;
  const double bytes = adds * kTileFloats * 4;
  const int grid = groups * n_kv;
  for (int xcd_local = 0; xcd_local < 2; xcd_local++)
    for (int mode = 0; mode < 4; mode++) {
      float best = 1e30f;
      for (int rep = 0; rep < 4; rep++) {
        CHECK(hipMemsetAsync(acc, 0, n * sizeof(float), 0));
        CHECK(hipEventRecord(e0, 0));
        if (mode == 0) hipLaunchKernelGGL(dq_accumulate_kernel<0>, dim3(grid), dim3(512), 0, 0, acc, groups, heads_per_group, n_kv, doc_tiles, xcd_local);
        if (mode == 1) hipLaunchKernelGGL(dq_accumulate_kernel<1>, dim3(grid), dim3(512), 0, 0, acc, groups, heads_per_group, n_kv, doc_tiles, xcd_local);
        if (mode == 2) hipLaunchKernelGGL(dq_accumulate_kernel<2>, dim3(grid), dim3(512), 0, 0, acc, groups, heads_per_group, n_kv, doc_tiles, xcd_local);
        if (mode == 3) hipLaunchKernelGGL(dq_accumulate_kernel<3>, dim3(grid), dim3(512), 0, 0, acc, groups, heads_per_group, n_kv, doc_tiles, xcd_local);
        CHECK(hipGetLastError());
        CHECK(hipEventRecord(e1, 0));
        CHECK(hipEventSynchronize(e1));
        float ms;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        if (ms < best) best = ms;
      }
      printf("doc_tiles %d xcd_local %d mode %d: %.3f ms, %.1f GB/s of accumulated tiles (%.2f GB, %.0f tile additions)\n",
             doc_tiles, xcd_local, mode, best, bytes / best / 1e6, bytes / 1e9, adds);
      fflush(stdout);
    }
  CHECK(hipFree(acc));
  return 0;
}
