// Row partition by modality: mask[M] -> perm[M] (visual rows first, each group in ascending
// row order) and counts[2].  The reference tests mask rows inside every GEMM tile
// (ffn_kernel/linear.py:120-149); here the same row -> weight assignment is made once,
// as an integer permutation, so that GEMM tiles never mix modalities.
//
// One launch, no inter-block dependency: every block re-counts the visual rows that
// precede its rows (and the total) straight from the mask, which is at most M bytes of
// L2-resident reads per block, then places its own rows, 1024 at a time.  The launch has at most
// kRouteMaxBlocks blocks (each takes more 1024-row chunks instead), so the counting reads stay
// linear in M: kRouteMaxBlocks * M bytes.
#include "common.hpp"
#include "launch.hpp"

namespace ffnk {

constexpr int kRouteThreads = 256;
constexpr int kRouteRowsPerThread = 4;
constexpr int kRouteChunk = kRouteThreads * kRouteRowsPerThread;  // 1024 rows per pass of a block: the launch is latency-bound, short chains per thread
constexpr int kRouteMaxBlocks = 256;                              // one per CU; past 256 K rows a block places several chunks in turn

// 16-bit mask of the non-zero bytes of a 16-byte vector (bit j = byte j).
__device__ __forceinline__ uint32_t nonzero_bytes16(uint4 v) {
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
  uint32_t bits = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t t = (w[i] | ((w[i] & 0x7f7f7f7fu) + 0x7f7f7f7fu)) & 0x80808080u;  // bit 7 of each non-zero byte
    uint32_t nib = (((t >> 7) * 0x01020408u) >> 24) & 0xFu;                     // gather to 4 bits
    bits |= nib << (4 * i);
  }
  return bits;
}

// Bits [lo, hi) of a 16-bit field, lo/hi clamped to [0, 16].
__device__ __forceinline__ uint32_t range_bits16(int64_t lo, int64_t hi) {
  int l = lo < 0 ? 0 : (lo > 16 ? 16 : (int)lo);
  int h = hi < 0 ? 0 : (hi > 16 ? 16 : (int)hi);
  if (h <= l) return 0;
  return ((1u << h) - 1u) & ~((1u << l) - 1u);
}

__global__ __launch_bounds__(kRouteThreads) void route_kernel(const uint8_t* __restrict__ mask, int M,
                                                               int32_t* __restrict__ perm,
                                                               int32_t* __restrict__ counts, int chunks_per_block) {
  __shared__ int s_red[2][kRouteThreads / kWave];
  __shared__ int s_wave[kRouteThreads / kWave];
  const int t = threadIdx.x;
  const int64_t lo = (int64_t)blockIdx.x * chunks_per_block * kRouteChunk;  // first row of this block

  // Phase 1: total visual rows, and visual rows before `lo`, from aligned 16-byte reads.
  const int a = (int)(reinterpret_cast<uintptr_t>(mask) & 15);
  const uint4* base = reinterpret_cast<const uint4*>(mask - a);
  const int64_t nvec = M > 0 ? ((int64_t)a + M + 15) / 16 : 0;  // M == 0: mask may be NULL
  int tot = 0, bef = 0;
  for (int64_t v = t; v < nvec; v += kRouteThreads) {
    const int64_t f = v * 16 - a;  // row index of byte 0 of this vector
    const uint32_t bits = nonzero_bytes16(base[v]) & range_bits16(-f, (int64_t)M - f);
    tot += __popc(bits);
    bef += __popc(bits & range_bits16(-f, lo - f));
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    tot += __shfl_down(tot, off);
    bef += __shfl_down(bef, off);
  }
  if ((t & (kWave - 1)) == 0) {
    s_red[0][t / kWave] = tot;
    s_red[1][t / kWave] = bef;
  }
  __syncthreads();
  tot = 0;
  bef = 0;
#pragma unroll
  for (int w = 0; w < kRouteThreads / kWave; ++w) {
    tot += s_red[0][w];
    bef += s_red[1][w];
  }
  if (blockIdx.x == 0 && t == 0) {
    counts[0] = tot;
    counts[1] = M - tot;
  }

  // Phase 2, chunk by chunk: this thread owns kRouteRowsPerThread consecutive rows of the chunk, from r0;
  // `bef` counts the visual rows ahead of the chunk.
  for (int ch = 0; ch < chunks_per_block; ++ch) {
    if (lo + (int64_t)ch * kRouteChunk >= M) break;  // uniform over the block
    const int64_t r0 = lo + (int64_t)ch * kRouteChunk + (int64_t)t * kRouteRowsPerThread;
    uint32_t bits = 0;
#pragma unroll
    for (int j = 0; j < kRouteRowsPerThread; ++j) {
      if (r0 + j < M && mask[r0 + j] != 0) bits |= 1u << j;
    }
    const int c = __popc(bits);
    // Inclusive scan of the per-thread counts: inside each wave by shuffles, across the four waves through LDS.
    int incl = c;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if ((t & (kWave - 1)) >= off) incl += up;
    }
    if ((t & (kWave - 1)) == kWave - 1) s_wave[t / kWave] = incl;
    __syncthreads();
    int chunk_total = 0;
#pragma unroll
    for (int w = 0; w < kRouteThreads / kWave; ++w) {
      if (w < t / kWave) incl += s_wave[w];
      chunk_total += s_wave[w];
    }
    __syncthreads();  // s_wave is rewritten by the next chunk
    int vb = bef + incl - c;  // visual rows before r0
    bef += chunk_total;
#pragma unroll
    for (int j = 0; j < kRouteRowsPerThread; ++j) {
      const int64_t r = r0 + j;
      if (r < M) {
        if (bits & (1u << j)) {
          perm[vb] = (int32_t)r;
          ++vb;
        } else {
          perm[tot + (int)(r - vb)] = (int32_t)r;
        }
      }
    }
  }
}

hipError_t launch_route(const uint8_t* mask, int M, int32_t* perm, int32_t* counts, hipStream_t stream) {
  // M == 0 still runs one block so that counts[] is written.
  const int chunks = M > 0 ? cdiv(M, kRouteChunk) : 1;
  const int chunks_per_block = cdiv(chunks, kRouteMaxBlocks);
  const int blocks = cdiv(chunks, chunks_per_block);
  hipLaunchKernelGGL(route_kernel, dim3(blocks), dim3(kRouteThreads), 0, stream, mask, M, perm, counts, chunks_per_block);
  return hipGetLastError();
}

}  // namespace ffnk
