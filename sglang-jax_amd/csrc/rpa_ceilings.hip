// Measurement kernels for bench.py: what the memory system and the matrix pipe of THIS device deliver to the
// simplest possible kernel of the same shape as the attention kernels, so that a roofline fraction against the
// published peak can be read next to a fraction of what is reachable.  Built into lib/librpa_ceilings.so, a
// library of its own: nothing here is part of the attention path or of librpa_mi355.so.
//
//   rpa_ceiling_stream_read   every wave streams 16 KiB blocks (sixteen 16-byte loads per lane in flight, the
//                             next block requested before the current one is consumed: the decode kernels'
//                             block and pipeline), contiguous or through a page table, with plain or with
//                             non-temporal loads (what the decode kernels use), and folds them with xor
//   rpa_ceiling_lds_dma_read  the same stream moved into LDS by global_load_lds_dwordx4 (the tile rings' way)
//   rpa_ceiling_mfma          every wave issues v_mfma_f32_32x32x16_bf16 into four independent accumulators,
//                             two waves per SIMD (two workgroups of four waves per CU, held there by LDS size)
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kBlockBytes = 16384;  // 64 lanes x 16 B x 16 loads

struct Block {
  u32x4 v[16];
};

template <bool NT>
__device__ __forceinline__ void load_block(Block& b, const char* p, int lane) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const u32x4* q = reinterpret_cast<const u32x4*>(p + i * 1024 + lane * 16);
    b.v[i] = NT ? __builtin_nontemporal_load(q) : *q;
  }
}

__device__ __forceinline__ void fold_block(u32x4& acc, const Block& b) {
#pragma unroll
  for (int i = 0; i < 16; ++i) acc ^= b.v[i];
}

// order 0: wave w takes the contiguous run of blocks [w * per, (w + 1) * per)  (the balanced decode plan's shape)
// order 1: wave w takes blocks w, w + waves, w + 2 * waves, ...               (neighbouring waves, neighbouring memory)
// table != nullptr: block b lives in page table[b / blocks_per_page] at offset (b % blocks_per_page) * 16 KiB
// NT: non-temporal loads
template <bool NT>
__global__ __launch_bounds__(256) void stream_read_kernel(const char* __restrict__ base, const int32_t* __restrict__ table,
                                                          int64_t num_blocks, int blocks_per_page, int64_t page_bytes,
                                                          int order, uint32_t* __restrict__ sink) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t waves = (int64_t)gridDim.x * 4;
  const int64_t per = (num_blocks + waves - 1) / waves;
  int64_t b, step, end;
  if (order == 0) {
    b = wave * per, step = 1, end = b + per < num_blocks ? b + per : num_blocks;
  } else {
    b = wave, step = waves, end = num_blocks;
  }
  auto addr = [&](int64_t blk) -> const char* {
    if (table == nullptr) return base + blk * kBlockBytes;
    const int64_t page = table[blk / blocks_per_page];
    return base + page * page_bytes + (blk % blocks_per_page) * kBlockBytes;
  };
  u32x4 acc = {0, 0, 0, 0};
  if (b < end) {
    Block cur, nxt;
    load_block<NT>(cur, addr(b), lane);
    for (b += step; b < end; b += step) {
      load_block<NT>(nxt, addr(b), lane);
      fold_block(acc, cur);
      cur = nxt;
    }
    fold_block(acc, cur);
  }
  // the result has to be observable or the loads go away; random data never folds to this value
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x5a17c0deu) sink[0] = (uint32_t)wave;
}

// The same stream, moved into LDS by global_load_lds_dwordx4 instead of into registers (the way the prefill and MLA
// kernels fill their tile rings): four waves per workgroup, every wave two 16 KiB buffers, the copies of block i + 1
// in flight while block i's have landed; one word of every block is read back from LDS and folded.
template <bool NT>
__global__ __launch_bounds__(256) void lds_dma_read_kernel(const char* __restrict__ base, int64_t num_blocks,
                                                          uint32_t* __restrict__ sink) {
  __shared__ __attribute__((aligned(1024))) char ring[4][2][kBlockBytes];
  const int lane = threadIdx.x & 63;
  const int w = threadIdx.x >> 6;
  const int64_t wave = (int64_t)blockIdx.x * 4 + w;
  const int64_t waves = (int64_t)gridDim.x * 4;
  const int64_t per = (num_blocks + waves - 1) / waves;
  int64_t b = wave * per;
  const int64_t end = b + per < num_blocks ? b + per : num_blocks;
  typedef __attribute__((address_space(3))) char* lds_ptr_t;
  auto copy_block = [&](int slot, int64_t blk) {
    const char* src = base + blk * kBlockBytes + lane * 16;
    const uint32_t dst = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)&ring[w][slot][0]);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (NT)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(dst + i * 1024), "v"(src + i * 1024) : "memory", "m0");
      else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst + i * 1024), "v"(src + i * 1024) : "memory", "m0");
    }
  };
  uint32_t acc = 0;
  if (b < end) {
    int slot = 0;
    copy_block(0, b);
    for (++b; b < end; ++b) {
      copy_block(slot ^ 1, b);
      asm volatile("s_waitcnt vmcnt(16)" ::: "memory");  // all but the newest block's copies have landed
      acc ^= *reinterpret_cast<const uint32_t*>(&ring[w][slot][lane * 4]);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the slot is read before the block after next overwrites it
      slot ^= 1;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    acc ^= *reinterpret_cast<const uint32_t*>(&ring[w][slot][lane * 4]);
  }
  if (acc == 0x5a17c0deu) sink[0] = (uint32_t)wave;
}

__global__ __launch_bounds__(256) void mfma_issue_kernel(int iters, float* __restrict__ sink) {
  extern __shared__ char hold[];  // nothing is kept here: its size limits a CU to two workgroups
  const int lane = threadIdx.x & 63;
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(0.01f * (float)((lane * 7 + i * 3) % 17 - 8));
    b[i] = (__bf16)(0.01f * (float)((lane * 5 + i * 11) % 13 - 6));
  }
  f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
  if (s == 12345.678f) sink[0] = s + (float)hold[lane];
}

}  // namespace

#define CEIL_API extern "C" __attribute__((visibility("default")))

// Streams `bytes` (a multiple of 16 KiB) from `src` on `waves` wavefronts (a multiple of 4).  `table` (device,
// nullable) maps page slots to pages of `page_bytes` (a multiple of 16 KiB).  `order`: 0 / 1 as above, + 4 for
// non-temporal loads.  Returns a hipError_t.
CEIL_API int rpa_ceiling_stream_read(const void* src, int64_t bytes, const int32_t* table, int64_t page_bytes,
                                     int waves, int order, void* sink, void* stream) {
  if (bytes <= 0 || bytes % kBlockBytes || waves <= 0 || waves % 4) return (int)hipErrorInvalidValue;
  if (table != nullptr && (page_bytes <= 0 || page_bytes % kBlockBytes)) return (int)hipErrorInvalidValue;
  const int bpp = table ? (int)(page_bytes / kBlockBytes) : 1;
  if (order & 4)
    hipLaunchKernelGGL(stream_read_kernel<true>, dim3(waves / 4), dim3(256), 0, (hipStream_t)stream, (const char*)src, table,
                       bytes / kBlockBytes, bpp, page_bytes, order & 3, (uint32_t*)sink);
  else
    hipLaunchKernelGGL(stream_read_kernel<false>, dim3(waves / 4), dim3(256), 0, (hipStream_t)stream, (const char*)src, table,
                       bytes / kBlockBytes, bpp, page_bytes, order & 3, (uint32_t*)sink);
  return (int)hipGetLastError();
}

// The same read through global_load_lds_dwordx4 into LDS: `waves` a multiple of 4, one workgroup of four waves per
// CU (128 KiB of LDS); nt != 0: with the non-temporal bit.  Returns a hipError_t.
CEIL_API int rpa_ceiling_lds_dma_read(const void* src, int64_t bytes, int waves, int nt, void* sink, void* stream) {
  if (bytes <= 0 || bytes % kBlockBytes || waves <= 0 || waves % 4) return (int)hipErrorInvalidValue;
  if (nt)
    hipLaunchKernelGGL(lds_dma_read_kernel<true>, dim3(waves / 4), dim3(256), 0, (hipStream_t)stream, (const char*)src,
                       bytes / kBlockBytes, (uint32_t*)sink);
  else
    hipLaunchKernelGGL(lds_dma_read_kernel<false>, dim3(waves / 4), dim3(256), 0, (hipStream_t)stream, (const char*)src,
                       bytes / kBlockBytes, (uint32_t*)sink);
  return (int)hipGetLastError();
}

// `workgroups` workgroups of four waves, each wave `iters` x 16 matrix instructions of 32768 FLOP.
CEIL_API int rpa_ceiling_mfma(int workgroups, int iters, void* sink, void* stream) {
  if (workgroups <= 0 || iters <= 0) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(mfma_issue_kernel, dim3(workgroups), dim3(256), 65536, (hipStream_t)stream, iters, (float*)sink);
  return (int)hipGetLastError();
}
