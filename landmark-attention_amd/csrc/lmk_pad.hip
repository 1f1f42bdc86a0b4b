// Row moves between the two layouts of a tensor whose landmark blocks are narrower than the kernels' block
// sizes.  The attention kernels work on blocks of 32, 64 or 128 slots; a block of n_real tokens
// (llama/ltriton/flash_landmark_attention.py:318 allows any block_size) is stored in the next larger size
// with its n_real-1 normal tokens in front, its landmark in the last slot and zero rows in between, which
// the kernels mask.  Pure data movement: 16 bytes per lane, whole rows, any 16-bit dtype.
#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

template <int D, bool UNPAD>
__global__ __launch_bounds__(256) void lmk_pad_blocks_kernel(PadParams p) {
  constexpr int LPR = D / 8;                               // lanes per row
  constexpr int RPW = 256 / LPR;                           // rows per workgroup
  const int tid = threadIdx.x, j = tid % LPR;
  const int64_t row = (int64_t)blockIdx.x * RPW + tid / LPR;   // (batch*head, destination row)
  if (row >= (int64_t)p.B * p.H * p.L_dst) return;
  const int bh = (int)(row / p.L_dst), d = (int)(row % p.L_dst);
  const int b = bh / p.H, hh = bh % p.H;
  int s;                                                   // source row, or -1 for a padding slot
  if (UNPAD) {
    const int blk = d / p.n_real, i = d % p.n_real;
    s = blk * p.block + (i == p.n_real - 1 ? p.block - 1 : i);
  } else {
    const int blk = d / p.block, i = d % p.block;
    s = (i < p.n_real - 1) ? blk * p.n_real + i : (i == p.block - 1 ? blk * p.n_real + p.n_real - 1 : -1);
  }
  u32x4_t x = {0, 0, 0, 0};
  if (s >= 0 && s < p.L_src)
    x = *(const u32x4_t*)((const char*)p.src + 2 * (b * p.ss_b + hh * p.ss_h + (int64_t)s * p.ss_r) + 16 * j);
  *(u32x4_t*)((char*)p.dst + 2 * (b * p.ds_b + hh * p.ds_h + (int64_t)d * p.ds_r) + 16 * j) = x;
}

template <int D>
static int launch_pad_t(const PadParams& p, bool unpad, hipStream_t stream) {
  constexpr int RPW = 256 / (D / 8);
  const int64_t rows = (int64_t)p.B * p.H * p.L_dst;
  const dim3 grid((unsigned)((rows + RPW - 1) / RPW));
  if (unpad) hipLaunchKernelGGL((lmk_pad_blocks_kernel<D, true>), grid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((lmk_pad_blocks_kernel<D, false>), grid, dim3(256), 0, stream, p);
  return (int)hipGetLastError();
}

int launch_pad_blocks(const PadParams& p, int D, bool unpad, hipStream_t stream) {
  if (D == 128) return launch_pad_t<128>(p, unpad, stream);
  if (D == 64) return launch_pad_t<64>(p, unpad, stream);
  return LMK_ERR_UNSUPPORTED;
}

}  // namespace lmk
