// Host-side parameter blocks and launcher declarations shared by the C ABI
// (lmk_api.hip) and the kernel translation units.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/lmk.h"

namespace lmk {

// A kernel's dynamic-LDS limit is an attribute of the function ON ONE DEVICE: it is raised once per
// (kernel instantiation, device); `done` is that instantiation's bit mask of devices already served.
// Returns 0 or a hipError_t.
template <class K>
inline int allow_dynamic_lds(K kern, int bytes, std::atomic<uint64_t>& done) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  const uint64_t bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return 0;
  e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return (int)e;
  done.fetch_or(bit, std::memory_order_release);
  return 0;
}

// Compute units of the current device (looked up once; 256 if the query fails).
inline int cu_count() {
  static std::atomic<int> n{0};
  int v = n.load(std::memory_order_relaxed);
  if (v == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    n.store(v, std::memory_order_relaxed);
  }
  return v;
}

struct FwdParams {
  const void *q, *k, *v;
  void* o;
  float *L, *M;
  int B, H, Lq, Lk;
  int n_prefix;   // history blocks in front of the queries
  int n_qtiles;   // ceil(Lq / 128)
  int n_real;     // tokens of a block that exist (normal keys in front, landmark last); == block unless padded
  // Lq_real > 0: q, k, v, o, L, M hold Lq_real / Lk_real rows of blocks of n_real tokens as they are ("token
  // layout"), and Lq, Lk above count the slots the kernels work on (whole blocks widened to `block` slots, a
  // partial last block keeps its length); the kernels translate slot rows to token rows themselves.
  // 0: the tensors are stored in slots already (n_real < block: with padding rows).
  int Lq_real, Lk_real;
  // token layout with blocks of unequal length (landmarks at irregular positions): seg[b] = first token of key block
  // b, n_blocks + 1 entries in device memory, n_full_k of the blocks complete (ending in their landmark); null:
  // every block holds n_real tokens.  n_full_q, n_full_k are set in both cases.
  const int* seg;
  int n_full_q, n_full_k;
  // optional (blocks of 64 / 128 slots, token layout only): factor of earlier block b's contribution to query row i,
  // group_scale[bh * gs_bh + b * gs_blk + i] -- 0 drops the block for that row, 1 / (1 - p) keeps it under group
  // dropout (lm_benchmark/models/landmark.py:110-113); the softmax over the landmarks is not renormalised
  const float* group_scale;
  int64_t gs_bh, gs_blk;
  // optional: q arrives without rotary and is rotated as it is loaded (null tables: q is used as it is)
  const void *rope_cos, *rope_sin;
  const int64_t* rope_pos;        // position of query row r of batch b: rope_pos[b * rope_pos_stride_b + r]
  int64_t rope_pos_stride_b, rope_cs_r, rope_n_pos;
  int64_t qs_b, qs_h, qs_r, ks_b, ks_h, ks_r, vs_b, vs_h, vs_r, os_b, os_h, os_r;  // element strides
  float scale_log2;  // sm_scale * log2(e)
};

int launch_fwd(const FwdParams& p, int D, int BS, int dtype, hipStream_t stream);
int launch_fwd32(const FwdParams& p, int D, int dtype, hipStream_t stream);   // block 32 specialisation

struct BwdParams {
  const void *q, *k, *v, *o, *dout;
  void *dq, *dk, *dv;
  const float *L, *M;            // forward statistics, (B*H, Lq)
  float *delta, *mhat;           // (B*H, Lq) each, written by the pre kernel
  float *stat_a, *stat_n, *stat_l;   // (B*H, n_blocks, Lq) each, written by the dq kernel
  // hand-over (block 32 only): the dq kernel leaves dS of every (query tile, key block) pair behind as a 2 KB
  // 16-bit tile and the dK/dV kernel reads it instead of forming dP and dS again; then stat_n and stat_l are unused.
  // Tiles of a head are ordered by query tile, then key block: tile (j, k), k <= n_prefix + j, is number
  // j * (n_prefix + 1) + j * (j - 1) / 2 + k.  Null: no hand-over.
  void* ds_tiles;
  int B, H, Lq, Lk;
  int n_prefix, n_blocks;        // history blocks; Lk / block
  int n_qtiles, n_kvtiles;       // ceil(Lq / 128), ceil(Lk / 128)
  int n_real;                    // tokens of a block that exist; == block unless padded (blocks 64 and 128 only)
  int Lq_real, Lk_real;          // > 0: tensors in token layout, as in FwdParams (the workspace stays indexed by slot rows)
  const int* seg;                // blocks of unequal length, as in FwdParams (null: n_real tokens each)
  int n_full_q, n_full_k;
  const float* group_scale;      // optional, as in FwdParams (token layout only)
  int64_t gs_bh, gs_blk;
  int64_t qs_b, qs_h, qs_r, ks_b, ks_h, ks_r, vs_b, vs_h, vs_r, os_b, os_h, os_r, dos_b, dos_h, dos_r;
  int64_t dqs_b, dqs_h, dqs_r, dks_b, dks_h, dks_r, dvs_b, dvs_h, dvs_r;
  float scale, scale_log2;
};

// phases: bit 0 = pre, bit 1 = dq, bit 2 = dkdv
int launch_bwd(const BwdParams& p, int D, int BS, int dtype, int phases, hipStream_t stream);
int launch_bwd_dq32(const BwdParams& p, int D, int dtype, hipStream_t stream);     // block 32 specialisation
int launch_bwd_dkdv32(const BwdParams& p, int D, int BS, int dtype, hipStream_t stream);   // two-role kernel, all block sizes
int launch_bwd_dkdv32_handover(const BwdParams& p, int D, int dtype, hipStream_t stream);  // block 32, dS read from p.ds_tiles

// dS tiles (2 KB each) one (batch, head) leaves behind in the hand-over: query tile j sees key blocks 0 .. n_prefix + j
__host__ __device__ inline int64_t handover_tiles_per_head(int64_t n_qtiles32, int64_t n_prefix) {
  return n_qtiles32 * (n_prefix + 1) + n_qtiles32 * (n_qtiles32 - 1) / 2;
}

// The rotated landmark keys are kept in tiles of 32 keys, 16-byte chunk c (8 head dims) of key n of the tile at byte
// (32 c + n) * 16: every consumer gives a lane one landmark, so a wave reading chunk c of 32 or 64 consecutive
// landmarks reads 512 contiguous bytes per tile -- as MFMA operand (lane = landmark, chunk = 8 of the 16 head dims
// of a step) and in the sequential dot products alike.  Keys past num_mems in the last tile are never written.
__host__ __device__ inline int64_t lk_tiles(int num_mems) { return ((int64_t)num_mems + 31) >> 5; }
__host__ __device__ inline int64_t lk_tile_bytes(int D) { return 32 * 2 * (int64_t)D; }
// byte offset of chunk 0 of landmark m inside one (batch, head)'s tiles; chunk c lies 512 c bytes further
__host__ __device__ inline int64_t lk_key_offset(int m, int D) { return (int64_t)(m >> 5) * lk_tile_bytes(D) + 16 * (m & 31); }

struct RetrParams {
  const void *q, *kcache, *vcache, *cos, *sin;   // q rotated; caches un-rotated; tables (n_pos, D)
  const void* o_loc;                              // attention over the local chunk (gather step)
  const float *L_loc, *M_loc;
  int64_t stat_stride;                            // floats between consecutive (batch, head) rows of L_loc, M_loc
  void* out;
  int64_t* idx;                                   // (B, H, T, k) ascending block indices
  int64_t idx_sb, idx_sh, idx_st;                 // gather step: elements between the index rows of batches, heads, queries
  void* lk_rot;                                   // rotated landmark keys, (B*H, ceil(num_mems / 32)) tiles: see lk_tile_bytes
  float* lk_norm;                                 // (B*H, num_mems)
  float *approx, *exact;                          // (B*H*T, num_mems) each
  uint32_t* agg;                                  // (B*H, num_mems) per-head maxima of the 16-bit probabilities
  uint16_t* agg_out;                              // optional copy of agg in the model dtype
  int B, H, T, S, block, num_mems, k;
  int ring_start;                                 // slot of the oldest block (0 unless the cache is a ring buffer of blocks)
  int agg_over_heads;                             // shared selection: agg is (B*T, num_mems), maxima over the heads
  int prob32;                                     // shared selection: agg holds fp32 probabilities, not 16-bit ones
  int lm_dense;                                   // kcache holds the landmark keys alone, one row per block
  int merge_slices;                               // gather step: > 0 = approx / exact hold the candidates of so many slices per row (k each),
                                                  // the k best of which are picked first and written to idx
  int64_t prefix_len;                             // full_len - (k + 1) * block, may be -block
  // gather step with the rows' local window inside (local != 0): the new tokens' keys and values (rotated by the
  // caller), the number of cached tokens behind the last complete block, their first row in the cache and its position
  int local, local_inc;
  const void *k_new, *v_new;
  int64_t kns_b, kns_h, kns_r, vns_b, vns_h, vns_r, local_row0, local_pos0;
  int64_t qs_b, qs_h, qs_r, kcs_b, kcs_h, kcs_r, vcs_b, vcs_h, vcs_r, cs_r;
  int64_t ols_b, ols_h, ols_r, outs_b, outs_h, outs_r;
  float sqrt_hd, scale_log2;
};

// local window of the attend step: [n_sel rows of selected blocks | inc tail tokens | T new tokens]
struct WindowParams {
  const void *q, *kcache, *vcache, *k_loc, *v_loc, *cos, *sin;
  void* q_win;                                    // (B, H, inc + T, D), may be null when inc == 0
  void *k_win, *v_win;                            // (B, H, n_sel + inc + T, D) each
  const int64_t* idx;                             // (B, H, k) ascending block indices (n_sel > 0 only)
  int B, H, T, inc;
  int n_sel, k, block, num_mems;                  // n_sel = k * block rows of selected blocks in front, or 0
  int64_t prefix_len;
  int64_t full_len;                               // first cached row of the tail
  int64_t tail_pos;                               // its rotary position (the same number in the llama cache)
  int64_t qs_b, qs_h, qs_r, kcs_b, kcs_h, kcs_r, vcs_b, vcs_h, vcs_r, kls_b, kls_h, kls_r, vls_b, vls_h, vls_r;
  int64_t qws_b, qws_h, qws_r, kws_b, kws_h, kws_r, vws_b, vws_h, vws_r, cs_r;
};

// rotary embedding of a (B, H, L, D) tensor at positions pos[b * pos_stride_b + l]
struct RotaryParams {
  const void *x, *cos, *sin;
  void* out;
  const void* x2;                                 // optional second tensor of the same shape, rotated alongside
  void* out2;
  int64_t x2s_b, x2s_h, x2s_r, o2s_b, o2s_h, o2s_r;
  const int64_t* pos;
  int64_t pos_stride_b, n_pos;
  int B, H, L;
  int64_t xs_b, xs_h, xs_r, os_b, os_h, os_r, cs_r;
};

// Moves whole rows between a tensor with blocks of n_real tokens and one whose blocks are stored in `block`
// slots (normal tokens in front, landmark in the last slot, zero rows in between).
struct PadParams {
  const void* src;
  void* dst;
  int B, H, L_src, L_dst, n_real, block;
  int64_t ss_b, ss_h, ss_r, ds_b, ds_h, ds_r;
};
int launch_pad_blocks(const PadParams& p, int D, bool unpad, hipStream_t stream);

int launch_rotary(const RotaryParams& p, int D, int dtype, hipStream_t stream);

// Selection by slices, for a handful of query rows (decoding): a row's cached blocks are split into slices of 256
// over as many workgroups of four waves, and a row's slices are merged afterwards.
constexpr int kSliceWaves = 4;
constexpr int kSliceMems = 64 * kSliceWaves;                      // cached blocks per workgroup
constexpr int kSliceMaxRows = 1024;                               // rows (batch x head x query) up to which this path is used,
constexpr int kSliceMaxRowsPerHead = 4;                           // or queries per (batch, head): the other path works on 32 at a time
constexpr int kSliceMaxCand = 1024;                               // candidates (slices x k) the merge holds, 16 per lane
// slices per row when launch_retrieve_topk selects that way, else 0
inline int topk_slices(const RetrParams& p) {
  const int64_t rows = (int64_t)p.B * p.H * p.T;
  const int n_slices = (p.num_mems + kSliceMems - 1) / kSliceMems;
  const bool few = rows <= kSliceMaxRows || (p.T <= kSliceMaxRowsPerHead && rows * n_slices < ((int64_t)1 << 30));
  return (few && (int64_t)n_slices * p.k <= kSliceMaxCand) ? n_slices : 0;
}
int launch_retrieve_topk(const RetrParams& p, int D, int dtype, bool reuse_landmark_keys, hipStream_t stream);
int launch_retrieve_topk_shared(const RetrParams& p, int D, int dtype, hipStream_t stream);   // one selection per head
int launch_local_window(const WindowParams& p, int D, int dtype, hipStream_t stream);
// block-32 forward (pf) and the rotation of the landmark keys (pr: what launch_retrieve_topk would do first) in one launch
int launch_fwd32_landmark_keys(const FwdParams& pf, const RetrParams& pr, int D, int dtype, hipStream_t stream);
// block-32 forward (pf) and the slice step of the selection (pr, topk_slices(pr) > 0) in one launch: a row's candidates
// are left in pr.approx / pr.exact for a gather step with merge_slices set
int launch_fwd32_topk_slices(const FwdParams& pf, const RetrParams& pr, int D, int dtype, hipStream_t stream);
int launch_landmark_keys(const RetrParams& p, int D, int dtype, hipStream_t stream);   // the rotation alone
int launch_topk_slices(const RetrParams& p, int D, int dtype, hipStream_t stream);     // the selection's slice step alone
// rows whose local window the gather kernel attends to itself: window inside one block, a handful of new tokens
constexpr int kLocalMaxT = 4;
inline bool gather_takes_local_window(int T, int S, int block) {
  return (block == 32 || block == 64 || block == 128) && T <= kLocalMaxT && S % block + T <= block;
}
// BS: slots per block (32, 64 or 128); p.block <= BS tokens per block in the cache
int launch_gather_attend(const RetrParams& p, int D, int BS, int dtype, hipStream_t stream);

}  // namespace lmk
