// Mem-cache retrieval for gfx950: landmark scoring, top-k block selection, gather + attend.
//
// Replaces the inline retrieval of LlamaAttention.forward (llama/llama_mem.py:344-412) and
// the attend step over retrieved blocks (:447-477) for the per-head, per-token branch.
//
// Selection must be reproducible bit for bit, so the score of (query, landmark) is defined
// as: fp32 dot product accumulated sequentially over the head dim with one fma per element,
// rounded to the model dtype, divided in fp32 by sqrt(hd), rounded again (the two roundings of
// `matmul(...) / math.sqrt(head_dim)`, :367).  Evaluating that for every pair on the vector
// ALU would dominate the step, so the work is split:
//   lk      rotate every cached landmark key at its slot position (:359-366), exactly as the
//           model dtype would round it, into a dense side array, with its 2-norm
//   score   MFMA product q . lk^T -> approximate fp32 scores
//   select  per query: bracket every score by the accumulation-error bound
//           eps = 2^-14 |q| |k|, push both ends through the (monotone) rounding contract, find
//           the k-th best lower end, and re-evaluate in the defined order only the "contenders"
//           whose upper end reaches it; then pick the k best under (score desc, index asc)
//           and write them in ascending order as int64 (:384).
//   gather  per query: stream the k selected K/V blocks straight from the cache, rotate keys at
//           their gather positions (:386-388, :408-410), local softmax per block gated by its
//           landmark, and merge with the attention over the local chunk (computed by the fused
//           forward kernel) through the shared global softmax bucket.
#include "lmk_common.hpp"
#include "lmk_landmark_keys.hpp"
#include "lmk_launch.hpp"
#include "lmk_topk_slice.hpp"

namespace lmk {

__device__ __forceinline__ u32x4_t shfl_xor4(u32x4_t v, int mask) {
  u32x4_t r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = (uint32_t)__shfl_xor((int)v[i], mask, 64);
  return r;
}

// ---------------------------------------------------------------------------
// lk: rotated landmark keys (dense) and their norms
// ---------------------------------------------------------------------------
template <class T, int D>
__global__ __launch_bounds__(256) void lmk_landmark_keys_kernel(RetrParams p) {
  landmark_keys_body<T, D, 256>(p, (int)blockIdx.x);
}

// ---------------------------------------------------------------------------
// one selection per head (llama_mem.py:373-384 with aggregate == "max_over_tokens"): every query's
// scores go through an fp32 softmax over the cached blocks, are rounded to the model dtype and
// reduced with a maximum over the queries; the head's k best blocks serve all its queries.
// The softmax needs every score exactly as the contract defines it, so there is no bracketing
// here: a lane evaluates the sequential dot product for its blocks.
// ---------------------------------------------------------------------------

// 2^t for t <= 0 with every rounding fixed, so that a CPU can reproduce it bit for bit:
// n = rint(t), f = t - n (exact), degree-6 Horner polynomial with one rounding after each product
// and each sum (the empty asm keeps the compiler from fusing them), times 2^n (exact).
__device__ __forceinline__ float exp2_contract(float t) {
  if (t < -126.f) return 0.f;
  const float n = __builtin_rintf(t);
  const float f = t - n;
  float pl = 1.5403530393381608e-4f;
  const float c[6] = {1.3333558146428443e-3f, 9.618129107628477e-3f, 5.550410866482158e-2f,
                      2.402265069591007e-1f,  6.931471805599453e-1f, 1.0f};
#pragma unroll
  for (int i = 0; i < 6; ++i) {
    float m = pl * f;
    asm volatile("" : "+v"(m));
    pl = m + c[i];
  }
  return __builtin_ldexpf(pl, (int)n);
}

template <class T>
__device__ __forceinline__ uint32_t prob_bits(float x);   // non-negative fp32 -> 16-bit pattern (RNE); monotone
template <>
__device__ __forceinline__ uint32_t prob_bits<bf16_t>(float x) {
  const uint32_t u = __float_as_uint(x);
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;           // integer rounding: also right for subnormal x
}
template <>
__device__ __forceinline__ uint32_t prob_bits<f16_t>(float x) { return pack2<f16_t>(x, 0.f) & 0xffffu; }

// Scores of every query against every landmark key, in the contract's order, into p.approx (B*H*T, num_mems).
// The contract's dot product is a chain of fp32 fmas over d ascending, and v_mfma_f32_32x32x1_2b_f32 is 2 x 32 x 32 of
// exactly that step: C[i][j] = fma(A[i], B[j], C[i][j]).  A wave takes 64 query rows (a lane holds its row, packed) and
// 64 keys (lanes 0..31 hold keys 0..31, lanes 32..63 keys 32..63, packed, 16 bytes per lane and chunk straight from the
// tiles of the rotated keys); per dimension one unpack each and two MFMAs -- the 64 rows as two blocks of 32 against
// the keys of the first 32 lanes (BLGP 1), then against those of the other 32 (BLGP 2) -- 4 matrix-pipe cycles per
// score.  (On the vector unit a score is 128 fmas plus whatever brings the key's value to every lane -- an unpack per
// fma with a key per lane, scalar loads of 8 bytes per score with the key in scalar registers, 16 times the LDS
// traffic with every lane reading the value, fmas that take the value from the lane that holds it (row_newbcast) --
// and every such kernel took 50-60 us at config 4's shapes.)
constexpr int kScoreRows = 64, kScoreKeys = 64;                   // per wave

template <class T, int D>
__global__ __launch_bounds__(256) void lmk_block_score_kernel(RetrParams p) {
  constexpr int CPR = D / 8;                                      // 16-byte chunks per row of 16-bit values
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int NM = p.num_mems;
  const int n_qg = (p.T + kScoreRows - 1) / kScoreRows, n_kc = (NM + kScoreKeys - 1) / kScoreKeys;
  // wave -> (query group, keys, head), query group first: the waves that run side by side read the same keys
  const int64_t wid = (int64_t)blockIdx.x * 4 + wave;
  {
    // the vectors the next kernel takes its maxima into start at zero: every wave of this one clears its share
    const int64_t words = (int64_t)(p.agg_over_heads ? p.B * p.T : p.B * p.H) * NM, n_waves = (int64_t)gridDim.x * 4;
    const int64_t per = (words + n_waves - 1) / n_waves, end = min(words, (wid + 1) * per);
    for (int64_t i = wid * per + lane; i < end; i += 64) p.agg[i] = 0u;
  }
  const int qg = (int)(wid % n_qg), kc = (int)((wid / n_qg) % n_kc);
  const int64_t bh64 = wid / n_qg / n_kc;
  if (bh64 >= (int64_t)p.B * p.H) return;                         // no workgroup-wide barrier in this kernel
  const int bh = (int)bh64;
  const int b = bh / p.H, hh = bh % p.H;
  const int m0 = kc * kScoreKeys;
  u32x4_t qp[CPR], kp[CPR];                                       // this lane's query row and key, packed
  {
    const int t = min(qg * kScoreRows + lane, p.T - 1);           // rows behind the last one: a re-read, never stored
    const char* src = (const char*)p.q + 2 * (b * p.qs_b + hh * p.qs_h + (int64_t)t * p.qs_r);
#pragma unroll
    for (int c = 0; c < CPR; ++c) qp[c] = *(const u32x4_t*)(src + 16 * c);
    const int m = min(m0 + lane, (int)(32 * lk_tiles(NM)) - 1);   // keys behind the last tile: likewise
    const char* lk = (const char*)p.lk_rot + (int64_t)bh * lk_tiles(NM) * lk_tile_bytes(D) + lk_key_offset(m, D);
#pragma unroll
    for (int c = 0; c < CPR; ++c) kp[c] = *(const u32x4_t*)(lk + 512 * c);
  }
  f32x32_t lo, hi;                                                // scores against keys m0 .. +31 and m0 + 32 .. + 63
#pragma unroll
  for (int r = 0; r < 32; ++r) lo[r] = hi[r] = 0.f;
#pragma unroll
  for (int c = 0; c < CPR; ++c)
#pragma unroll
    for (int i = 0; i < 8; ++i) {                                 // dimension 8 c + i
      const float qv = (i & 1) ? unpack_hi<T>(qp[c][i >> 1]) : unpack_lo<T>(qp[c][i >> 1]);
      const float kv = (i & 1) ? unpack_hi<T>(kp[c][i >> 1]) : unpack_lo<T>(kp[c][i >> 1]);
      lo = __builtin_amdgcn_mfma_f32_32x32x1f32(qv, kv, lo, 0, 0, 1);
      hi = __builtin_amdgcn_mfma_f32_32x32x1f32(qv, kv, hi, 0, 0, 2);
    }
  // register 16 blk + r of lane l: row 32 blk + 8 (r / 4) + 4 (l / 32) + r % 4, key l % 32 of the accumulator's 32
  const int key = lane & 31, rsub = 4 * (lane >> 5);
  const int64_t row0 = (int64_t)bh * p.T;
#pragma unroll
  for (int r = 0; r < 32; ++r) {
    const int t = qg * kScoreRows + 32 * (r >> 4) + 8 * ((r & 15) >> 2) + rsub + (r & 3);
    if (t >= p.T) continue;
    float* dst = p.approx + (row0 + t) * NM + m0 + key;
    if (m0 + key < NM) dst[0] = contract<T>(lo[r], p.sqrt_hd);
    if (m0 + 32 + key < NM) dst[32] = contract<T>(hi[r], p.sqrt_hd);
  }
}

// The rows' scores (p.approx) -> softmax -> 16-bit probabilities -> maximum per block into agg, which holds zeros on
// entry: one vector per (batch, head), maxima over the queries -- or per (batch, query), maxima over the heads.
// A lane owns the blocks m = lane, lane + 64, ...; a row's sum is each lane's running sum in that order, folded
// across lanes by halves.  A wave takes `rows_per_wave` rows that share a vector one after the other with the row in
// registers (NPL values per lane: num_mems <= 64 NPL) and the running maxima too, so a row is read once, nothing is
// written back and the vector sees one atomic per block and wave.  fp32 probabilities are positive, so their bit
// patterns order like the values.
template <int NPL>
__global__ __launch_bounds__(256) void lmk_block_prob_kernel(RetrParams p, int model_is_bf16, int rows_per_wave) {
  const int lane = threadIdx.x & 63;
  const int NM = p.num_mems;
  // rows that share a vector: the T queries of a (batch, head), or the H heads of a (batch, query)
  const int group = p.agg_over_heads ? p.H : p.T;
  const int per_group = (group + rows_per_wave - 1) / rows_per_wave;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= (int64_t)per_group * (p.agg_over_heads ? p.B * p.T : p.B * p.H)) return;
  const int64_t vec = w / per_group;                              // (batch, query) or (batch, head)
  const int first = (int)(w % per_group) * rows_per_wave, last = min(first + rows_per_wave, group);
  uint32_t best[NPL];
#pragma unroll
  for (int i = 0; i < NPL; ++i) best[i] = 0u;
  for (int g = first; g < last; ++g) {
    // over heads: vec = b T + t, row (b H + g) T + t; over queries: vec = b H + h, row vec T + g
    const int64_t row = p.agg_over_heads ? ((vec / p.T) * p.H + g) * p.T + vec % p.T : vec * p.T + g;
    const float* sc = p.approx + row * NM;
    float x[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) x[i] = (lane + 64 * i < NM) ? sc[lane + 64 * i] : -INFINITY;
    float mx = x[0];
#pragma unroll
    for (int i = 1; i < NPL; ++i) mx = fmaxf(mx, x[i]);
#pragma unroll
    for (int msk = 32; msk >= 1; msk >>= 1) mx = fmaxf(mx, __shfl_xor(mx, msk, 64));
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      if (lane + 64 * i < NM) {
        float d = x[i] - mx;
        asm volatile("" : "+v"(d));                               // the product below stays a product
        x[i] = exp2_contract(d * kLog2e);
        sum += x[i];
      }
    }
#pragma unroll
    for (int msk = 32; msk >= 1; msk >>= 1) sum = sum + __shfl_xor(sum, msk, 64);
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      if (lane + 64 * i < NM) {
        const float pr = __fdiv_rn(x[i], sum);
        const uint32_t bits = p.prob32 ? __float_as_uint(pr) : (model_is_bf16 ? prob_bits<bf16_t>(pr) : prob_bits<f16_t>(pr));
        best[i] = max(best[i], bits);
      }
    }
  }
  uint32_t* agg = p.agg + vec * NM;
#pragma unroll
  for (int i = 0; i < NPL; ++i)
    if (lane + 64 * i < NM) atomicMax(agg + lane + 64 * i, best[i]);
}

// The same for vectors of any length: one wave per row, the row's exponentials written back over its scores.
__global__ __launch_bounds__(256) void lmk_block_prob_long_kernel(RetrParams p, int model_is_bf16) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= (int64_t)p.B * p.H * p.T) return;
  const int bh = (int)(row / p.T), t = (int)(row % p.T), b = bh / p.H;
  const int NM = p.num_mems;
  float* sc = p.approx + row * NM;                                // this row's scores, then its exponentials
  float mx = -INFINITY;
  for (int m = lane; m < NM; m += 64) mx = fmaxf(mx, sc[m]);
#pragma unroll
  for (int msk = 32; msk >= 1; msk >>= 1) mx = fmaxf(mx, __shfl_xor(mx, msk, 64));
  float sum = 0.f;
  for (int m = lane; m < NM; m += 64) {
    float d = sc[m] - mx;
    asm volatile("" : "+v"(d));                                   // the product below stays a product
    const float e = exp2_contract(d * kLog2e);
    sc[m] = e;
    sum += e;
  }
#pragma unroll
  for (int msk = 32; msk >= 1; msk >>= 1) sum = sum + __shfl_xor(sum, msk, 64);
  uint32_t* agg = p.agg + (int64_t)(p.agg_over_heads ? b * p.T + t : bh) * NM;
  for (int m = lane; m < NM; m += 64) {
    const float pr = __fdiv_rn(sc[m], sum);
    const uint32_t bits = p.prob32 ? __float_as_uint(pr) : (model_is_bf16 ? prob_bits<bf16_t>(pr) : prob_bits<f16_t>(pr));
    atomicMax(agg + m, bits);
  }
}

// One workgroup per (batch, head): the k best blocks of agg under (value desc, index asc), ascending.
// Four waves bring the head's vector into LDS (and write the copy the caller may have asked for); the
// first wave then picks k times over it.  Vectors too long for the LDS buffer are read in place.
constexpr int kSelectLds = 8192;                                  // words of the LDS copy

__global__ __launch_bounds__(256) void lmk_block_select_kernel(RetrParams p) {
  __shared__ uint32_t cached[kSelectLds];
  const int tid = threadIdx.x, lane = tid & 63, bh = blockIdx.x, NM = p.num_mems;
  const uint32_t* agg = p.agg + (int64_t)bh * NM;
  const bool in_lds = NM <= kSelectLds;                           // uniform
  for (int m = tid; m < NM; m += 256) {
    const uint32_t v = agg[m];
    if (in_lds) cached[m] = v;
    if (p.agg_out != nullptr) p.agg_out[(int64_t)bh * NM + m] = (uint16_t)v;   // the head's vector itself, in the model dtype
  }
  __syncthreads();
  if (tid >= 64) return;
  int mine = -1;
  float pv = INFINITY;
  int pi = -1;
  for (int j = 0; j < p.k; ++j) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int m = lane; m < NM; m += 64) {
      const uint32_t u = in_lds ? cached[m] : agg[m];
      const float x = p.prob32 ? __uint_as_float(u) : (float)u;   // 16-bit patterns as numbers: exact, order-preserving
      const bool after = (x < pv) || (x == pv && m > pi);
      if (after && (x > bv || (x == bv && m < bi))) {
        bv = x;
        bi = m;
      }
    }
    wave_best(bv, bi);
    pv = bv;
    pi = bi;
    if (lane == j) mine = bi;
  }
  write_ascending(p.idx + (int64_t)bh * p.k, mine, lane, p.k, p.num_mems, p.ring_start);
}

// ---------------------------------------------------------------------------
// fused score + select: the approximate scores of 32 query rows never leave the CU
// ---------------------------------------------------------------------------
// A workgroup (16 waves) owns 32 consecutive query rows of one (batch, head) and walks the cached blocks
// in segments of at most kFusedMaxMems:
//   score   the waves split the segment's landmarks; S = Q LK^T by MFMA with the landmark in the lane,
//           so a register (= one query row) lands in 32 consecutive LDS words
//   select  each wave takes 2 of the rows in turn; a lane holds the 16 scores m = 64 j + lane of the
//           row in registers: bracket, k-th best lower end, exact re-evaluation of the contenders
//           (written back over their approximate score), k best
//   merge   (more than one segment) a row's k best are the k best of the segments' k best: lane j of the
//           row's wave keeps the j-th best (score, index) so far and every segment's picks are inserted
//           in order; ascending index order at the end
// The bracket uses a cheap monotone over-/under-estimate of the rounding contract: round_T(x) / sqrt(hd)
// is replaced by a multiplication by the rounded reciprocal, pushed outwards by 2^-21 relative (the
// product is within 2^-22 of the correctly rounded quotient) before the final rounding.  That only
// adds contenders; the ranking itself uses the exact contract.
constexpr int kFusedMaxMems = 1024;
constexpr int kFusedRows = 32;
constexpr int kFusedWaves = 16;
constexpr int kFusedList = 64;                                    // a row's contender list: what one pass of the exact evaluation takes

template <class T, int D, bool SEGMENTS>
__global__ __launch_bounds__(64 * kFusedWaves) void lmk_topk_fused_kernel(RetrParams p) {
  constexpr int KS = D / 16;
  constexpr int NJ = kFusedMaxMems / 64;                          // scores per lane and row
  extern __shared__ __align__(16) unsigned char smem[];
  const int NMall = p.num_mems;
  constexpr int NMp = kFusedMaxMems + 8;                          // row stride (words): the two half-waves of a store (rows 4
                                                                  // apart) then hit different banks; a constant, so that the
                                                                  // sixteen stores of a tile share their address registers
  float* sc = (float*)smem;                                       // [32][NMp]
  float* q_lds = sc + kFusedRows * NMp;                           // [32][D]: the query rows in fp32
  unsigned short* cand = (unsigned short*)(q_lds + kFusedRows * D);   // [32][kFusedList]: a row's contenders (index in the segment)
  unsigned char* q_raw = (unsigned char*)(cand + kFusedRows * kFusedList);    // [32][D] in the model dtype, rows of QROWB bytes
  constexpr int QROWB = 2 * D + 16;                               // 16 lanes reading 16 B of 16 rows hit every bank once
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // in a scalar register: what depends on it alone is scalar too
  const int ql = lane & 31, h = lane >> 5;
  const int n_qt = (p.T + kFusedRows - 1) / kFusedRows;
  // Workgroups go to the eight XCDs in turn; the ones that read the same head's landmark keys are put on
  // one XCD, so the keys come out of HBM once rather than once per L2.
  const int wg = (gridDim.x & 7) ? (int)blockIdx.x : (int)((blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3));
  const int bh = wg / n_qt, t0 = (wg % n_qt) * kFusedRows;
  const int b = bh / p.H, hh = bh % p.H;
  const char* qp = (const char*)p.q + 2 * (b * p.qs_b + hh * p.qs_h);
  const char* lk_all = (const char*)p.lk_rot + (int64_t)bh * lk_tiles(NMall) * lk_tile_bytes(D);
  const float* lkn_all = p.lk_norm + (int64_t)bh * NMall;

  // ---- the 32 query rows -> LDS (MFMA operand of the score phase; the select phase reads them from there too):
  // requested behind the first segment's landmark keys, so that one memory round trip lies in front of the first MFMA
  static_assert(kFusedRows * (D / 8) <= 64 * kFusedWaves && kFusedRows * (D / 8) % 64 == 0, "one chunk of the query rows per thread, whole waves");
  // running k best of every row this wave owns (rows wave, wave + 16): lane j holds the j-th best so far
  float run_v[kFusedRows / kFusedWaves];
  int run_i[kFusedRows / kFusedWaves];
#pragma unroll
  for (int i = 0; i < kFusedRows / kFusedWaves; ++i) {
    run_v[i] = -INFINITY;
    run_i[i] = 0x7fffffff;
  }
  // ---- the cached blocks in segments of at most kFusedMaxMems: a row's k best are the k best of the
  // segments' k best, merged under the same order
  for (int seg = 0; seg < NMall; seg += kFusedMaxMems) {
    const int NM = min(NMall - seg, kFusedMaxMems);                 // landmarks of this segment
    const int NMr = (NM + 63) & ~63;                                // columns read by the select phase
    const char* lk = lk_all + lk_key_offset(seg, D);                // a segment starts a tile
    const float* lkn = lkn_all + seg;
    float nrm[NJ];                                                  // |k_m| of this lane's landmarks, for the select phase:
#pragma unroll                                                     // requested with the keys
    for (int j = 0; j < NJ; ++j) {
      const int m = 64 * j + lane;
      nrm[j] = (m < NM) ? lkn[m] : 0.f;
    }
    // ---- score: A = query rows (lane -> row, from LDS), B = landmark keys (lane -> landmark).  A wave's tiles are
    // 32 * kFusedWaves landmarks apart, at most two per segment, and both are requested before the first is used.
    // MFMA step ks takes chunks 2 ks, 2 ks + 1 of the landmark in the lane: one load instruction reads 1 KB in a row.
    {
      constexpr int NT = kFusedMaxMems / (32 * kFusedWaves);
      u32x4_t kf[NT][KS];
#pragma unroll
      for (int it = 0; it < NT; ++it) {
        const int m0 = 32 * wave + 32 * kFusedWaves * it;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          u32x4_t z = {0, 0, 0, 0};
          kf[it][ks] = z;
          if (m0 < NM) kf[it][ks] = *(const u32x4_t*)(lk + lk_key_offset(m0 + ql, D) + 512 * (2 * ks + h));
        }
      }
      if (seg == 0) {
        if (wave < kFusedRows * (D / 8) / 64) {                     // wave-uniform
          u32x4_t q_chunk = {0, 0, 0, 0};
          if (t0 + tid / (D / 8) < p.T)
            q_chunk = *(const u32x4_t*)(qp + 2 * ((int64_t)(t0 + tid / (D / 8)) * p.qs_r + 8 * (tid % (D / 8))));
          *(u32x4_t*)(q_raw + (tid / (D / 8)) * QROWB + 16 * (tid % (D / 8))) = q_chunk;
        }
        __syncthreads();
      }
#pragma unroll
      for (int it = 0; it < NT; ++it) {
        const int m0 = 32 * wave + 32 * kFusedWaves * it;
        if (m0 < NMr) {                                             // wave-uniform
          const int m = m0 + ql;
          f32x16_t s;
#pragma unroll
          for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            s = mfma32<T>(*(const u32x4_t*)(q_raw + ql * QROWB + 32 * ks + 16 * h), kf[it][ks], s);
          // register r belongs to query row 8 (r / 4) + 4 h + r % 4: four address registers, made here and not kept,
          // and the row within the four as the store's immediate offset (the score tile starts the LDS, at byte 0)
          int base0 = (4 * h * NMp + m) * 4;
          asm volatile("" : "+v"(base0));                           // opaque: what follows is computed here, each time
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            const int base = base0 + 8 * a * NMp * 4;
#pragma unroll
            for (int b = 0; b < 4; ++b) lds_st32(base + b * NMp * 4, (m < NM) ? s[4 * a + b] : -INFINITY);
          }
        }
      }
    }
    __syncthreads();

    // ---- select.  A wave owns the rows wave and wave + 16: bracket, threshold and contender list of each, then
    // ONE exact evaluation for the contenders of both (a lane per contender: the two short lists share a pass),
    // then the k best of each.
    const float sq = p.sqrt_hd, inv_sq = 1.0f / sq;
    const int nj = NMr >> 6;                                        // slices in use (wave-uniform)
    constexpr int RPW = kFusedRows / kFusedWaves;
    static_assert(RPW == 2, "two rows per wave");
    auto row_of = [&](int ri) { return wave + kFusedWaves * ri; };

    // wave-wide arg-best of v[] under (value desc, index asc); the winner's slot is set to -inf
    auto take_best = [&](float* v, float& bv_out, int& bi_out) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
#pragma unroll
      for (int j = 0; j < NJ; ++j)
        if (j < nj && v[j] > bv) {                                  // ascending j = ascending index: strict > keeps the first
          bv = v[j];
          bi = 64 * j + lane;
        }
      wave_best(bv, bi);
      const int win = __builtin_amdgcn_readfirstlane(bi);
      const bool owner = lane == (win & 63);
#pragma unroll
      for (int j = 0; j < NJ; ++j) v[j] = (owner && j == (win >> 6)) ? -INFINITY : v[j];
      bv_out = bv;
      bi_out = win;
    };

    // the same with one candidate (value v, index id, unique in the wave) per lane
    auto take_one = [&](float& v, int id, float& bv_out, int& bi_out) {
      wave_best_one(v, id, bv_out, bi_out);
      if (bi_out == id) v = -INFINITY;
    };

    // exact scores of the first cA contenders of row riA and the first cB of row riB, one lane per contender,
    // written over their approximate scores
    auto evaluate = [&](int cA, int riA, int cB, int riB) {
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_s_waitcnt(0xc07f);                           // this wave's LDS writes (q rows, lists) are visible
      for (int c0 = 0; c0 < cA + cB; c0 += 64) {
        const int c = c0 + lane;
        if (c < cA + cB) {
          const bool second = c >= cA;
          const int qi = row_of(second ? riB : riA);
          const int m = cand[qi * kFusedList + (second ? c - cA : c)];
          const float* qrow = q_lds + qi * D;
          const char* kr = lk + lk_key_offset(m, D);
          float acc = 0.f;
#pragma unroll
          for (int g = 0; g < D / 64; ++g) {                        // 8 loads in flight, then their 64 dependent fmas
            u32x4_t kv[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) kv[i] = *(const u32x4_t*)(kr + 512 * (8 * g + i));
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              const u32x4_t kk = kv[i];
              const float4 qa = *(const float4*)&qrow[8 * (8 * g + i)];
              const float4 qb = *(const float4*)&qrow[8 * (8 * g + i) + 4];
              acc = __builtin_fmaf(qa.x, unpack_lo<T>(kk[0]), acc);
              acc = __builtin_fmaf(qa.y, unpack_hi<T>(kk[0]), acc);
              acc = __builtin_fmaf(qa.z, unpack_lo<T>(kk[1]), acc);
              acc = __builtin_fmaf(qa.w, unpack_hi<T>(kk[1]), acc);
              acc = __builtin_fmaf(qb.x, unpack_lo<T>(kk[2]), acc);
              acc = __builtin_fmaf(qb.y, unpack_hi<T>(kk[2]), acc);
              acc = __builtin_fmaf(qb.z, unpack_lo<T>(kk[3]), acc);
              acc = __builtin_fmaf(qb.w, unpack_hi<T>(kk[3]), acc);
            }
          }
          sc[qi * NMp + m] = contract<T>(acc, sq);
        }
      }
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_s_waitcnt(0xc07f);
    };

    // what a row leaves for the steps behind its list: entries still in the list, whether the list was emptied
    // on the way, the slices of this lane that hold a contender
    int left[RPW] = {0, 0};
    bool flushed[RPW] = {false, false};
    uint32_t is_c[RPW] = {0u, 0u};
#pragma unroll 1
    for (int ri = 0; ri < RPW; ++ri) {
      const int qi = row_of(ri);
      if (t0 + qi >= p.T) break;                                    // wave-uniform
      // q row -> fp32 in LDS (read back by the evaluation), and its norm
      const unsigned char* qr = q_raw + qi * QROWB;
      float* qrow_lds = q_lds + qi * D;
      float qn = 0.f;
      for (int d = 2 * lane; d < D; d += 128) {
        const uint32_t u = *(const uint32_t*)(qr + 2 * d);
        const float x0 = unpack_lo<T>(u), x1 = unpack_hi<T>(u);
        qrow_lds[d] = x0;
        qrow_lds[d + 1] = x1;
        qn += x0 * x0 + x1 * x1;
      }
#pragma unroll
      for (int m = 32; m >= 1; m >>= 1) qn += __shfl_xor(qn, m, 64);
      const float eps_q = sqrtf(qn) * 1.000001f * (1.0f / 16384.0f);

      const float* srow = sc + qi * NMp;
      // raw bracket of the fp32 dot product: [a - e, a + e] around the MFMA score a.  The contract (round, divide,
      // round) is monotone, and so are the outward-rounded estimates T_lo / T_hi of it below, so the order
      // statistics are taken on the raw ends and only the few values that matter go through T_lo / T_hi.
      float up[NJ];
      float lm = -INFINITY;                                         // this lane's best raw lower end
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        up[j] = -INFINITY;
        if (j < nj) {
          const float a = srow[64 * j + lane];
          const float e = eps_q * nrm[j];
          up[j] = a + e;                                            // -inf (no landmark) stays -inf
          lm = fmaxf(lm, a - e);
        }
      }
      auto t_lo = [&](float x) {
        const float cl = round_to<T>(x) * inv_sq;
        return round_to<T>(cl - fabsf(cl) * 4.76837158203125e-7f);
      };
      auto t_hi = [&](float x) {
        const float ch = round_to<T>(x) * inv_sq;
        return round_to<T>(ch + fabsf(ch) * 4.76837158203125e-7f);
      };
      // tau = T_lo of the k-th best of the lanes' best lower ends: k different blocks reach it, so the k-th best
      // exact score does too (a little below the k-th best lower end itself, and k times cheaper to find)
      float tau_raw = -INFINITY;
      for (int j = 0; j < p.k; ++j) {
        int bi;
        take_one(lm, lane, tau_raw, bi);
      }
      const float tau = t_lo(tau_raw);
      // T_hi(x) >= tau needs x >= tau_raw up to the roundings of both estimates (two roundings to 8 or 11 bits
      // each, 3 % covers them; 1e-5 covers the subnormal range): everything below theta is out without being rounded
      const float theta = tau_raw - (fabsf(tau_raw) * 0.03f + 1e-5f);
      // contenders: upper end reaches tau.  They go into the row's list, which holds what one pass of the exact
      // evaluation takes; the seldom row with more is evaluated here, a list at a time.
      unsigned short* cnd = cand + qi * kFusedList;
      uint32_t mine_c = 0;
      int count = 0;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if (j < nj && __any(up[j] >= theta && up[j] > -INFINITY)) {   // wave-uniform: most slices hold no contender
          const bool c = up[j] >= theta && up[j] > -INFINITY && t_hi(up[j]) >= tau;
          const uint64_t bal = __ballot(c);
          const int at = count + __popcll(bal & ((1ull << lane) - 1));
          if (c) {
            if (at < kFusedList) cnd[at] = (unsigned short)(64 * j + lane);
            mine_c |= 1u << j;
          }
          count += __popcll(bal);
        }
      }
      bool emptied = false;                                         // wave-uniform
      if (count > kFusedList) {
        const int total = count;
#pragma unroll 1
        for (int first = 0; first < total; first += kFusedList) {   // contenders first .. first + 63, in the order of above
          __builtin_amdgcn_wave_barrier();                          // the list has been read
          int seen = 0;
#pragma unroll
          for (int j = 0; j < NJ; ++j) {
            const bool c = (mine_c >> j) & 1;
            const uint64_t bal = __ballot(c);
            const int at = seen + __popcll(bal & ((1ull << lane) - 1)) - first;
            if (c && at >= 0 && at < kFusedList) cnd[at] = (unsigned short)(64 * j + lane);
            seen += __popcll(bal);
          }
          evaluate(min(total - first, kFusedList), ri, 0, ri);
        }
        count = 0;
        emptied = true;
      }
      if (ri == 0) {
        left[0] = count;
        flushed[0] = emptied;
        is_c[0] = mine_c;
      } else {
        left[1] = count;
        flushed[1] = emptied;
        is_c[1] = mine_c;
      }
    }
    if (left[0] + left[1] > 0) evaluate(left[0], 0, left[1], 1);

#pragma unroll 1
    for (int ri = 0; ri < RPW; ++ri) {
      const int qi = row_of(ri);
      const int t = t0 + qi;
      if (t >= p.T) break;                                          // wave-uniform
      const float* srow = sc + qi * NMp;
      const int count = ri == 0 ? left[0] : left[1];
      const bool emptied = ri == 0 ? flushed[0] : flushed[1];
      const uint32_t mine_c = ri == 0 ? is_c[0] : is_c[1];
      // k best exact scores, best first, handed to `use`: in a single segment they are the row's (written
      // in ascending index order), otherwise each is inserted into the row's running list
      auto consume = [&](auto&& pick) {
        if constexpr (!SEGMENTS) {
          int mine = -1;                                           // lane j keeps the j-th pick
          for (int j = 0; j < p.k; ++j) {
            float bv;
            int bi;
            pick(bv, bi);
            if (lane == j) mine = bi;
          }
          write_ascending(p.idx + ((int64_t)bh * p.T + t) * p.k, mine, lane, p.k, p.num_mems, p.ring_start);
        } else {
          float rv = ri == 0 ? run_v[0] : run_v[1];
          int rx = ri == 0 ? run_i[0] : run_i[1];
          for (int j = 0; j < p.k; ++j) {
            float bv;
            int bi;
            pick(bv, bi);
            if (!(bv > -INFINITY)) break;                           // fewer than k landmarks in this segment (wave-uniform)
            bi += seg;
            const bool better = lane < p.k && (rv > bv || (rv == bv && rx < bi));   // a prefix of the sorted list
            const int pos = __popcll(__ballot(better));
            if (pos >= p.k) break;                                  // worse than the k kept: so are the rest
            const float up_v = __shfl_up(rv, 1, 64);
            const int up_i = __shfl_up(rx, 1, 64);
            if (lane > pos) {
              rv = up_v;
              rx = up_i;
            } else if (lane == pos) {
              rv = bv;
              rx = bi;
            }
          }
          if (ri == 0) {
            run_v[0] = rv;
            run_i[0] = rx;
          } else {
            run_v[1] = rv;
            run_i[1] = rx;
          }
        }
      };
      if (!emptied) {                                               // the usual case: few contenders, still in the list
        float cv = -INFINITY;
        int ci = 0x7fffffff;
        if (lane < count) {
          ci = cand[qi * kFusedList + lane];
          cv = srow[ci];
        }
        consume([&](float& bv, int& bi) { take_one(cv, ci, bv, bi); });
      } else {                                                      // exact scores picked up from the row, 16 per lane
        float x[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) x[j] = (j < nj && ((mine_c >> j) & 1)) ? srow[64 * j + lane] : -INFINITY;
        consume([&](float& bv, int& bi) { take_best(x, bv, bi); });
      }
    }
    __syncthreads();                                                // the next segment overwrites the score tile
  }

  // ---- ascending order of the k kept blocks
  if constexpr (!SEGMENTS) return;
  for (int qi = wave, ri = 0; qi < kFusedRows; qi += kFusedWaves, ++ri) {
    const int t = t0 + qi;
    if (t >= p.T) break;
    int mine = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < kFusedRows / kFusedWaves; ++i)
      if (i == ri) mine = run_i[i];
    write_ascending(p.idx + ((int64_t)bh * p.T + t) * p.k, mine, lane, p.k, p.num_mems, p.ring_start);
  }
}

// ---------------------------------------------------------------------------
// select without the bracket, for a handful of query rows (decoding): see lmk_topk_slice.hpp
// ---------------------------------------------------------------------------
template <class T, int D>
__global__ __launch_bounds__(64 * kSliceWaves) void lmk_topk_slice_kernel(RetrParams p, int n_slices) {
  __shared__ __align__(16) unsigned char lds[kSliceLdsBytes];
  topk_slice_body<T, D>(p, n_slices, (int)blockIdx.x, lds);
}

// One wave per query row: the k best of the row's n_slices * k candidates, written in ascending index order.
__global__ __launch_bounds__(256) void lmk_topk_slice_merge_kernel(RetrParams p, int n_slices) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= (int64_t)p.B * p.H * p.T) return;                      // wave-uniform
  const int mine = merge_slices_row(p, n_slices, row, lane);
  write_ascending(p.idx + row * p.k, mine, lane, p.k, p.num_mems, p.ring_start);
}

// ---------------------------------------------------------------------------
// gather + attend over the selected blocks, merged with the local-chunk attention
// ---------------------------------------------------------------------------
__device__ __forceinline__ float sum8(float d) {                  // sum over the 8 lanes of a key group (lane & 7)
  d += dpp_f<0xB1>(d);                                            // quad_perm [1,0,3,2]
  d += dpp_f<0x4E>(d);                                            // quad_perm [2,3,0,1]
  d += dpp_f<0x141>(d);                                           // row_half_mirror
  return d;
}

// One wave per query row.  Eight lanes share a key: lane j of the group holds head dims 8j..8j+7 and
// 64+8j..64+8j+7 (head dim 128; 4j..4j+3 and 32+4j..32+4j+3 at head dim 64), i.e. both partners of the rotary pair, so the rotation needs no exchange between
// lanes; the eight key groups of the wave take keys g, g+8, .. of a block.  Rotation and scores are
// evaluated in fp32 from the 16-bit cache and table values (the reference rounds the rotated key to
// the model dtype first; the difference is far inside the 2e-2 bound of this step, and selection --
// where bits matter -- does not go through here).
// A block passes through the registers in chunks of at most 64 keys -- first the keys of every chunk
// (scores of the whole block, which the block's softmax needs before any weight is final), then the
// values, so keys and values are never live together and the kernel keeps several waves per SIMD.  The
// loads of the next chunk are issued before the arithmetic on the current one.
// PADDED: the cache's blocks hold p.block < BS tokens (the benchmark models' 51).  A block is then worked on in BS
// slots: slot s < p.block - 1 is normal key s, the last slot is the landmark (token p.block - 1), the slots in
// between re-read a normal key and get the score -inf, i.e. weight 0 in the block's softmax and in the output.
// The picked blocks of a row are read at p.idx[b * idx_sb + h * idx_sh + t * idx_st + 0 .. k-1] (selections shared
// by the heads or by the queries have a zero stride there); a block counts among the k newest, whose keys sit one
// block further on, by its age in the ring (p.ring_start = slot of the oldest block, 0 for a flat cache).
template <int E> struct PieceVec;
template <> struct PieceVec<8> { using type = u32x4_t; };
template <> struct PieceVec<4> { using type = u32x2_t; };

// MERGE: the row's blocks are picked from the slices' candidates first (p.merge_slices > 0); a template parameter
// because the four registers it holds on to would cost the plain kernel its third wave per SIMD (172 against 168).
// LOCAL: the row's local window -- the tokens of the cache behind its last complete block and the new tokens up to
// the row's own, at most one block together -- is attended to here as well, as one more item of the row's online
// softmax, instead of coming in as (o_loc, L_loc, M_loc) from a forward launch over a window another launch built:
// a decode step is then the selection and this kernel.  Its keys join the global bucket directly (own-block rule:
// causal, the landmark token does not see itself; flash_landmark_attention.py:78-100).
// With SPLIT the window has a fifth wave of its own (blocks of 128 keep four waves, whose registers the kernel needs:
// there the window goes to the wave next in turn behind the blocks).
template <class T, int D, int BS, bool SPLIT, bool PADDED, bool MERGE = false, bool LOCAL = false>
__global__ __launch_bounds__((SPLIT && LOCAL && BS <= 64) ? 320 : 256) void lmk_gather_attend_kernel(RetrParams p) {
  constexpr int NWV = (SPLIT && LOCAL && BS <= 64) ? 5 : 4;      // waves of a workgroup
  static_assert((D == 128 || D == 64) && (BS == 32 || BS % 64 == 0), "8 lanes x 2 pieces per row; whole chunks of keys");
  static_assert(!LOCAL || !PADDED, "the local window sits in a block of BS tokens");
  constexpr int E = D / 16;                                       // head dims per lane and rotary half: 8 or 4
  constexpr int PB = 2 * E;                                       // bytes of one piece
  using vec_t = typename PieceVec<E>::type;                       // one piece: E 16-bit values
  constexpr int CK = BS < 64 ? BS : 64;                           // keys per chunk
  constexpr int KPG = CK / 8;                                     // keys per 8-lane group and chunk
  constexpr int NC = BS / CK;                                     // chunks per block
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int j = lane & 7, g = lane >> 3;                           // head-dim chunk pair, key group
  // (bh, t): a wave's own row, or -- SPLIT, for launches with few rows -- the workgroup's row, whose
  // selected blocks the four waves share out (block js goes to wave js % 4) and merge at the end
  const int64_t row = SPLIT ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + wave;
  if (row >= (int64_t)p.B * p.H * p.T) return;                    // SPLIT: the whole workgroup leaves
  const int js0 = SPLIT ? (wave < 4 ? wave : p.k) : 0, jstep = SPLIT ? 4 : 1;   // (the window's wave takes no block)
  const int bh = (int)(row / p.T), t = (int)(row % p.T);
  const int b = bh / p.H, hh = bh % p.H;

  auto unpack8 = [](const vec_t u, float* o) {
#pragma unroll
    for (int i = 0; i < E / 2; ++i) {
      o[2 * i] = unpack_lo<T>(u[i]);
      o[2 * i + 1] = unpack_hi<T>(u[i]);
    }
  };
  float qlo[E], qhi[E];
  {
    const char* qp = (const char*)p.q + 2 * (b * p.qs_b + hh * p.qs_h + (int64_t)t * p.qs_r);
    unpack8(*(const vec_t*)(qp + PB * j), qlo);
    unpack8(*(const vec_t*)(qp + D + PB * j), qhi);
  }
  const char* kc = (const char*)p.kcache + 2 * (b * p.kcs_b + hh * p.kcs_h);
  const char* vc = (const char*)p.vcache + 2 * (b * p.vcs_b + hh * p.vcs_h);
  const float c2 = p.scale_log2;
  const int nreal = PADDED ? p.block : BS;                        // tokens of a block in the cache
  auto token_of = [&](int slot) {                                 // slot of the block's BS -> token of the block it reads
    if (!PADDED) return slot;
    return slot == BS - 1 ? nreal - 1 : min(slot, nreal - 2);
  };
  const int64_t* idx_row = p.idx + (b * p.idx_sb + hh * p.idx_sh + (int64_t)t * p.idx_st);
  // The decode-time selection leaves a row's candidates (k per slice of the cache) rather than its indices: the wave
  // picks the k best first -- lane r of `sorted` gets the r-th block in the order of the output -- and one wave per
  // row writes them where the caller expects the indices.
  constexpr bool merged = MERGE;
  int sorted = 0;
  if constexpr (MERGE) {
    int mine = merge_slices_row(p, p.merge_slices, row, lane);
    const int rank = rank_ascending(mine, lane, p.k, p.num_mems, p.ring_start);
    sorted = __builtin_amdgcn_ds_permute(4 * (lane < p.k ? rank : lane), mine);
    if (lane < p.k && (!SPLIT || wave == 0)) p.idx[b * p.idx_sb + hh * p.idx_sh + (int64_t)t * p.idx_st + rank] = (int64_t)mine;
  }
  auto picked = [&](int js) {                                      // idx is a caller's array: never read outside the cache
    return merged ? __shfl(sorted, js, 64) : min(max((int)idx_row[js], 0), p.num_mems - 1);
  };
  auto newest = [&](int blk) {                                    // one of the k newest blocks: its keys sit one block further on
    int age = blk - p.ring_start;
    age += age < 0 ? p.num_mems : 0;
    return age >= p.num_mems - p.k;
  };

  float Mrun = -INFINITY, lrun = 0.f;
  float alo[E], ahi[E];
#pragma unroll
  for (int i = 0; i < E; ++i) {
    alo[i] = 0.f;
    ahi[i] = 0.f;
  }

  // one chunk = CK rows of K or of V: this lane's KPG rows (g, g+8, ..) x its two 16-byte pieces
  vec_t clo[KPG], chi[KPG], nlo[KPG], nhi[KPG];
  auto fetch = [&](const char* base, int64_t row_stride, int64_t key0, int slot0) {
#pragma unroll
    for (int i = 0; i < KPG; ++i) {
      const char* r = base + 2 * ((key0 + token_of(slot0 + g + 8 * i)) * row_stride) + PB * j;
      nlo[i] = *(const vec_t*)(r);
      nhi[i] = *(const vec_t*)(r + D);
    }
  };
  auto take = [&]() {
#pragma unroll
    for (int i = 0; i < KPG; ++i) {
      clo[i] = nlo[i];
      chi[i] = nhi[i];
    }
  };
  if constexpr (LOCAL) {
    if (!SPLIT || wave == (NWV == 5 ? 4 : (p.k & 3))) {
      const int inc = p.local_inc, own = inc + t;                 // window rows: inc of the cache, then the new tokens
      const char* kn = (const char*)p.k_new + 2 * (b * p.kns_b + hh * p.kns_h);
      const char* vn = (const char*)p.v_new + 2 * (b * p.vns_b + hh * p.vns_h);
      float s_loc[KPG * NC];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        if (CK * c > own) {                                       // a chunk behind the row's own token (wave-uniform)
#pragma unroll
          for (int i = 0; i < KPG; ++i) s_loc[KPG * c + i] = -INFINITY;
          continue;
        }
#pragma unroll
        for (int i = 0; i < KPG; ++i) {
          const int r = CK * c + g + 8 * i;
          const bool visible = r <= own && !(r == BS - 1 && own == BS - 1);
          const int rc = min(r, own);                             // rows behind the row's own are never read
          const bool cached = rc < inc;
          const char* kr = (cached ? kc + 2 * ((p.local_row0 + rc) * p.kcs_r) : kn + 2 * ((int64_t)(rc - inc) * p.kns_r)) + PB * j;
          const int64_t pos = inc > 0 ? p.local_pos0 + min(rc, inc - 1) : 0;   // a position the tables hold, used by cached rows only
          const char* cr = (const char*)p.cos + 2 * (pos * p.cs_r) + PB * j;
          const char* sr = (const char*)p.sin + 2 * (pos * p.cs_r) + PB * j;
          float kl[E], kh[E], cl[E], ch[E], sl[E], sh[E];
          unpack8(*(const vec_t*)(kr), kl);
          unpack8(*(const vec_t*)(kr + D), kh);
          unpack8(*(const vec_t*)(cr), cl);
          unpack8(*(const vec_t*)(cr + D), ch);
          unpack8(*(const vec_t*)(sr), sl);
          unpack8(*(const vec_t*)(sr + D), sh);
          float d = 0.f;
#pragma unroll
          for (int e = 0; e < E; ++e) {                           // cached keys are rotated in the model dtype, as the cache's
            const float rl = cached ? round_to<T>(__builtin_fmaf(kl[e], cl[e], -kh[e] * sl[e])) : kl[e];   // window is (llama_mem.py:336-338)
            const float rh = cached ? round_to<T>(__builtin_fmaf(kh[e], ch[e], kl[e] * sh[e])) : kh[e];
            d = __builtin_fmaf(qlo[e], rl, d);
            d = __builtin_fmaf(qhi[e], rh, d);
          }
          s_loc[KPG * c + i] = visible ? sum8(d) * c2 : -INFINITY;
        }
      }
      float mx = s_loc[0];                                        // row 0 is always visible
#pragma unroll
      for (int i = 1; i < KPG * NC; ++i) mx = fmaxf(mx, s_loc[i]);
      mx = fmaxf(mx, dpp_f<0x128>(mx));
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      float den = 0.f;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        if (CK * c > own) continue;
#pragma unroll
        for (int i = 0; i < KPG; ++i) {
          const int rc = min(CK * c + g + 8 * i, own);
          const bool cached = rc < inc;
          const char* vr = (cached ? vc + 2 * ((p.local_row0 + rc) * p.vcs_r) : vn + 2 * ((int64_t)(rc - inc) * p.vns_r)) + PB * j;
          const vec_t vlo = *(const vec_t*)(vr), vhi = *(const vec_t*)(vr + D);
          const float e = fast_exp2(s_loc[KPG * c + i] - mx);
          den += e;
          const float w = round_to<T>(e);                         // weights enter PV in the model dtype
#pragma unroll
          for (int e2 = 0; e2 < E / 2; ++e2) {
            alo[2 * e2] = __builtin_fmaf(w, unpack_lo<T>(vlo[e2]), alo[2 * e2]);
            alo[2 * e2 + 1] = __builtin_fmaf(w, unpack_hi<T>(vlo[e2]), alo[2 * e2 + 1]);
            ahi[2 * e2] = __builtin_fmaf(w, unpack_lo<T>(vhi[e2]), ahi[2 * e2]);
            ahi[2 * e2 + 1] = __builtin_fmaf(w, unpack_hi<T>(vhi[e2]), ahi[2 * e2 + 1]);
          }
        }
      }
      den += dpp_f<0x128>(den);
      den += __shfl_xor(den, 16, 64);
      den += __shfl_xor(den, 32, 64);
      Mrun = mx;
      lrun = den;
    }
  }
  int blk = 0;
  if (js0 < p.k) {
    blk = picked(js0);
    fetch(kc, p.kcs_r, (int64_t)blk * nreal, 0);
  }
  for (int js = js0; js < p.k; js += jstep) {
    const int64_t key0 = (int64_t)blk * nreal;
    const int64_t pos0 = (int64_t)js * nreal + (newest(blk) ? nreal : 0) + p.prefix_len;
    float sc[KPG * NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      take();
      if (c + 1 < NC) fetch(kc, p.kcs_r, key0, CK * (c + 1));
      else fetch(vc, p.vcs_r, key0, 0);
#pragma unroll
      for (int i = 0; i < KPG; ++i) {
        const int slot = CK * c + g + 8 * i;
        const int kk = token_of(slot);
        const char* cr = (const char*)p.cos + 2 * ((pos0 + kk) * p.cs_r) + PB * j;
        const char* sr = (const char*)p.sin + 2 * ((pos0 + kk) * p.cs_r) + PB * j;
        float kl[E], kh[E], cl[E], ch[E], sl[E], sh[E];
        unpack8(clo[i], kl);
        unpack8(chi[i], kh);
        unpack8(*(const vec_t*)(cr), cl);
        unpack8(*(const vec_t*)(cr + D), ch);
        unpack8(*(const vec_t*)(sr), sl);
        unpack8(*(const vec_t*)(sr + D), sh);
        float d = 0.f;
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const float rl = __builtin_fmaf(kl[e], cl[e], -kh[e] * sl[e]);
          const float rh = __builtin_fmaf(kh[e], ch[e], kl[e] * sh[e]);
          d = __builtin_fmaf(qlo[e], rl, d);
          d = __builtin_fmaf(qhi[e], rh, d);
        }
        sc[KPG * c + i] = sum8(d) * c2;                           // log2 domain
        if (PADDED && slot >= nreal - 1 && slot != BS - 1) sc[KPG * c + i] = -INFINITY;   // a slot without a token
      }
    }
    // landmark = key BS-1 = last chunk, group 7, last of the group's keys
    const float t_lm = __shfl(sc[KPG * NC - 1], 56, 64);
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < KPG * NC; ++i)
      if (!(i == KPG * NC - 1 && g == 7)) mx = fmaxf(mx, sc[i]);
    mx = fmaxf(mx, dpp_f<0x128>(mx));                             // row_ror 8: the other key group of the row
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    float den = 0.f;
#pragma unroll
    for (int i = 0; i < KPG * NC; ++i) {
      float e = fast_exp2(sc[i] - mx);
      if (i == KPG * NC - 1 && g == 7) e = 0.f;
      sc[i] = e;
      den += e;
    }
    den += dpp_f<0x128>(den);
    den += __shfl_xor(den, 16, 64);
    den += __shfl_xor(den, 32, 64);
    const float Mnew = fmaxf(Mrun, t_lm);
    const float alpha = fast_exp2(Mrun - Mnew);
    const float gate = fast_exp2(t_lm - Mnew);
    lrun = lrun * alpha + gate;
    Mrun = Mnew;
    const float f = gate / den;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      alo[e] *= alpha;
      ahi[e] *= alpha;
    }
    int blk_next = blk;
    if (js + jstep < p.k) blk_next = picked(js + jstep);
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      take();
      if (c + 1 < NC) fetch(vc, p.vcs_r, key0, CK * (c + 1));
      else if (js + jstep < p.k) fetch(kc, p.kcs_r, (int64_t)blk_next * nreal, 0);
#pragma unroll
      for (int i = 0; i < KPG; ++i) {
        const float w = round_to<T>(sc[KPG * c + i] * f);         // weights enter PV in the model dtype
#pragma unroll
        for (int e = 0; e < E / 2; ++e) {
          alo[2 * e] = __builtin_fmaf(w, unpack_lo<T>(clo[i][e]), alo[2 * e]);
          alo[2 * e + 1] = __builtin_fmaf(w, unpack_hi<T>(clo[i][e]), alo[2 * e + 1]);
          ahi[2 * e] = __builtin_fmaf(w, unpack_lo<T>(chi[i][e]), ahi[2 * e]);
          ahi[2 * e + 1] = __builtin_fmaf(w, unpack_hi<T>(chi[i][e]), ahi[2 * e + 1]);
        }
      }
    }
    blk = blk_next;
  }
#pragma unroll
  for (int e = 0; e < E; ++e) {                                   // sum over the eight key groups
    alo[e] += dpp_f<0x128>(alo[e]);
    ahi[e] += dpp_f<0x128>(ahi[e]);
    alo[e] += __shfl_xor(alo[e], 16, 64);
    ahi[e] += __shfl_xor(ahi[e], 16, 64);
    alo[e] += __shfl_xor(alo[e], 32, 64);
    ahi[e] += __shfl_xor(ahi[e], 32, 64);
  }
  if constexpr (SPLIT) {                                          // the four waves' partial (M, l, acc) -> wave 0
    __shared__ float part_acc[NWV][D];
    __shared__ float part_ml[NWV][2];
    if (g == 0) {
#pragma unroll
      for (int e = 0; e < E; ++e) {
        part_acc[wave][E * j + e] = alo[e];
        part_acc[wave][D / 2 + E * j + e] = ahi[e];
      }
      if (j == 0) {
        part_ml[wave][0] = Mrun;
        part_ml[wave][1] = lrun;
      }
    }
    __syncthreads();
    if (wave != 0) return;
    float Mall = part_ml[0][0];                                   // wave 0 always has a block (k >= 1)
#pragma unroll
    for (int w = 1; w < NWV; ++w) Mall = fmaxf(Mall, part_ml[w][0]);
    lrun = 0.f;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      alo[e] = 0.f;
      ahi[e] = 0.f;
    }
#pragma unroll
    for (int w = 0; w < NWV; ++w) {
      const float sw = fast_exp2(part_ml[w][0] - Mall);           // 0 for a wave without blocks (M = -inf)
      lrun = __builtin_fmaf(part_ml[w][1], sw, lrun);
#pragma unroll
      for (int e = 0; e < E; ++e) {
        alo[e] = __builtin_fmaf(part_acc[w][E * j + e], sw, alo[e]);
        ahi[e] = __builtin_fmaf(part_acc[w][D / 2 + E * j + e], sw, ahi[e]);
      }
    }
    Mrun = Mall;
  }
  if constexpr (LOCAL) {                                          // the local window is in the sums already
    const float inv = 1.0f / lrun;
    if (g == 0) {
      char* outp = (char*)p.out + 2 * (b * p.outs_b + hh * p.outs_h + (int64_t)t * p.outs_r) + PB * j;
      vec_t ov;
#pragma unroll
      for (int i = 0; i < E / 2; ++i) ov[i] = pack2<T>(alo[2 * i] * inv, alo[2 * i + 1] * inv);
      *(vec_t*)(outp) = ov;
#pragma unroll
      for (int i = 0; i < E / 2; ++i) ov[i] = pack2<T>(ahi[2 * i] * inv, ahi[2 * i + 1] * inv);
      *(vec_t*)(outp + D) = ov;
    }
    return;
  }
  // merge with the local chunk: out_loc (normalised), L_loc, M_loc (natural-log units)
  const int64_t srow = (int64_t)bh * p.stat_stride + t;
  const float Ml = p.M_loc[srow] * kLog2e, Ll = p.L_loc[srow];
  const float Mt = fmaxf(Mrun, Ml);
  const float wr = fast_exp2(Mrun - Mt), wl = fast_exp2(Ml - Mt) * Ll;
  const float inv = 1.0f / (lrun * wr + wl);
  if (g == 0) {
    const char* olp = (const char*)p.o_loc + 2 * (b * p.ols_b + hh * p.ols_h + (int64_t)t * p.ols_r) + PB * j;
    char* outp = (char*)p.out + 2 * (b * p.outs_b + hh * p.outs_h + (int64_t)t * p.outs_r) + PB * j;
    float ol[E], o[E];
    vec_t ov;
    unpack8(*(const vec_t*)(olp), ol);
#pragma unroll
    for (int i = 0; i < E; ++i) o[i] = (alo[i] * wr + ol[i] * wl) * inv;
#pragma unroll
    for (int i = 0; i < E / 2; ++i) ov[i] = pack2<T>(o[2 * i], o[2 * i + 1]);
    *(vec_t*)(outp) = ov;
    unpack8(*(const vec_t*)(olp + D), ol);
#pragma unroll
    for (int i = 0; i < E; ++i) o[i] = (ahi[i] * wr + ol[i] * wl) * inv;
#pragma unroll
    for (int i = 0; i < E / 2; ++i) ov[i] = pack2<T>(o[2 * i], o[2 * i + 1]);
    *(vec_t*)(outp + D) = ov;
  }
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
template <class T, int D>
static int launch_topk_t(const RetrParams& p, bool reuse_landmark_keys, hipStream_t stream) {
  constexpr int RPW = 256 / (D / 8);
  const int64_t lkrows = (int64_t)p.B * p.H * p.num_mems;
  int rc;
  if (!reuse_landmark_keys) {
    hipLaunchKernelGGL((lmk_landmark_keys_kernel<T, D>), dim3((unsigned)((lkrows + RPW - 1) / RPW)), dim3(256), 0, stream, p);
    if ((rc = (int)hipGetLastError())) return rc;
  }
  const int64_t rows = (int64_t)p.B * p.H * p.T;
  const int n_slices = topk_slices(p);
  if (n_slices > 0) {                                               // a handful of rows: every score exact, slices over the chip
    hipLaunchKernelGGL((lmk_topk_slice_kernel<T, D>), dim3((unsigned)(rows * n_slices)), dim3(64 * kSliceWaves), 0, stream, p, n_slices);
    if ((rc = (int)hipGetLastError())) return rc;
    hipLaunchKernelGGL(lmk_topk_slice_merge_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, p, n_slices);
    return (int)hipGetLastError();
  }
  constexpr int lds_max = (kFusedRows * (kFusedMaxMems + 8) + kFusedRows * D) * 4 + kFusedRows * kFusedList * 2 + kFusedRows * (2 * D + 16);
  static_assert(lds_max <= 160 * 1024, "the score tile, the query rows and the lists fill the LDS of a compute unit");
  constexpr int lds = lds_max;                                    // one workgroup of 16 waves per compute unit whatever it takes
  const int n_rt = (p.T + kFusedRows - 1) / kFusedRows;
  const dim3 grid(p.B * p.H * n_rt), block(64 * kFusedWaves);
  if (p.num_mems <= kFusedMaxMems) {
    auto kern = lmk_topk_fused_kernel<T, D, false>;
    static std::atomic<uint64_t> lds_ok{0};
    if ((rc = allow_dynamic_lds(kern, lds_max, lds_ok))) return rc;
    hipLaunchKernelGGL(kern, grid, block, lds, stream, p);
  } else {
    auto kern = lmk_topk_fused_kernel<T, D, true>;
    static std::atomic<uint64_t> lds_ok{0};
    if ((rc = allow_dynamic_lds(kern, lds_max, lds_ok))) return rc;
    hipLaunchKernelGGL(kern, grid, block, lds, stream, p);
  }
  return (int)hipGetLastError();
}

template <class T, int D>
static int launch_topk_shared_t(const RetrParams& p, hipStream_t stream) {
  constexpr int RPW = 256 / (D / 8);
  const int64_t lkrows = (int64_t)p.B * p.H * p.num_mems;
  int rc;
  hipLaunchKernelGGL((lmk_landmark_keys_kernel<T, D>), dim3((unsigned)((lkrows + RPW - 1) / RPW)), dim3(256), 0, stream, p);
  if ((rc = (int)hipGetLastError())) return rc;
  const int64_t sel_rows = p.agg_over_heads ? (int64_t)p.B * p.T : (int64_t)p.B * p.H;   // vectors to pick from
  const int64_t score_waves = (int64_t)p.B * p.H * ((p.T + kScoreRows - 1) / kScoreRows) * ((p.num_mems + kScoreKeys - 1) / kScoreKeys);
  hipLaunchKernelGGL((lmk_block_score_kernel<T, D>), dim3((unsigned)((score_waves + 3) / 4)), dim3(256), 0, stream, p);
  if ((rc = (int)hipGetLastError())) return rc;
  const int64_t rows = (int64_t)p.B * p.H * p.T;
  const int is_bf16 = std::is_same<T, bf16_t>::value ? 1 : 0;
  if (p.num_mems <= 64 * 32) {
    // rows per wave: as many as leave the chip a few thousand waves, at most 8
    const int group = p.agg_over_heads ? p.H : p.T;
    const int rpw = (int)std::max<int64_t>(1, std::min<int64_t>(std::min(8, group), rows / 4096));
    const int64_t waves = (int64_t)((group + rpw - 1) / rpw) * sel_rows;
    const dim3 grid((unsigned)((waves + 3) / 4));
    if (p.num_mems <= 64) hipLaunchKernelGGL(lmk_block_prob_kernel<1>, grid, dim3(256), 0, stream, p, is_bf16, rpw);
    else if (p.num_mems <= 64 * 4) hipLaunchKernelGGL(lmk_block_prob_kernel<4>, grid, dim3(256), 0, stream, p, is_bf16, rpw);
    else if (p.num_mems <= 64 * 16) hipLaunchKernelGGL(lmk_block_prob_kernel<16>, grid, dim3(256), 0, stream, p, is_bf16, rpw);
    else hipLaunchKernelGGL(lmk_block_prob_kernel<32>, grid, dim3(256), 0, stream, p, is_bf16, rpw);
  } else {
    hipLaunchKernelGGL(lmk_block_prob_long_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, p, is_bf16);
  }
  if ((rc = (int)hipGetLastError())) return rc;
  hipLaunchKernelGGL(lmk_block_select_kernel, dim3((unsigned)sel_rows), dim3(256), 0, stream, p);
  return (int)hipGetLastError();
}

int launch_retrieve_topk_shared(const RetrParams& p, int D, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_topk_shared_t<bf16_t, 128>(p, stream);
    if (D == 64) return launch_topk_shared_t<bf16_t, 64>(p, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_topk_shared_t<f16_t, 128>(p, stream);
    if (D == 64) return launch_topk_shared_t<f16_t, 64>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

template <class T, int D>
static int launch_lk_t(const RetrParams& p, hipStream_t stream) {
  constexpr int RPW = 256 / (D / 8);
  const int64_t lkrows = (int64_t)p.B * p.H * p.num_mems;
  hipLaunchKernelGGL((lmk_landmark_keys_kernel<T, D>), dim3((unsigned)((lkrows + RPW - 1) / RPW)), dim3(256), 0, stream, p);
  return (int)hipGetLastError();
}

// The slice step of the selection alone (topk_slices(p) > 0): a row's candidates stay in p.approx / p.exact for a
// gather step that merges them (RetrParams::merge_slices).
template <class T, int D>
static int launch_slices_t(const RetrParams& p, hipStream_t stream) {
  const int n_slices = topk_slices(p);
  if (n_slices <= 0) return LMK_ERR_UNSUPPORTED;
  const int64_t rows = (int64_t)p.B * p.H * p.T;
  hipLaunchKernelGGL((lmk_topk_slice_kernel<T, D>), dim3((unsigned)(rows * n_slices)), dim3(64 * kSliceWaves), 0, stream, p, n_slices);
  return (int)hipGetLastError();
}

int launch_topk_slices(const RetrParams& p, int D, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_slices_t<bf16_t, 128>(p, stream);
    if (D == 64) return launch_slices_t<bf16_t, 64>(p, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_slices_t<f16_t, 128>(p, stream);
    if (D == 64) return launch_slices_t<f16_t, 64>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

int launch_landmark_keys(const RetrParams& p, int D, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_lk_t<bf16_t, 128>(p, stream);
    if (D == 64) return launch_lk_t<bf16_t, 64>(p, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_lk_t<f16_t, 128>(p, stream);
    if (D == 64) return launch_lk_t<f16_t, 64>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

int launch_retrieve_topk(const RetrParams& p, int D, int dtype, bool reuse_landmark_keys, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_topk_t<bf16_t, 128>(p, reuse_landmark_keys, stream);
    if (D == 64) return launch_topk_t<bf16_t, 64>(p, reuse_landmark_keys, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_topk_t<f16_t, 128>(p, reuse_landmark_keys, stream);
    if (D == 64) return launch_topk_t<f16_t, 64>(p, reuse_landmark_keys, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

template <class T, int D, int BS, bool PADDED>
static int launch_gather_b(const RetrParams& p, hipStream_t stream) {
  const int64_t rows = (int64_t)p.B * p.H * p.T;
  if (p.local) {                          // with the row's local window: blocks as they are only
    if constexpr (!PADDED) {
      const bool split = rows <= 1024 && p.k > 1;
      const dim3 grid((unsigned)(split ? rows : (rows + 3) / 4));
      if (p.merge_slices > 0) {
        if (split) hipLaunchKernelGGL((lmk_gather_attend_kernel<T, D, BS, true, PADDED, true, true>), grid, dim3(BS <= 64 ? 320 : 256), 0, stream, p);
        else hipLaunchKernelGGL((lmk_gather_attend_kernel<T, D, BS, false, PADDED, true, true>), grid, dim3(256), 0, stream, p);
      } else {
        if (split) hipLaunchKernelGGL((lmk_gather_attend_kernel<T, D, BS, true, PADDED, false, true>), grid, dim3(BS <= 64 ? 320 : 256), 0, stream, p);
        else hipLaunchKernelGGL((lmk_gather_attend_kernel<T, D, BS, false, PADDED, false, true>), grid, dim3(256), 0, stream, p);
      }
      return (int)hipGetLastError();
    } else {
      return LMK_ERR_UNSUPPORTED;
    }
  }
  if (p.merge_slices > 0) {               // the selection stopped after its slice step: blocks of 32 as they are only
    if constexpr (BS == 32 && !PADDED) {
      if (rows <= 1024 && p.k > 1)
        hipLaunchKernelGGL((lmk_gather_attend_kernel<T, D, BS, true, PADDED, true>), dim3((unsigned)rows), dim3(256), 0, stream, p);
      else
        hipLaunchKernelGGL((lmk_gather_attend_kernel<T, D, BS, false, PADDED, true>), dim3((unsigned)((rows + 3) / 4)), dim3(256),
                           0, stream, p);
      return (int)hipGetLastError();
    } else {
      return LMK_ERR_UNSUPPORTED;
    }
  }
  if (rows <= 1024 && p.k > 1) {          // fewer rows than SIMDs: one workgroup per row, its waves share the blocks out
    hipLaunchKernelGGL((lmk_gather_attend_kernel<T, D, BS, true, PADDED>), dim3((unsigned)rows), dim3(256), 0, stream, p);
  } else {
    hipLaunchKernelGGL((lmk_gather_attend_kernel<T, D, BS, false, PADDED>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                       stream, p);
  }
  return (int)hipGetLastError();
}

// BS: slots a block is worked on in (32, 64, 128); p.block: tokens of a block in the cache (<= BS)
template <class T, int D>
static int launch_gather_t(const RetrParams& p, int BS, hipStream_t stream) {
  if (p.block > BS || p.block < 2) return LMK_ERR_UNSUPPORTED;
  if (p.block == BS) {
    if (BS == 32) return launch_gather_b<T, D, 32, false>(p, stream);
    if (BS == 64) return launch_gather_b<T, D, 64, false>(p, stream);
    if (BS == 128) return launch_gather_b<T, D, 128, false>(p, stream);
  } else {
    if (BS == 64) return launch_gather_b<T, D, 64, true>(p, stream);
    if (BS == 128) return launch_gather_b<T, D, 128, true>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

// ---------------------------------------------------------------------------
// local window: [cached tail | new chunk] when the cache ends in an incomplete block
// (llama_mem.py:321-342), optionally behind the k blocks one per-head selection picked
// (:386-388, :400-406).  One 16-byte chunk per thread:
//   k_win = [rot(selected keys, slot positions) ; rot(tail keys, positions full_len ..) ; k_loc]
//   v_win = [selected values ; tail values ; v_loc]
//   q_win = [zero rows for the tail ; q]   -- rows in front of the queries so that the fused forward
//           kernel, run with the selected blocks as history, yields the new tokens' attention in its
//           last T rows
// ---------------------------------------------------------------------------
template <class T, int D>
__global__ __launch_bounds__(256) void lmk_local_window_kernel(WindowParams p) {
  constexpr int LPR = D / 8;
  constexpr int RPW = 256 / LPR;
  const int tid = threadIdx.x, j = tid % LPR;
  const int W = p.n_sel + p.inc + p.T;
  const int64_t row = (int64_t)blockIdx.x * RPW + tid / LPR;      // (bh, r)
  if (row >= (int64_t)p.B * p.H * W) return;
  const int bh = (int)(row / W), r = (int)(row % W);
  const int b = bh / p.H, hh = bh % p.H;
  u32x4_t qo = {0, 0, 0, 0}, ko, vo;
  if (r < p.n_sel + p.inc) {
    int64_t src_row, pos;
    if (r < p.n_sel) {
      const int slot = r / p.block, tok = r % p.block;
      int64_t blk = p.idx[(int64_t)bh * p.k + slot];
      blk = blk < 0 ? 0 : (blk >= p.num_mems ? p.num_mems - 1 : blk);   // never read outside the cache
      src_row = blk * p.block + tok;
      pos = (int64_t)r + (blk >= p.num_mems - p.k ? p.block : 0) + p.prefix_len;   // llama_mem.py:386-388
    } else {
      src_row = p.full_len + (r - p.n_sel);
      pos = p.tail_pos + (r - p.n_sel);
    }
    const char* src = (const char*)p.kcache + 2 * (b * p.kcs_b + hh * p.kcs_h + src_row * p.kcs_r);
    const u32x4_t x = *(const u32x4_t*)(src + 16 * j);
    const u32x4_t other = *(const u32x4_t*)(src + 16 * (j ^ (LPR / 2)));
    const u32x4_t c = *(const u32x4_t*)((const char*)p.cos + 2 * (pos * p.cs_r) + 16 * j);
    const u32x4_t s = *(const u32x4_t*)((const char*)p.sin + 2 * (pos * p.cs_r) + 16 * j);
    float o[8];
    rotate_chunk<T>(x, other, c, s, j >= LPR / 2, o);
    ko = u32x4_t{pack2<T>(o[0], o[1]), pack2<T>(o[2], o[3]), pack2<T>(o[4], o[5]), pack2<T>(o[6], o[7])};
    vo = *(const u32x4_t*)((const char*)p.vcache + 2 * (b * p.vcs_b + hh * p.vcs_h + src_row * p.vcs_r) + 16 * j);
  } else {
    const int t = r - p.n_sel - p.inc;
    qo = *(const u32x4_t*)((const char*)p.q + 2 * (b * p.qs_b + hh * p.qs_h + t * p.qs_r) + 16 * j);
    ko = *(const u32x4_t*)((const char*)p.k_loc + 2 * (b * p.kls_b + hh * p.kls_h + t * p.kls_r) + 16 * j);
    vo = *(const u32x4_t*)((const char*)p.v_loc + 2 * (b * p.vls_b + hh * p.vls_h + t * p.vls_r) + 16 * j);
  }
  if (r >= p.n_sel && p.q_win != nullptr)
    *(u32x4_t*)((char*)p.q_win + 2 * (b * p.qws_b + hh * p.qws_h + (int64_t)(r - p.n_sel) * p.qws_r) + 16 * j) = qo;
  *(u32x4_t*)((char*)p.k_win + 2 * (b * p.kws_b + hh * p.kws_h + (int64_t)r * p.kws_r) + 16 * j) = ko;
  *(u32x4_t*)((char*)p.v_win + 2 * (b * p.vws_b + hh * p.vws_h + (int64_t)r * p.vws_r) + 16 * j) = vo;
}

template <class T, int D>
static int launch_window_t(const WindowParams& p, hipStream_t stream) {
  constexpr int RPW = 256 / (D / 8);
  const int64_t rows = (int64_t)p.B * p.H * (p.n_sel + p.inc + p.T);
  hipLaunchKernelGGL((lmk_local_window_kernel<T, D>), dim3((unsigned)((rows + RPW - 1) / RPW)), dim3(256), 0, stream, p);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// rotary embedding of a whole (B, H, L, D) tensor at per-(batch, token) positions
// (apply_rotary_pos_emb, llama_mem.py:134-149): x*cos + rotate_half(x)*sin with the model dtype's
// rounding after each of the three elementwise operations.  One 16-byte chunk per thread; a row's
// chunks sit in one wave and every lane loads before any lane stores, so out may be x itself.
// PAIR: a second tensor of the same shape (the layer's q and k, :298) is rotated by the same thread with the
// same table rows, in the same launch.
// ---------------------------------------------------------------------------
template <class T, int D, bool PAIR>
__global__ __launch_bounds__(256) void lmk_rotary_kernel(RotaryParams p) {
  constexpr int LPR = D / 8;
  constexpr int RPW = 256 / LPR;
  const int tid = threadIdx.x, j = tid % LPR;
  const int64_t row = (int64_t)blockIdx.x * RPW + tid / LPR;      // (b, h, l)
  if (row >= (int64_t)p.B * p.H * p.L) return;
  const int l = (int)(row % p.L);
  const int bh = (int)(row / p.L);
  const int b = bh / p.H, hh = bh % p.H;
  int64_t pos = p.pos[(int64_t)b * p.pos_stride_b + l];
  pos = pos < 0 ? 0 : (pos >= p.n_pos ? p.n_pos - 1 : pos);      // never read outside the tables
  const char* src = (const char*)p.x + 2 * (b * p.xs_b + hh * p.xs_h + (int64_t)l * p.xs_r);
  const u32x4_t x = *(const u32x4_t*)(src + 16 * j);
  const u32x4_t other = *(const u32x4_t*)(src + 16 * (j ^ (LPR / 2)));
  u32x4_t x2 = {0, 0, 0, 0}, other2 = {0, 0, 0, 0};
  if (PAIR) {                                                     // the second tensor's row at the same (b, h, l)
    const char* src2 = (const char*)p.x2 + 2 * (b * p.x2s_b + hh * p.x2s_h + (int64_t)l * p.x2s_r);
    x2 = *(const u32x4_t*)(src2 + 16 * j);
    other2 = *(const u32x4_t*)(src2 + 16 * (j ^ (LPR / 2)));
  }
  const u32x4_t c = *(const u32x4_t*)((const char*)p.cos + 2 * (pos * p.cs_r) + 16 * j);
  const u32x4_t s = *(const u32x4_t*)((const char*)p.sin + 2 * (pos * p.cs_r) + 16 * j);
  float o[8];
  rotate_chunk<T>(x, other, c, s, j >= LPR / 2, o);
  const u32x4_t r = {pack2<T>(o[0], o[1]), pack2<T>(o[2], o[3]), pack2<T>(o[4], o[5]), pack2<T>(o[6], o[7])};
  *(u32x4_t*)((char*)p.out + 2 * (b * p.os_b + hh * p.os_h + (int64_t)l * p.os_r) + 16 * j) = r;
  if (PAIR) {
    rotate_chunk<T>(x2, other2, c, s, j >= LPR / 2, o);
    const u32x4_t r2 = {pack2<T>(o[0], o[1]), pack2<T>(o[2], o[3]), pack2<T>(o[4], o[5]), pack2<T>(o[6], o[7])};
    *(u32x4_t*)((char*)p.out2 + 2 * (b * p.o2s_b + hh * p.o2s_h + (int64_t)l * p.o2s_r) + 16 * j) = r2;
  }
}

template <class T, int D>
static int launch_rotary_t(const RotaryParams& p, hipStream_t stream) {
  constexpr int RPW = 256 / (D / 8);
  const int64_t rows = (int64_t)p.B * p.H * p.L;
  const dim3 grid((unsigned)((rows + RPW - 1) / RPW));
  if (p.x2 != nullptr) hipLaunchKernelGGL((lmk_rotary_kernel<T, D, true>), grid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((lmk_rotary_kernel<T, D, false>), grid, dim3(256), 0, stream, p);
  return (int)hipGetLastError();
}

int launch_rotary(const RotaryParams& p, int D, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_rotary_t<bf16_t, 128>(p, stream);
    if (D == 64) return launch_rotary_t<bf16_t, 64>(p, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_rotary_t<f16_t, 128>(p, stream);
    if (D == 64) return launch_rotary_t<f16_t, 64>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

int launch_local_window(const WindowParams& p, int D, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_window_t<bf16_t, 128>(p, stream);
    if (D == 64) return launch_window_t<bf16_t, 64>(p, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_window_t<f16_t, 128>(p, stream);
    if (D == 64) return launch_window_t<f16_t, 64>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

int launch_gather_attend(const RetrParams& p, int D, int BS, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_gather_t<bf16_t, 128>(p, BS, stream);
    if (D == 64) return launch_gather_t<bf16_t, 64>(p, BS, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_gather_t<f16_t, 128>(p, BS, stream);
    if (D == 64) return launch_gather_t<f16_t, 64>(p, BS, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

}  // namespace lmk
