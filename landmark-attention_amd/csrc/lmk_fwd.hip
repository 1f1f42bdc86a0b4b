// Forward kernel of fused landmark attention for gfx950.
//
// Replaces `_fwd_kernel` of the reference (llama/ltriton/flash_landmark_attention.py:6-122).
// This file: landmark blocks of 64 and 128 keys (block 32 has its own kernel in lmk_fwd32.hip).
// One workgroup = 8 waves = 256 consecutive query rows; every wave owns 32 queries and
// keeps S^T = K Q^T tiles in the MFMA C layout (lane = query, registers = keys), so the
// landmark grouped softmax never leaves a lane pair:
//   first pass:       the maximum R of the scores of the earlier blocks' landmarks (1/BS of the score work)
//   earlier block b:  local softmax over its BS-1 normal keys, gate = exp(landmark score - R),
//                     acc += (gate * P_local) V -- no running maximum, no rescaling
//   own block:        plain causal online softmax joined to the same (M, l), M starting at R
// K and V stream through LDS 128 keys per stage, double buffered, by direct global->LDS
// loads (no staging registers: two waves share a SIMD, so a wave has 256 registers);
// V is kept row-major and transposed on the way out of LDS by ds_read_b64_tr_b16.
#include <cstdlib>
#include <type_traits>

#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

template <class T, int D, int BS>
struct FwdCfg {
  static constexpr int NT = BS / 32;                    // 32-key tiles per landmark block
  static constexpr int NW = 8;
  static constexpr int ROWB = 2 * D;
  static constexpr int CH = D / 8;                      // 16-byte chunks per row
  static constexpr int NB = (BS >= 128) ? 1 : 128 / BS;  // landmark blocks per stage
  static constexpr int SK = NB * BS;                    // keys per stage
  static constexpr int TILE_BYTES = SK * ROWB;          // K (or V) of one stage
  static constexpr int STAGE_BYTES = 2 * TILE_BYTES;    // K, then V
  static constexpr int KS = D / 16;                     // MFMA k-steps over the head dim
  static constexpr int DC = D / 32;                     // 32-wide output chunks of the head dim
  static constexpr int LM_BASE = 2 * STAGE_BYTES;       // behind the two stages: 128 landmark keys for the first pass
  static constexpr int LDS_BYTES = LM_BASE + 128 * ROWB;
  static_assert(128 * ROWB / NW >= 2048, "a wave's share of that area also takes its output tile, 32 columns at a time");
  static constexpr int RPD = 1024 / ROWB;               // rows covered by one 1 KB request
  static constexpr int NREQ = 2 * SK / RPD;             // requests per stage
  static constexpr int PER_WAVE = NREQ / NW;
  static_assert(NREQ % NW == 0, "every wave issues the same number of requests");
};

// One 1 KB direct global->LDS request of a wave: lane i's 16 bytes land at lds_off + 16*i.
// lds_off must be wave-uniform (it travels in M0).
__device__ __forceinline__ void fwd_dma16(const void* base_uniform, uint32_t voff, uint32_t lds_off) {
  const uint64_t b = (uint64_t)base_uniform;
  const uint64_t base = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(b >> 32)) << 32) |
                        (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory");
}

// SEG: token layout with blocks of unequal length, looked up in p.seg (a template parameter: decided at run time
// the lookup costs the other launches 7 %).
// GS: group dropout factors in p.group_scale (a template parameter as well: the load's wait for the memory counter
// would otherwise sit in every launch's loop, where it also waits for the next stage's requests).
// PLAIN: every block has BS tokens in BS slots and the tensors' rows are the kernel's rows (the common case: the
// token-layout and padding paths, decided at run time, cost it 5 % -- 24 registers and the scalar registers of
// their masks).
template <class T, int D, int BS, bool SEG = false, bool GS = false, bool PLAIN = false>
__global__ __launch_bounds__(512, 2) void lmk_fwd_kernel(FwdParams p) {
  static_assert(!PLAIN || (!SEG && !GS), "the plain variant has no table and no factors");
  using C = FwdCfg<T, D, BS>;
  const int* const seg_k = SEG ? p.seg : nullptr;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ql = lane & 31, h = lane >> 5;

  // ---- workgroup -> (batch*head, 256-row query tile); heavy tiles first, one head per XCD slot
  const int nq256 = (p.Lq + 255) >> 8;
  int bh, qt;
  {
    const int bid = blockIdx.x;
    const int BH = p.B * p.H;
    if ((BH & 7) == 0) {
      const int xcd = bid & 7, j = bid >> 3, ngrp = BH >> 3;
      qt = nq256 - 1 - j / ngrp;
      bh = (j % ngrp) * 8 + xcd;
    } else {
      qt = nq256 - 1 - bid / BH;
      bh = bid % BH;
    }
  }
  const int b = bh / p.H, hh = bh % p.H;
  const char* qp = (const char*)p.q + 2 * (b * p.qs_b + hh * p.qs_h);
  const char* kp = (const char*)p.k + 2 * (b * p.ks_b + hh * p.ks_h);
  const char* vp = (const char*)p.v + 2 * (b * p.vs_b + hh * p.vs_h);
  char* op = (char*)p.o + 2 * (b * p.os_b + hh * p.os_h);

  const int q0 = qt * 256 + wave * 32;                  // first query row of this wave
  const int dt = p.n_prefix * C::NT + (q0 >> 5);        // its diagonal 32-key tile (absolute)
  const int cblk = dt / C::NT, tsub = dt % C::NT;       // its landmark block and sub-tile
  const bool active = q0 < p.Lq;
  const int qrow = q0 + ql;
  // token layout: the tensors' rows are tokens, the kernel's rows are slots
  const bool virt = !PLAIN && p.Lq_real > 0;            // uniform over the launch
  const int nfull_q = p.n_full_q, nfull_k = p.n_full_k;
  const int* seg_q = SEG ? p.seg + p.n_prefix : nullptr;   // the queries' first block
  const int qtok = !virt ? (qrow < p.Lq ? qrow : -1) : (qrow < p.Lq ? slot_to_token_row<BS>(qrow, p.n_real, nfull_q, seg_q) : -1);

  // ---- Q fragments (B operand): query qrow, head dims 16*ks + 8h .. +7
  u32x4_t qf[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    u32x4_t z = {0, 0, 0, 0};
    qf[ks] = z;
    if (qtok >= 0) qf[ks] = *(const u32x4_t*)(qp + 2 * ((int64_t)qtok * p.qs_r + 16 * ks + 8 * h));
  }
  if (p.rope_cos != nullptr && qtok >= 0) {                        // q without rotary: rotate the fragments at the row's position
    int64_t pos = p.rope_pos[(int64_t)b * p.rope_pos_stride_b + qtok];
    pos = pos < 0 ? 0 : (pos >= p.rope_n_pos ? p.rope_n_pos - 1 : pos);
    rotate_fragments<T, C::KS>(qf, (const char*)p.rope_cos + 2 * pos * p.rope_cs_r, (const char*)p.rope_sin + 2 * pos * p.rope_cs_r, h);
  }

  // ---- stages of SK keys (one or two landmark blocks), up to the own block of the workgroup's last
  // query tile.  K and V rows come by direct global->LDS loads, requested one stage ahead, each wave its
  // share: request r covers rows RPD*(r % (SK/RPD)) .. of K (r < SK/RPD) or of V.  The LDS swizzle is applied
  // on the source side: lane i lands at +16*i, i.e. row i/CH, chunk position i%CH, so it fetches the
  // chunk tile_off() stores there.  Rows past Lk (a partial last stage) are clamped to the last row;
  // they are keys no query can see.
  const int last_q0 = min(qt * 256 + 224, ((p.Lq - 1) >> 5) << 5);
  const int n_kstages = (p.Lk + C::SK - 1) / C::SK;
  const int n_stages = min(n_kstages, ((p.n_prefix * C::NT + (last_q0 >> 5)) / C::NT) / C::NB + 1);
  constexpr int n_k = C::SK / C::RPD;                   // requests that fetch K rows; the rest fetch V rows
  uint32_t src[C::PER_WAVE], src_last[C::PER_WAVE];     // per-lane byte offsets inside the (batch, head) slice
#pragma unroll
  for (int i = 0; i < C::PER_WAVE; ++i) {
    const int r = wave * C::PER_WAVE + i;
    const bool is_v = r >= n_k;
    const int row = C::RPD * (r % n_k) + lane / C::CH, cp = lane % C::CH;
    const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (C::CH - 1);
    const int64_t rs = is_v ? p.vs_r : p.ks_r;
    src[i] = (uint32_t)(2 * ((int64_t)row * rs + 8 * (cp ^ f)));
    const int row_last = min((n_kstages - 1) * C::SK + row, p.Lk - 1);
    src_last[i] = (uint32_t)(2 * ((int64_t)row_last * rs + 8 * (cp ^ f)));
  }
  const uint32_t step_k = (uint32_t)(2 * (int64_t)C::SK * p.ks_r), step_v = (uint32_t)(2 * (int64_t)C::SK * p.vs_r);
  int blk_req = 0;                                      // stage the next request fetches
  auto request = [&](int buf) __attribute__((always_inline)) {
    const bool last = blk_req == n_kstages - 1;         // wave-uniform
#pragma unroll
    for (int i = 0; i < C::PER_WAVE; ++i) {
      const int r = wave * C::PER_WAVE + i;
      const bool is_v = r >= n_k;                       // wave-uniform
      const int dst = buf * C::STAGE_BYTES + (is_v ? C::TILE_BYTES : 0) + C::RPD * (r % n_k) * C::ROWB;
      if (virt) {                                       // the slot's token row, worked out per request
        const int row = C::RPD * (r % n_k) + lane / C::CH, cp = lane % C::CH;
        const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (C::CH - 1);
        const int tok = slot_to_token_row_clamped<BS>(min(blk_req * C::SK + row, p.Lk - 1), p.n_real, nfull_k, seg_k);
        fwd_dma16(is_v ? vp : kp, (uint32_t)(2 * ((int64_t)tok * (is_v ? p.vs_r : p.ks_r) + 8 * (cp ^ f))), dst);
      } else {
        fwd_dma16(is_v ? vp : kp, last ? src_last[i] : src[i], dst);
        src[i] += is_v ? step_v : step_k;
      }
    }
    ++blk_req;
  };

  // ---- running state (log2 domain): M = max of the global bucket, l = its sum
  float Mrun = -INFINITY, lrun = 0.f;
  f32x16_t acc[C::DC];
#pragma unroll
  for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dc][r] = 0.f;

  const float c2 = p.scale_log2;
  // A block narrower than BS tokens is stored with its n_norm normal keys in front, its landmark in the
  // last slot and padding in between: slots n_norm .. BS-2 hold no key and no query may see them.
  // With blocks of unequal length n_norm is the block's at hand (uniform over the workgroup).
  const int n_norm_all = p.n_real - 1;
  const bool padded = !PLAIN && (n_norm_all < BS - 1 || SEG);   // uniform over the launch

  // LDS byte offsets of this lane's operand fragments inside a 32-row tile: the swizzle repeats every 16
  // rows, so a tile at row 32u is the same offsets plus 32u rows -- an immediate of the LDS instruction
  int koff[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) {
    koff[ks] = tile_off<D>(ql, 2 * ks + h);
    // the compiler must not know the value's range: it would turn "offset + constant" into an OR computed by a
    // vector instruction per read; as a plain sum the constant stays the read's immediate offset
    asm volatile("" : "+v"(koff[ks]));
  }
  int voff[C::DC][2];
  {
    const int i = lane & 15, g2 = (lane >> 4) & 1;
#pragma unroll
    for (int dc = 0; dc < C::DC; ++dc) {
      const int col = 32 * dc + 16 * g2 + 4 * (i & 3);
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
        voff[dc][hf] = tile_off<D>(4 * h + (i >> 2) + 8 * hf, col >> 3) + ((col >> 2) & 1) * 8;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) asm volatile("" : "+v"(voff[dc][hf]));   // as for koff
    }
  }
  auto qk_tile = [&](int tile_bytes) __attribute__((always_inline)) {                  // S^T of the 32 keys at LDS byte address tile_bytes
    f32x16_t s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) s = mfma32<T>(lds_ld128(tile_bytes + koff[ks]), qf[ks], s);
    return s;
  };
  auto pv_tile = [&](int tile_bytes, const float* w) __attribute__((always_inline)) {  // O^T += (V tile)^T W
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      u32x4_t wf = {pack2<T>(w[8 * j + 0], w[8 * j + 1]), pack2<T>(w[8 * j + 2], w[8 * j + 3]),
                    pack2<T>(w[8 * j + 4], w[8 * j + 5]), pack2<T>(w[8 * j + 6], w[8 * j + 7])};
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc) {
        const int base = tile_bytes + 16 * j * C::ROWB;
        const u32x2_t a0 = lds_ld_tr(base + voff[dc][0]), a1 = lds_ld_tr(base + voff[dc][1]);
        const u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
        acc[dc] = mfma32<T>(a, wf, acc[dc]);
      }
    }
  };
  auto rescale = [&](float alpha) __attribute__((always_inline)) {
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dc][r] *= alpha;
    }
  };

  // ---------------- earlier block at LDS byte addresses kb (K rows) / vb (V rows): local softmax gated by its landmark
  auto earlier_block = [&](const int kb, const int vb, const int blk) __attribute__((always_inline)) {
    int n_norm = n_norm_all;
    if constexpr (SEG) n_norm = block_normal_keys<BS>(blk, p.n_real, nfull_k, seg_k);
    float gscale = 1.f;                                 // group dropout: this block's factor for this query row
    if constexpr (GS)
      if (qtok >= 0) gscale = p.group_scale[(int64_t)bh * p.gs_bh + (int64_t)blk * p.gs_blk + qtok];
    // S^T of the block's tiles: the wave issues in order, so the instruction stream is the schedule -- every
    // operand is asked for two MFMAs ahead of its use and the order is pinned
    f32x16_t sc[C::NT];
    {
      constexpr int NX = C::NT * C::KS, PFX = 2;
      u32x4_t fk[NX];
#pragma unroll
      for (int n = 0; n < PFX; ++n) fk[n] = lds_ld128(kb + 32 * (n / C::KS) * C::ROWB + koff[n % C::KS]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int n = 0; n < NX; ++n) {
        if (n + PFX < NX) fk[n + PFX] = lds_ld128(kb + 32 * ((n + PFX) / C::KS) * C::ROWB + koff[(n + PFX) % C::KS]);
        const int u = n / C::KS, ks = n % C::KS;
        if (ks == 0) {
#pragma unroll
          for (int r = 0; r < 16; ++r) sc[u][r] = 0.f;
        }
        sc[u] = mfma32<T>(fk[n], qf[ks], sc[u]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // key of register r in tile u: 32u + 8*(r/4) + 4h + r%4; the landmark is (NT-1, r=15, h=1)
    if (padded) {                                       // padding slots leave the local softmax
#pragma unroll
      for (int u = 0; u < C::NT; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int kl = 32 * u + 8 * (r >> 2) + 4 * h + (r & 3);
          if (kl >= n_norm && kl < BS - 1) sc[u][r] = -INFINITY;
        }
    }
    const float s_last = sc[C::NT - 1][15];
    float mx = (h == 0) ? s_last : -INFINITY;
#pragma unroll
    for (int u = 0; u < C::NT; ++u)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (!(u == C::NT - 1 && r == 15)) mx = fmaxf(mx, sc[u][r]);
    mx = pair_max(mx);
    const float t_lm = pair_hi(s_last) * c2;            // landmark score, log2 domain
    const float mloc = mx * c2;
    float den = 0.f;
#pragma unroll
    for (int u = 0; u < C::NT; ++u)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float e = fast_exp2(__builtin_fmaf(sc[u][r], c2, -mloc));
        if (u == C::NT - 1 && r == 15) e = (h == 0) ? e : 0.f;
        sc[u][r] = e;
        den += e;
      }
    den = pair_sum(den);
    const float gate = fast_exp2(t_lm - Mrun);          // Mrun is the first pass's maximum here: no greater landmark comes
    lrun += gate;
    const float f = gate * fast_rcp(den) * gscale;
    // O^T += V^T W, W = f * e in slices of 16 keys: a slice is scaled and packed under the MFMAs of the one before
    {
      constexpr int NZ = C::NT * 2 * C::DC, PFZ = 2;
      auto zload = [&](int n) __attribute__((always_inline)) {
        const int sl = n / C::DC, dc = n % C::DC;         // slice = (tile, half)
        const int base = vb + 16 * sl * C::ROWB;
        const u32x2_t a0 = lds_ld_tr(base + voff[dc][0]), a1 = lds_ld_tr(base + voff[dc][1]);
        const u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
        return a;
      };
      auto wslice = [&](int sl) __attribute__((always_inline)) {
        const int u = sl >> 1, j = sl & 1;
        u32x4_t wf;
#pragma unroll
        for (int i = 0; i < 4; ++i) wf[i] = pack2<T>(sc[u][8 * j + 2 * i] * f, sc[u][8 * j + 2 * i + 1] * f);
        return wf;
      };
      u32x4_t zf[NZ], wf[2];
#pragma unroll
      for (int n = 0; n < PFZ; ++n) zf[n] = zload(n);
      wf[0] = wslice(0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int n = 0; n < NZ; ++n) {
        if (n + PFZ < NZ) zf[n + PFZ] = zload(n + PFZ);
        const int sl = n / C::DC, dc = n % C::DC;
        acc[dc] = mfma32<T>(zf[n], wf[sl & 1], acc[dc]);
        if (dc == 0 && sl + 1 < 2 * C::NT) wf[(sl + 1) & 1] = wslice(sl + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // Stages in front of the workgroup's first query block hold earlier blocks only, for every wave: they run two
  // at a time without a branch, the LDS addresses of both buffers as immediates of the instructions.
  const int first_cblk = (p.n_prefix * C::NT + qt * 8) / C::NT;   // wave 0's own block: the least of the workgroup's
  const int s_uniform = min(first_cblk / C::NB, n_stages - 1);
  auto uniform_stage = [&](auto buf_c, int s) __attribute__((always_inline)) {
    constexpr int buf = decltype(buf_c)::value;
    __builtin_amdgcn_s_waitcnt(0x0f70);                 // vmcnt(0): this wave's share of stage s has landed
    __syncthreads();                                    // ... and everyone's; stage s-1 has been consumed
    request(buf ^ 1);
    if (active) {
#pragma unroll
      for (int jb = 0; jb < C::NB; ++jb)
        earlier_block(buf * C::STAGE_BYTES + jb * BS * C::ROWB, buf * C::STAGE_BYTES + jb * BS * C::ROWB + C::TILE_BYTES,
                      s * C::NB + jb);
    }
  };

  // ---- first pass: the maximum over the landmark scores of the wave's earlier blocks, 128 landmarks at a time
  // through an LDS area of their own.  With it as the reference of the global bucket the earlier blocks need no
  // running maximum and never rescale the accumulator (the reference's loop carries both, :64-76; same sums).
  // The scores are the main pass's to the bit (same rows, same products), so no gate exceeds one.
  {
    constexpr int LM_PER_WAVE = n_k / C::NW;
    const int wg_cblk = (p.n_prefix * C::NT + (last_q0 >> 5)) / C::NT;   // own block of the last wave with queries
    float mx = -INFINITY;
    for (int base = 0; base < wg_cblk; base += 128) {
#pragma unroll
      for (int i = 0; i < LM_PER_WAVE; ++i) {
        const int r = wave * LM_PER_WAVE + i;
        const int row = C::RPD * r + lane / C::CH, cp = lane % C::CH;
        const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (C::CH - 1);
        const int slot = min(base + row, wg_cblk - 1) * BS + BS - 1;     // an earlier block: complete, inside the table
        const int tok = virt ? slot_to_token_row_clamped<BS>(slot, p.n_real, nfull_k, seg_k) : slot;
        fwd_dma16(kp, (uint32_t)(2 * ((int64_t)tok * p.ks_r + 8 * (cp ^ f))), C::LM_BASE + C::RPD * r * C::ROWB);
      }
      if (base == 0) {
        request(0);                                     // stage 0 travels behind the landmarks
        __builtin_amdgcn_s_waitcnt(0x0f70 | (C::PER_WAVE & 15) | ((C::PER_WAVE >> 4) << 14));   // all but the stage's requests
      } else {
        __builtin_amdgcn_s_waitcnt(0x0f70);
      }
      __syncthreads();
      if (active) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (base + 32 * u < cblk) {
            const f32x16_t sl = qk_tile(C::LM_BASE + 32 * u * C::ROWB);
#pragma unroll
            for (int r = 0; r < 16; ++r)
              mx = (base + 32 * u + 8 * (r >> 2) + 4 * h + (r & 3) < cblk) ? fmaxf(mx, sl[r]) : mx;
          }
        }
      }
      if (base + 128 < wg_cblk) __syncthreads();        // the area is written again
    }
    if (wg_cblk == 0) request(0);
    Mrun = pair_max(mx) * c2;
  }

  int s = 0;
  for (; s + 2 <= s_uniform; s += 2) {
    uniform_stage(std::integral_constant<int, 0>{}, s);
    uniform_stage(std::integral_constant<int, 1>{}, s + 1);
  }
  for (; s < n_stages; ++s) {
    const int buf = s & 1;
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    if (s + 1 < n_stages) request(buf ^ 1);
    if (!active) continue;
#pragma unroll
    for (int jb = 0; jb < C::NB; ++jb) {
      const int blk = s * C::NB + jb;                     // absolute landmark block
      // LDS byte addresses of the block's K and V rows (the dynamic array starts at 0)
      const int kb = buf * C::STAGE_BYTES + jb * BS * C::ROWB, vb = kb + C::TILE_BYTES;
      // (a stage may reach past the wave's own block, and past the table: those blocks are not looked at)
      if (blk < cblk) {
        earlier_block(kb, vb, blk);
      } else if (blk == cblk) {
        int n_norm = n_norm_all;
        if constexpr (SEG) n_norm = block_normal_keys<BS>(blk, p.n_real, nfull_k, seg_k);
        // ---------------- own block: causal tiles 0..tsub join the global bucket
        const int lim = ql - ((tsub == C::NT - 1 && ql == 31) ? 1 : 0);  // landmark query looks one left
#pragma unroll
        for (int u = 0; u < C::NT; ++u) {
          if (u <= tsub) {
            f32x16_t sc = qk_tile(kb + 32 * u * C::ROWB);
            float x[16];
            float mt = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int key = 8 * (r >> 2) + 4 * h + (r & 3);
              const int kl = 32 * u + key;
              const bool pad = padded && kl >= n_norm && kl < BS - 1;   // only the landmark query could reach one
              x[r] = ((u < tsub || key <= lim) && !pad) ? sc[r] * c2 : -INFINITY;
              mt = fmaxf(mt, x[r]);
            }
            mt = pair_max(mt);
            const float Mnew = fmaxf(Mrun, mt);
            const float alpha = fast_exp2(Mrun - Mnew);
            float sum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              x[r] = fast_exp2(x[r] - Mnew);
              sum += x[r];
            }
            sum = pair_sum(sum);
            lrun = lrun * alpha + sum;
            Mrun = Mnew;
            rescale(alpha);
            pv_tile(vb + 32 * u * C::ROWB, x);
          }
        }
      }
    }
  }

  // ---- epilogue: out = acc / l, statistics in natural-log units like the reference
  // the output leaves as row segments through the wave's share of the first pass's LDS area, which nothing has
  // touched since (a slot without a token, or past the last row, stores nothing)
  if (active)
    store_tile_rows<T, C::DC>(acc, 1.0f / lrun, C::LM_BASE + wave * (128 * C::ROWB / C::NW),
                              [&](int r) __attribute__((always_inline)) -> char* {
      const int qr = q0 + r;
      if (qr >= p.Lq) return nullptr;
      const int tok = virt ? slot_to_token_row<BS>(qr, p.n_real, nfull_q, seg_q) : qr;
      return tok < 0 ? nullptr : op + 2 * ((int64_t)tok * p.os_r);
    });
  if (active && qtok >= 0) {
    if (h == 0) {                                       // statistics follow the tensors' layout
      const int64_t si = (int64_t)bh * (virt ? p.Lq_real : p.Lq) + qtok;
      p.L[si] = lrun;
      p.M[si] = Mrun * kLn2;
    }
  }
}

template <class T, int D, int BS, bool SEG, bool GS, bool PLAIN = false>
static int launch_fwd_s(const FwdParams& p, hipStream_t stream) {
  using C = FwdCfg<T, D, BS>;
  auto kern = lmk_fwd_kernel<T, D, BS, SEG, GS, PLAIN>;
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok)) return rc;
  const int grid = ((p.Lq + 255) / 256) * p.B * p.H;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * C::NW), C::LDS_BYTES, stream, p);
  return (int)hipGetLastError();
}

template <class T, int D, int BS>
static int launch_fwd_t(const FwdParams& p, hipStream_t stream) {
  if (p.seg != nullptr) return p.group_scale != nullptr ? LMK_ERR_UNSUPPORTED : launch_fwd_s<T, D, BS, true, false>(p, stream);
  if (p.group_scale != nullptr) return launch_fwd_s<T, D, BS, false, true>(p, stream);
  if (p.Lq_real <= 0 && p.n_real == BS) return launch_fwd_s<T, D, BS, false, false, true>(p, stream);
  return launch_fwd_s<T, D, BS, false, false>(p, stream);
}

template <class T>
static int launch_fwd_d(const FwdParams& p, int D, int BS, hipStream_t stream) {
  if (D == 128) {                                          // block 32 has its own kernel (lmk_fwd32.hip)
    if (BS == 64) return launch_fwd_t<T, 128, 64>(p, stream);
    if (BS == 128) return launch_fwd_t<T, 128, 128>(p, stream);
  } else if (D == 64) {
    if (BS == 64) return launch_fwd_t<T, 64, 64>(p, stream);
    if (BS == 128) return launch_fwd_t<T, 64, 128>(p, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

int launch_fwd(const FwdParams& p, int D, int BS, int dtype, hipStream_t stream) {
  if (BS == 32) return launch_fwd32(p, D, dtype, stream);
  if (dtype == LMK_DTYPE_BF16) return launch_fwd_d<bf16_t>(p, D, BS, stream);
  if (dtype == LMK_DTYPE_F16) return launch_fwd_d<f16_t>(p, D, BS, stream);
  return LMK_ERR_UNSUPPORTED;
}

}  // namespace lmk
