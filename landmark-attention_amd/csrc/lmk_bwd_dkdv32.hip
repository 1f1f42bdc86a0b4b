// dK/dV kernel of the backward pass.  Written for a landmark block of 32 keys (one MFMA tile) and
// extended to blocks of 64 and 128 keys, which are 2 or 4 key tiles: what changes is which block a key
// tile belongs to (its terms, its landmark lane) and which query tiles share that block.
//
// Key-stationary.  A workgroup is 8 waves = 4 key tiles of 32 keys x 2 roles; the two waves of a
// key tile sit on the same SIMD (waves t and t+4) and split the work so that each holds one
// accumulator and both pipes of the SIMD have work from two instruction streams at once:
//     wave V (t):    S = Q K^T,  W = exp2(S c - x)  (the attention weights),  dV^T += dO^T W
//     wave K (t+4):  dP = dO V^T,  dS = W (dP - y) + z,                       dK^T += Q^T dS
// W goes from wave V to wave K through LDS as packed 16-bit values, lane for lane (both waves hold
// the same accumulator layout: lane = key, register r = query row 8*(r/4) + 4*(l/32) + r%4), and
// wave K runs one query tile behind wave V, so one barrier per query tile orders everything.
// Within a wave the products of the next tile are interleaved with the elementwise work of the
// current one (the wave issues in order, so the instruction stream is the schedule).
//
// Query tiles (32 rows of Q and of dO) and the terms the elementwise steps need (per row: mhat,
// delta; per (row, block): a, nD, dS at the landmark, left behind by the dQ kernel) stream through
// a ring of six LDS slots filled by direct global->LDS loads (global_load_lds_dwordx4): tile i+4 is
// requested while tile i is computed, no registers are tied up by data in flight, and vmcnt is
// counted by hand.  The LDS swizzle is applied on the source side: lane i of a request lands at
// +16*i, so it fetches the chunk that belongs there.
//     earlier block (query tile past the key tile):  x = a, y = nD, z = 0; at the block's landmark
//         key W = 0 (x = 1e30) and z = the dS stored by the dQ kernel
//     own block / not yet visible:  W = [key <= lim] exp2(s*c - mhat),  y = delta, z = 0
//
// A workgroup serves several 128-key tiles of one (batch, head) in a row when there are more tiles than CUs
// (at most four, in a zig-zag over the head's tiles so that every workgroup gets the same work).  The ring does
// not stop between them: behind a tile's last query tile the requests go on with the first query tiles of the
// workgroup's next key tiles, so only the stationary operand and the accumulator change hands at the boundary.
#include <type_traits>

#include "lmk_common.hpp"
#include "lmk_launch.hpp"

namespace lmk {

template <class T, int D, int BS = 32>
struct Dkv32Cfg {
  static constexpr int TPB = BS / 32;                      // key (and query) tiles per landmark block
  static constexpr int NKT = 4;                            // key tiles per workgroup
  static constexpr int NW = 2 * NKT;
  static constexpr int NTHR = 64 * NW;
  static constexpr int CH = D / 8;
  static constexpr int KS = D / 16;
  static constexpr int DC = D / 32;
  static constexpr int ROWB = 2 * D;
  static constexpr int TILE_BYTES = 32 * ROWB;             // one query tile of Q (or of dO)
  static constexpr int STAT_BYTES = 1024 * NKT;            // per key tile: a, nD, dslm, mhat, delta (128 B each) + pad
  static constexpr int BUF_BYTES = 2 * TILE_BYTES + STAT_BYTES;   // Q, dO, terms
  static constexpr int NBUF = 6;                           // ring slots: tiles i-1, i, i+1 in use, i+2 .. i+4 in flight
  static constexpr int RPD = 1024 / ROWB;                  // tile rows covered by one 1 KB request
  static constexpr int NDMA = 32 / RPD / NKT;              // requests per wave and tile for one tensor
  static constexpr int PER_TILE_V = 2 * NDMA + 1;          // the V-role waves fetch everything: Q rows, the key tile's terms,
                                                           // dO rows (the K role is the longer chain of every iteration)
  static constexpr int XCH_OFF = NBUF * BUF_BYTES;         // W hand-over: [parity 2][key tile][piece 2][lane][16 B]
  static constexpr int XCH_TILE = 2048;
  static constexpr int CONST_OFF = XCH_OFF + 2 * NKT * XCH_TILE;   // 32 x 1e30f, then 32 x 0.0f
  static constexpr int LDS_BYTES = CONST_OFF + 256;
};

// One 1 KB direct global->LDS request of a wave: lane i's 16 bytes land at lds_off + 16*i.
// lds_off must be wave-uniform (it travels in M0).
__device__ __forceinline__ void dma16_s(const void* base_uniform, uint32_t voff, uint32_t lds_off) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base_uniform), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory");
}
__device__ __forceinline__ void dma16_v(const void* ptr, uint32_t lds_off) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :: "v"(ptr), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {             // s_waitcnt vmcnt(N) only (gfx9 encoding)
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

#define LMK_INL __attribute__((always_inline))

// VIRT (blocks of 64 and 128 slots only): q, k, v, dout, dk, dv are in token layout (BwdParams::Lq_real > 0) while
// p.Lq, p.Lk and the workspace count slots.  Slots without a token need no mask here: the dQ kernel left a = 1e30
// and mhat = 1e30 for such query rows, so their W and dS are exact zeros whatever rows are read for them, and the
// accumulator rows of such keys are not stored.
// SEG (with VIRT): blocks of unequal length, rows looked up in p.seg (a template parameter: the lookup in the
// request stream costs the other variants 5 us at B2 H8 L510 when it is decided at run time).
template <class T, int D, int BS, bool VIRT = false, bool SEG = false>
__global__ __launch_bounds__(512, 2) void lmk_bwd_dkdv32_kernel(BwdParams p) {
  using C = Dkv32Cfg<T, D, BS>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int tile = wave & (C::NKT - 1);                    // key tile inside the workgroup
  const bool role_k = wave >= C::NKT;                      // false: S, W, dV; true: dP, dS, dK
  const int ql = lane & 31, h = lane >> 5;

  // A workgroup serves one (batch, head) and several 128-key tiles of it, one after the other ("items"):
  // with G workgroups per head, workgroup g takes tiles g, 2G-1-g, 2G+g, 4G-1-g, .. (a zig-zag, so that
  // every workgroup gets the same amount of work; tile 0 sees every query tile, the last one the fewest).
  const int BH = p.B * p.H;
  const int G = (int)gridDim.x / BH;                       // workgroups per head
  const int n_c = (p.n_kvtiles + G - 1) / G;               // items per workgroup (some may fall past the last tile)
  int bh, g_;
  {
    const int bid = blockIdx.x;
    if ((BH & 7) == 0) {                                   // all workgroups of a head on one XCD
      const int xcd = bid & 7, j = bid >> 3, ngrp = BH >> 3;
      g_ = j / ngrp;
      bh = (j % ngrp) * 8 + xcd;
    } else {
      g_ = bid / BH;
      bh = bid % BH;
    }
  }
  auto item_kvt = [&](int c) LMK_INL { return (c & 1) ? (c + 1) * G - 1 - g_ : c * G + g_; };
  auto next_item = [&](int c) LMK_INL {                    // first item index >= c with a tile that exists, or n_c
    while (c < n_c && item_kvt(c) >= p.n_kvtiles) ++c;
    return c;
  };
  int kvt = item_kvt(0);                                   // item 0 always exists (g_ < G <= n_kvtiles)
  const int b_ = bh / p.H, hh = bh % p.H;
  const char* qp = (const char*)p.q + 2 * (b_ * p.qs_b + hh * p.qs_h);
  const char* gp = (const char*)p.dout + 2 * (b_ * p.dos_b + hh * p.dos_h);

  const int nkt = p.Lk >> 5;                               // key tiles (TPB per landmark block)
  const int PT = p.n_prefix * C::TPB;                      // history tiles in front of the queries
  const int nq = p.Lq >> 5;
  // the item being computed
  int kt, kt_end, j_first;
  bool active, lm_lane;
  auto set_item = [&](int c) LMK_INL {
    kvt = item_kvt(c);
    kt = kvt * C::NKT + tile;
    active = kt < nkt;
    lm_lane = (ql == 31) && (kt % C::TPB == C::TPB - 1);   // this lane's key is its block's landmark
    kt_end = (kt / C::TPB + 1) * C::TPB;                   // first tile behind this key tile's block
    j_first = max(0, kvt * C::NKT - PT);                   // first query tile any wave here can see
  };
  set_item(0);
  const float c2 = p.scale_log2;

  u32x4_t bf[C::KS];                                       // stationary operand, loaded after the first requests

  int koff[C::KS];
#pragma unroll
  for (int ks = 0; ks < C::KS; ++ks) koff[ks] = tile_off<D>(ql, 2 * ks + h);
  int voff[C::DC][2];
  {
    const int i = lane & 15, g2 = (lane >> 4) & 1;
#pragma unroll
    for (int dc = 0; dc < C::DC; ++dc) {
      const int col = 32 * dc + 16 * g2 + 4 * (i & 3);
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
        voff[dc][hf] = tile_off<D>(4 * h + (i >> 2) + 8 * hf, col >> 3) + ((col >> 2) & 1) * 8;
    }
  }

  // ---- loaders.  The V-role wave of pair t fetches rows RPD*(t*NDMA + d) .. of a query tile's Q and dO and the
  // terms of key tile t; the K-role waves fetch nothing.
  static_assert(C::NDMA <= 2, "two source offsets per tensor");
  // The requests run four to five query tiles ahead of the arithmetic and do not stop at the end of an item:
  // behind an item's last query tile they go on with the first tiles of the workgroup's next item, so the ring
  // is full when that item starts.  The stream's position is a handful of scalars: the tile it fetches next
  // (j_req), the item's offset into the per-block planes (pl_req), and the same two for the item after it,
  // which the arithmetic side fills in whenever it starts an item (every item but a workgroup's last has more
  // query tiles than the stream runs ahead, so the entry is there before the stream needs it).
  // per-lane source offsets (bytes) of this wave's requests 0 and 1 inside tile 0 of Q and of dO
  uint32_t q_vo0 = 0, q_vo1 = 0, g_vo0 = 0, g_vo1 = 0;
  int vrow0 = 0, vcf0 = 0, vcf1 = 0;                       // VIRT: this lane's row inside a tile and its two chunk offsets
  const int nfull_q = p.n_full_q, nfull_k = p.n_full_k;
  const int* seg_k = SEG ? p.seg : nullptr;             // blocks of unequal length (null: n_real tokens each)
  const int* seg_q = SEG ? p.seg + p.n_prefix : nullptr;   // the queries' first block
  if (!role_k) {
    const int chp = lane % C::CH;
    const int row0 = C::RPD * (tile * C::NDMA) + lane / C::CH, row1 = row0 + C::RPD;
    const int f0 = (((row0 & 3) << 2) | ((row0 >> 2) & 3)) & (C::CH - 1);
    const int f1 = (((row1 & 3) << 2) | ((row1 >> 2) & 3)) & (C::CH - 1);
    q_vo0 = (uint32_t)(2 * (row0 * p.qs_r + 8 * (chp ^ f0)));      // the chunk that belongs at LDS position chp
    g_vo0 = (uint32_t)(2 * (row0 * p.dos_r + 8 * (chp ^ f0)));
    if (C::NDMA > 1) {
      q_vo1 = (uint32_t)(2 * (row1 * p.qs_r + 8 * (chp ^ f1)));
      g_vo1 = (uint32_t)(2 * (row1 * p.dos_r + 8 * (chp ^ f1)));
    }
    vrow0 = row0;
    vcf0 = 16 * (chp ^ f0);
    vcf1 = 16 * (chp ^ f1);
  }
  // VIRT: byte offset of this lane's chunk of slot row 32 j + its row (+ RPD for the second request) of a tensor
  auto virt_off = [&](int j, int second, int64_t row_stride) LMK_INL {
    const int tok = slot_to_token_row_clamped<BS>(32 * j + vrow0 + (second ? C::RPD : 0), p.n_real, nfull_q, seg_q);
    return 2u * (uint32_t)tok * (uint32_t)row_stride + (uint32_t)(second ? vcf1 : vcf0);
  };
  const uint32_t q_step = (uint32_t)(2 * 32 * p.qs_r), g_step = (uint32_t)(2 * 32 * p.dos_r);
  // this lane's 16 bytes of a query tile's terms: lanes 0-7 a, 8-15 nD, 16-23 dS at the landmark (planes, one row
  // of Lq per block), 24-31 mhat, 32-63 delta (one row per head)
  const float* st_lane;                                    // its array at the head's first row, tile 0
  {
    const int arr = min(lane / 8, 4), part = lane % 8;
    const int64_t plane0 = (int64_t)bh * p.n_blocks * p.Lq, head_row = (int64_t)bh * p.Lq;
    st_lane = (arr == 0) ? p.stat_a + plane0 : (arr == 1) ? p.stat_n + plane0 : (arr == 2) ? p.stat_l + plane0
              : (arr == 3) ? p.mhat + head_row : p.delta + head_row;
    st_lane += 4 * part;
  }
  auto item_first = [&](int c) LMK_INL { return max(0, item_kvt(c) * C::NKT - PT); };
  auto item_plane = [&](int c) LMK_INL {                   // element offset of this wave's key tile's block inside the planes
    return (int64_t)min((item_kvt(c) * C::NKT + tile) / C::TPB, p.n_blocks - 1) * p.Lq;
  };
  int j_req = item_first(0), jf_nx = 0;
  int64_t pl_req = item_plane(0), pl_nx = 0;
  bool has_nx = false;
  auto announce_next = [&](int c) LMK_INL {                // the arithmetic side starts item c: tell the stream what follows it
    const int c2 = next_item(c + 1);
    has_nx = c2 < n_c;
    if (has_nx) {
      jf_nx = item_first(c2);
      pl_nx = item_plane(c2);
    }
  };
  announce_next(0);
  // One piece of this wave's share of the stream's tile -> ring slot.  A tile's pieces go out one per MFMA
  // slot of the first product rather than together: all waves asking at once queue up in front of the
  // address unit.  Pieces 0 .. NDMA-1 fetch Q rows, piece NDMA the terms, pieces NDMA+1 .. 2 NDMA dO rows.
  const int dst_off = tile * C::NDMA * 1024;               // this wave's rows inside a tile of a slot
  auto request_piece = [&](int slot_bytes, auto Pc) LMK_INL {
    constexpr int P = decltype(Pc)::value;
    if constexpr (P == 0) {                                // a new tile: behind an item's last one, move to the next item
      const bool past = j_req >= nq, take = past && has_nx;    // (or re-read the last tile, which nobody uses)
      j_req = take ? jf_nx : (past ? nq - 1 : j_req);
      pl_req = take ? pl_nx : pl_req;
      has_nx = take ? false : has_nx;
    }
    if constexpr (P < C::NDMA) {
      if constexpr (VIRT) dma16_s(qp, virt_off(j_req, P, p.qs_r), slot_bytes + dst_off + P * 1024);
      else dma16_s(qp, ((P == 0) ? q_vo0 : q_vo1) + (uint32_t)j_req * q_step, slot_bytes + dst_off + P * 1024);
    } else if constexpr (P == C::NDMA) {
      const int64_t off = 32 * (int64_t)j_req + ((lane < 24) ? pl_req : 0);
      dma16_v(st_lane + off, slot_bytes + 2 * C::TILE_BYTES + tile * 1024);
    } else if constexpr (P <= 2 * C::NDMA) {
      constexpr int G = P - C::NDMA - 1;
      if constexpr (VIRT) dma16_s(gp, virt_off(j_req, G, p.dos_r), slot_bytes + C::TILE_BYTES + dst_off + G * 1024);
      else dma16_s(gp, ((G == 0) ? g_vo0 : g_vo1) + (uint32_t)j_req * g_step, slot_bytes + C::TILE_BYTES + dst_off + G * 1024);
      if (P == 2 * C::NDMA) ++j_req;
    }
  };
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  using P2 = std::integral_constant<int, 2>;
  using P3 = std::integral_constant<int, 3>;
  using P4 = std::integral_constant<int, 4>;
  static_assert(C::PER_TILE_V <= 5 && C::PER_TILE_V <= C::KS, "a tile's pieces are P0 .. P4, one per MFMA slot");
  auto request = [&](int slot_bytes) LMK_INL {             // the whole share at once (prologue); V role only
    request_piece(slot_bytes, P0{});
    request_piece(slot_bytes, P1{});
    request_piece(slot_bytes, P2{});
    request_piece(slot_bytes, P3{});
    request_piece(slot_bytes, P4{});
  };
  auto wait_tiles = [&]() LMK_INL {                        // all but this wave's two newest tiles have landed
    if (!role_k) wait_vmcnt<2 * C::PER_TILE_V>();
  };

  auto zero16 = [](f32x16_t& x) LMK_INL {
#pragma unroll
    for (int r = 0; r < 16; ++r) x[r] = 0.f;
  };
  auto row_tile = [&](int tile_bytes, f32x16_t& s) LMK_INL {   // (32 rows of the LDS tile) x (this wave's 32 keys)
    zero16(s);
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) s = mfma32<T>(*(const u32x4_t*)(smem + tile_bytes + koff[ks]), bf[ks], s);
  };
  // second product of a tile: acc[dc] += (tile at tile_bytes)^T x (packed B operands: rows 0..15, 16..31).
  // Its A operands do not depend on anything computed in the iteration, so they are fetched from LDS
  // during the first product (trfrag), one per MFMA slot, and are in registers when it starts.
  constexpr int NB = 2 * C::DC;
  auto trfrag = [&](int tile_bytes, int n) LMK_INL {
    const int j2 = n / C::DC, dc = n % C::DC;
    const int base = tile_bytes + 16 * j2 * C::ROWB;
    const u32x2_t a0 = lds_read_tr(smem + base + voff[dc][0]), a1 = lds_read_tr(smem + base + voff[dc][1]);
    const u32x4_t a = {a0[0], a0[1], a1[0], a1[1]};
    return a;
  };
  auto tr_product = [&](const u32x4_t* tf, const u32x4_t* pk, f32x16_t* acc) LMK_INL {
#pragma unroll
    for (int n = 0; n < NB; ++n) acc[n % C::DC] = mfma32<T>(tf[n], pk[n / C::DC], acc[n % C::DC]);
  };

  // ---- V role: one query tile i.  S of tile i+1 (slot nslot) is interleaved with W of tile i.
  auto body_v = [&](auto Mc, int i, int cslot, int nslot, int rslot, int par, f32x16_t& s, f32x16_t& sn, f32x16_t* acc, auto sync) LMK_INL {
    constexpr bool MASKED = decltype(Mc)::value;
    const int CST = cslot + 2 * C::TILE_BYTES + tile * 1024;   // this key tile's terms: a, nD, dslm, mhat, delta
    const int krel = 32 * (kt - (PT + i)) + ql;            // key position relative to the query tile's first row
    const bool lmq = (PT + i) % C::TPB == C::TPB - 1;      // the tile's last row is its block's landmark query
    const int xoff = (MASKED ? CST + 384 : (lm_lane ? C::CONST_OFF : CST)) + 16 * h;
    // terms of rows 8g + 4h .. +3, fetched two MFMA slots ahead of the slice that uses them (slot m works
    // on registers r with r / 4 == grp(m)): at the top of the iteration only what the first MFMA and the
    // first slice need is asked for, in that order, because LDS answers a wave in order
    float4 x4[4];
    auto ldx = [&](int g) LMK_INL { x4[g] = *(const float4*)(smem + xoff + 32 * g); };
    auto grp = [](int m) LMK_INL { return ((m * 16) / C::KS) >> 2; };
    u32x4_t wf[2];
    float w[16];
    auto elementwise = [&](int r) LMK_INL {                // register r <-> query row 8*(r/4) + 4h + r%4
      const int g = r >> 2, e = r & 3;
      const float xa = (e == 0) ? x4[g].x : (e == 1) ? x4[g].y : (e == 2) ? x4[g].z : x4[g].w;
      float ex = fast_exp2(__builtin_fmaf(s[r], c2, -xa));
      if (MASKED) {
        // key visible to this query row?  the landmark row of a block looks one position to the left
        const int qloc = 8 * g + 4 * h + e;
        ex = (krel <= qloc - ((qloc == 31 && lmq) ? 1 : 0)) ? ex : 0.f;
      }
      w[r] = ex;
      if (r & 1) {
        uint32_t pk = pack2<T>(w[r - 1], w[r]);
        asm volatile("" : "+v"(pk));                       // pins this slice between its two MFMAs
        wf[r >> 3][(r >> 1) & 3] = pk;
      }
    };
    zero16(sn);
    constexpr int PF = 2;
    u32x4_t fr[C::KS + PF], tf[NB];
#pragma unroll
    for (int m = 0; m < PF; ++m) fr[m] = *(const u32x4_t*)(smem + nslot + koff[m]);
    __builtin_amdgcn_sched_barrier(0);
    ldx(0);
    if (grp(1) != 0) ldx(grp(1));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < C::KS; ++m) {
      if (m + PF < C::KS) fr[m + PF] = *(const u32x4_t*)(smem + nslot + koff[m + PF]);
      if (m + 2 < C::KS && grp(m + 2) != grp(m + 1)) ldx(grp(m + 2));
#pragma unroll
      for (int n = (m * NB) / C::KS; n < ((m + 1) * NB) / C::KS; ++n) tf[n] = trfrag(cslot + C::TILE_BYTES, n);
      if (m == 0) request_piece(rslot, P0{});              // tile i+4, into the slot tile i-2 has left
      if (m == 1) request_piece(rslot, P1{});
      if (m == 2) request_piece(rslot, P2{});
      if (m == 3) request_piece(rslot, P3{});
      if (m == 4) request_piece(rslot, P4{});
      sn = mfma32<T>(fr[m], bf[m], sn);
#pragma unroll
      for (int r = (m * 16) / C::KS; r < ((m + 1) * 16) / C::KS; ++r) elementwise(r);
      __builtin_amdgcn_sched_barrier(0);
    }
    unsigned char* xp = smem + C::XCH_OFF + (par * C::NKT + tile) * C::XCH_TILE + lane * 16;
    *(u32x4_t*)(xp) = wf[0];
    *(u32x4_t*)(xp + 1024) = wf[1];
    sync();                                                // the iteration's barrier: what follows needs no LDS
    __builtin_amdgcn_sched_barrier(0);                     // keeps the MFMAs below behind the barrier
    tr_product(tf, wf, acc);                               // dV^T += dO^T W
  };

  // ---- K role: dP of tile i (slot cslot) interleaved with dS of tile i-1 (slot pslot), then dK of tile i-1.
  // MASKED: tile i-1 lies in the key tile's block or is not visible yet.
  auto body_k = [&](auto Mc, int cslot, int pslot, int par_prev, f32x16_t& dpp, f32x16_t& dpn, f32x16_t* acc, auto sync) LMK_INL {
    constexpr bool masked = decltype(Mc)::value;
    const int CST = pslot + 2 * C::TILE_BYTES + tile * 1024;
    // y: subtrahend of dP, z: addend of dS  (byte offsets of 32-float arrays)
    const int yoff = (masked ? CST + 512 : CST + 128) + 16 * h;
    const int zoff = ((!masked && lm_lane) ? CST + 256 : C::CONST_OFF + 128) + 16 * h;
    float4 y4[4], z4[4];                                   // fetched two MFMA slots ahead, as in the V role
    auto ldyz = [&](int g) LMK_INL {
      y4[g] = *(const float4*)(smem + yoff + 32 * g);
      z4[g] = *(const float4*)(smem + zoff + 32 * g);
    };
    auto grp = [](int m) LMK_INL { return ((m * 16) / C::KS) >> 2; };
    const unsigned char* xp = smem + C::XCH_OFF + (par_prev * C::NKT + tile) * C::XCH_TILE + lane * 16;
    u32x4_t wv[2];
    u32x4_t df[2];
    float ds[16];
    auto elementwise = [&](int r) LMK_INL {
      const int g = r >> 2, e = r & 3;
      const float ya = (e == 0) ? y4[g].x : (e == 1) ? y4[g].y : (e == 2) ? y4[g].z : y4[g].w;
      const float za = (e == 0) ? z4[g].x : (e == 1) ? z4[g].y : (e == 2) ? z4[g].z : z4[g].w;
      const uint32_t pk = wv[r >> 3][(r >> 1) & 3];
      const float wr = (r & 1) ? unpack_hi<T>(pk) : unpack_lo<T>(pk);
      ds[r] = __builtin_fmaf(wr, dpp[r] - ya, za);
      if (r & 1) {
        uint32_t pd = pack2<T>(ds[r - 1], ds[r]);
        asm volatile("" : "+v"(pd));                       // pins this slice between its two MFMAs
        df[r >> 3][(r >> 1) & 3] = pd;
      }
    };
    zero16(dpn);
    constexpr int PF = 2;
    u32x4_t fr[C::KS + PF], tf[NB];
#pragma unroll
    for (int m = 0; m < PF; ++m) fr[m] = *(const u32x4_t*)(smem + cslot + C::TILE_BYTES + koff[m]);
    __builtin_amdgcn_sched_barrier(0);
    wv[0] = *(const u32x4_t*)(xp);
    ldyz(0);
    if (grp(1) != 0) ldyz(grp(1));
    wv[1] = *(const u32x4_t*)(xp + 1024);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < C::KS; ++m) {
      if (m + PF < C::KS) fr[m + PF] = *(const u32x4_t*)(smem + cslot + C::TILE_BYTES + koff[m + PF]);
      if (m + 2 < C::KS && grp(m + 2) != grp(m + 1)) ldyz(grp(m + 2));
#pragma unroll
      for (int n = (m * NB) / C::KS; n < ((m + 1) * NB) / C::KS; ++n) tf[n] = trfrag(pslot, n);
      dpn = mfma32<T>(fr[m], bf[m], dpn);
#pragma unroll
      for (int r = (m * 16) / C::KS; r < ((m + 1) * 16) / C::KS; ++r) elementwise(r);
      __builtin_amdgcn_sched_barrier(0);
    }
    // The two roles meet the iteration's barrier in opposite phases: this role has its second product
    // (operands in registers, matrix pipe only) in front of the barrier, the V role behind it, so one
    // wave's MFMA-only stretch coincides with the other's LDS-and-vector stretch on their shared SIMD.
    tr_product(tf, df, acc);                               // dK^T += Q^T dS
    __builtin_amdgcn_sched_barrier(0);
    sync();
  };

  // this wave's stationary operand for key tile kt_i: K fragments (V role) or V fragments (K role), lane = key.
  // An item's operand is asked for at the end of the item before it, in front of that item's stores: behind them
  // the wait for it would also be the wait for the stores' acknowledgements.
  auto load_stationary = [&](int kt_i) LMK_INL {
    const char* src = role_k ? (const char*)p.v + 2 * (b_ * p.vs_b + hh * p.vs_h)
                             : (const char*)p.k + 2 * (b_ * p.ks_b + hh * p.ks_h);
    const int64_t rs = role_k ? p.vs_r : p.ks_r;
    const bool act = kt_i < nkt;
    int ln;                                                // the address is formed here from the lane id, not from values
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));   // kept across the loops (and spilled)
    int kr = kt_i * 32 + (ln & 31);
    if constexpr (VIRT) kr = slot_to_token_row_clamped<BS>(act ? kr : 0, p.n_real, nfull_k, seg_k);
    const char* row = src + 2 * ((int64_t)kr * rs + 8 * (ln >> 5));
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) {
      u32x4_t z = {0, 0, 0, 0};
      bf[ks] = z;
      if (act) bf[ks] = *(const u32x4_t*)(row + 32 * ks);
    }
  };
  // consume the operand at once: no wait for these loads can then end up inside the loop, where it would
  // drain the ring; the explicit wait covers everything this wave asked for up to and including the operand, which
  // the compiler does not count.  newer: what the wave has issued behind the operand's loads (an item's stores).
  // (await_stationary: wait_vmcnt<newer operations>() in front of this)
  auto use_stationary = [&]() LMK_INL {
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) asm volatile("" : "+v"(bf[ks]));
  };
  // an item's stores, issued behind the next item's loads: without rows that have no token their number is fixed
  // (such rows' stores are skipped lane by lane)
  constexpr int kStoresNewer = VIRT ? 0 : 2 * C::DC;
  // The end of item c: its accumulators leave, and the wave turns to the item behind it, if there is one (the ring
  // already holds that item's first tiles).  Returns that item's index, or n_c.
  auto finish_item = [&](int c, const f32x16_t* acc, char* dst, int64_t rs, float scl, auto store_acc) LMK_INL {
    const int c_nx = next_item(c + 1);
    if (c_nx < n_c) {
      // the wait stands in each branch, behind a known number of newer operations: the compiler puts its own wait for
      // these loads where their registers are first used, counted along the path with the fewest newer operations
      load_stationary(item_kvt(c_nx) * C::NKT + tile);
      if (active) {
        store_acc(acc, dst, rs, scl);
        wait_vmcnt<kStoresNewer>();
        use_stationary();
      } else {
        wait_vmcnt<0>();
        use_stationary();
      }
      set_item(c_nx);
      announce_next(c_nx);
    } else if (active) {
      store_acc(acc, dst, rs, scl);
    }
    return c_nx;
  };

  // ---- prologue of the first item.  The stationary operand and the first two tiles are asked for first and
  // awaited; tiles j_first+2, +3 go out behind that wait, so the workgroup does not sit through four tiles'
  // worth of traffic (every workgroup of a launch round starts at the same moment) before its first product.
  load_stationary(kt);
  if (!role_k) {
    request(0);
    request(C::BUF_BYTES);
  }
  if (tid < 64) ((float*)(smem + C::CONST_OFF))[tid] = (tid < 32) ? 1e30f : 0.f;
  wait_vmcnt<0>();
  use_stationary();
  if (!role_k) {
    request(2 * C::BUF_BYTES);
    request(3 * C::BUF_BYTES);
  }

  wait_tiles();
  __syncthreads();

  // Per item: iteration i = j_first .. nq, one barrier each, in both roles.  V role: tiles i (W, dV) and i+1 (S).
  // K role: tiles i (dP) and i-1 (dS, dK); it has nothing to finish in the first iteration and only
  // finishes in the last.  The ring slot of tile i is a wave-uniform counter that runs on from item to item: the
  // slots behind an item's last tile already hold the next item's first tiles.
  auto wrap = [](int x) LMK_INL { return x >= C::NBUF ? x - C::NBUF : x; };
  // An item's accumulators leave as row segments (store_tile_rows) through this wave's 2 KB of the W hand-over
  // area: the first role uses parity 0, the second parity 1 -- behind the item's last barrier nobody reads W there,
  // and the next item's first W goes to parity 0 behind the first role's own stores.  (Stored straight from the
  // registers the eight waves' 128 store instructions at an item's end took 4 us.)
  auto store_acc = [&](const f32x16_t* acc, char* dst, int64_t rs, float scl) LMK_INL {
    store_tile_rows<T, C::DC, VIRT>(acc, scl, C::XCH_OFF + ((role_k ? 1 : 0) * C::NKT + tile) * C::XCH_TILE,
                              [&](int r) LMK_INL -> char* {
      int kr = kt * 32 + r;
      if constexpr (VIRT) {                                // a slot without a token: nothing to store
        kr = slot_to_token_row<BS>(kr, p.n_real, nfull_k, seg_k);
        if (kr < 0) return nullptr;
      }
      return dst + 2 * ((int64_t)kr * rs);
    });
  };
  if (!role_k) {
    f32x16_t acc[C::DC];                                   // dV^T: rows = d, lane = key
    f32x16_t cur, nxt;                                      // S of tiles i and i+1
    int sc = 0;                                            // slot of the item's tile i
    for (int c = 0; c < n_c;) {
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc) zero16(acc[dc]);
      row_tile(sc * C::BUF_BYTES, cur);                     // S of the first tile
      auto step = [&](auto Mc, int i) LMK_INL {
        // the barrier sits between the two products: the second one has its operands in registers, so
        // its MFMAs run while the workgroup's stragglers arrive and the next tile's operands are fetched
        auto sync = [&]() LMK_INL {
          wait_vmcnt<2 * C::PER_TILE_V>();                  // tile i+2 has landed (tiles i+3, i+4 may be in flight)
          __syncthreads();
        };
        body_v(Mc, i, sc * C::BUF_BYTES, wrap(sc + 1) * C::BUF_BYTES, wrap(sc + 4) * C::BUF_BYTES, (i - j_first) & 1, cur, nxt, acc, sync);
        cur = nxt;
        sc = wrap(sc + 1);
      };
      // own block and tiles that cannot see these keys yet come first, then every later tile sees all keys:
      // two loops, so that each has one code path and the accumulators stay where they are
      int i = j_first;
      const int i_full = min(nq, max(j_first, kt_end - PT));
      for (; i < i_full; ++i) step(std::true_type{}, i);
      for (; i < nq; ++i) step(std::false_type{}, i);
      // the K role finishes tile nq-1 in one more iteration; nothing is requested here (the K role's request of
      // that iteration is the one its first iteration of the next item leaves out)
      wait_vmcnt<2 * C::PER_TILE_V>();
      __syncthreads();
      c = finish_item(c, acc, (char*)p.dv + 2 * (b_ * p.dvs_b + hh * p.dvs_h), p.dvs_r, 1.f, store_acc);
    }
    wait_vmcnt<0>();                                       // nothing may still be writing LDS when the wave ends
  } else {
    f32x16_t acc[C::DC];                                   // dK^T: rows = d, lane = key
    f32x16_t prv, cur;                                      // dP of tiles i-1 and i
    int sc = 0;                                            // slot of the item's first tile, then of tile i
    for (int c = 0; c < n_c;) {
#pragma unroll
      for (int dc = 0; dc < C::DC; ++dc) zero16(acc[dc]);
      int cs = sc * C::BUF_BYTES, ps;                       // byte offsets of the slots of tiles i and i-1
      row_tile(cs + C::TILE_BYTES, prv);                    // dP of the first tile
      __syncthreads();                                      // this role has no loads in flight: the V role's waits cover the ring
      auto sync = [&]() LMK_INL { __syncthreads(); };
      int par = 0;                                          // parity of tile i-1 in the W hand-over
      auto advance = [&]() LMK_INL {
        ps = cs;
        cs = (cs == (C::NBUF - 1) * C::BUF_BYTES) ? 0 : cs + C::BUF_BYTES;
      };
      advance();
      // iterations i = j_first+1 .. nq.  First those whose tile i-1 is masked (in the key tile's block or not
      // visible yet; a handful), then the rest two at a time, so that dP of tiles i-1 and i swap registers
      // instead of being copied.
      int i = j_first + 1;
      const int i_masked_end = min(nq, kt_end - PT);        // last i with PT + (i-1) < kt_end
      for (; i <= i_masked_end; ++i) {
        body_k(std::true_type{}, cs, ps, par, prv, cur, acc, sync);
        prv = cur;
        par ^= 1;
        advance();
      }
      for (; i + 1 <= nq; i += 2) {
        body_k(std::false_type{}, cs, ps, par, prv, cur, acc, sync);
        advance();
        body_k(std::false_type{}, cs, ps, par ^ 1, cur, prv, acc, sync);
        advance();
      }
      if (i <= nq) {
        body_k(std::false_type{}, cs, ps, par, prv, cur, acc, sync);
        advance();
      }
      sc = ps / C::BUF_BYTES;                               // the slot behind the last tile: the next item's first tile
      c = finish_item(c, acc, (char*)p.dk + 2 * (b_ * p.dks_b + hh * p.dks_h), p.dks_r, p.scale, store_acc);
    }
    wait_vmcnt<0>();
  }
}

#undef LMK_INL

template <class T, int D, int BS, bool VIRT, bool SEG = false>
static int launch_dkdv32_t(const BwdParams& p, hipStream_t stream) {
  using C = Dkv32Cfg<T, D, BS>;
  auto kern = lmk_bwd_dkdv32_kernel<T, D, BS, VIRT, SEG>;
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, C::LDS_BYTES, lds_ok)) return rc;
  // workgroups per head: enough for about one workgroup per CU, at most four 128-key tiles each
  const int64_t items = (int64_t)p.n_kvtiles * p.B * p.H;
  int per_wg = (int)(items / cu_count());
  per_wg = per_wg < 1 ? 1 : (per_wg > 4 ? 4 : per_wg);
  const int groups = (p.n_kvtiles + per_wg - 1) / per_wg;
  hipLaunchKernelGGL(kern, dim3(groups * p.B * p.H), dim3(C::NTHR), C::LDS_BYTES, stream, p);
  return (int)hipGetLastError();
}

template <class T, int D>
static int launch_dkdv32_b(const BwdParams& p, int BS, hipStream_t stream) {
  if (p.Lq_real > 0 && p.seg != nullptr) {                 // token layout, blocks of unequal length
    if (BS == 64) return launch_dkdv32_t<T, D, 64, true, true>(p, stream);
    if (BS == 128) return launch_dkdv32_t<T, D, 128, true, true>(p, stream);
    return LMK_ERR_UNSUPPORTED;
  }
  if (p.Lq_real > 0) {                                     // token layout: blocks narrower than their 64 or 128 slots
    if (BS == 64) return launch_dkdv32_t<T, D, 64, true>(p, stream);
    if (BS == 128) return launch_dkdv32_t<T, D, 128, true>(p, stream);
    return LMK_ERR_UNSUPPORTED;
  }
  if (BS == 32) return launch_dkdv32_t<T, D, 32, false>(p, stream);
  if (BS == 64) return launch_dkdv32_t<T, D, 64, false>(p, stream);
  if (BS == 128) return launch_dkdv32_t<T, D, 128, false>(p, stream);
  return LMK_ERR_UNSUPPORTED;
}

int launch_bwd_dkdv32(const BwdParams& p, int D, int BS, int dtype, hipStream_t stream) {
  if (dtype == LMK_DTYPE_BF16) {
    if (D == 128) return launch_dkdv32_b<bf16_t, 128>(p, BS, stream);
    if (D == 64) return launch_dkdv32_b<bf16_t, 64>(p, BS, stream);
  } else if (dtype == LMK_DTYPE_F16) {
    if (D == 128) return launch_dkdv32_b<f16_t, 128>(p, BS, stream);
    if (D == 64) return launch_dkdv32_b<f16_t, 64>(p, BS, stream);
  }
  return LMK_ERR_UNSUPPORTED;
}

}  // namespace lmk
