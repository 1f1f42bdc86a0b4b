// Shared device helpers for the gfx950 (CDNA4) landmark-attention kernels.
//
// Everything here is written for wave64 and the 32x32x16 bf16/f16 MFMA:
//   A (32 x 16): lane l holds row  l%32, k = 8*(l/32) .. +7   (8 x 16 bit = 4 VGPRs)
//   B (16 x 32): lane l holds col  l%32, k = 8*(l/32) .. +7
//   C (32 x 32): lane l holds col  l%32, rows 8*(r/4) + 4*(l/32) + r%4 for r = 0..15
// The kernels compute S^T = K Q^T so that a query owns one lane pair (l, l^32):
// a softmax over the 32 keys of a tile is 16 in-lane values plus one
// v_permlane32_swap.  The C registers r = 8j .. 8j+7 of a lane then hold keys
// 16j + {0..3, 8..11} + 4*(l/32), which is used directly as the B operand of the
// next product with the same key permutation applied to its A operand.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lmk {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(32 * sizeof(float)))) float f32x32_t;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4_t;

struct bf16_t {};  // element tags
struct f16_t {};

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// ---- MFMA ---------------------------------------------------------------
template <class T>
__device__ __forceinline__ f32x16_t mfma32(u32x4_t a, u32x4_t b, f32x16_t c);
template <>
__device__ __forceinline__ f32x16_t mfma32<bf16_t>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x16_t mfma32<f16_t>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

// ---- fp32 <-> 16-bit ------------------------------------------------------
template <class T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <>
__device__ __forceinline__ uint32_t pack2<bf16_t>(float lo, float hi) {
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));  // v_cvt_pk_bf16_f32 (RNE)
}
template <>
__device__ __forceinline__ uint32_t pack2<f16_t>(float lo, float hi) {
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
}

template <class T>
__device__ __forceinline__ float unpack_lo(uint32_t u);
template <class T>
__device__ __forceinline__ float unpack_hi(uint32_t u);
template <>
__device__ __forceinline__ float unpack_lo<bf16_t>(uint32_t u) { return __uint_as_float(u << 16); }
template <>
__device__ __forceinline__ float unpack_hi<bf16_t>(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
template <>
__device__ __forceinline__ float unpack_lo<f16_t>(uint32_t u) {
  return (float)__builtin_bit_cast(f16x2_t, u)[0];
}
template <>
__device__ __forceinline__ float unpack_hi<f16_t>(uint32_t u) {
  return (float)__builtin_bit_cast(f16x2_t, u)[1];
}

// ---- lane-pair (l, l^32) exchange ----------------------------------------
// v_permlane32_swap exchanges the upper half of its first operand with the lower
// half of its second; with both operands equal the two results are, for every
// lane, the value held by the low lane and by the high lane of its pair.
__device__ __forceinline__ float pair_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float pair_hi(float x) {  // value of the lane with l >= 32
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[1]);
}
__device__ __forceinline__ float pair_lo(float x) {  // value of the lane with l < 32
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// ---- LDS tile addressing ---------------------------------------------------
// Tiles are stored row-major, 2*D bytes per row, in 16-byte chunks whose index is
// XOR-swizzled with f(row) = ((row & 3) << 2) | ((row >> 2) & 3).  One layout serves
// both ways a tile is read:
//   * as an MFMA operand with the head dim along k: lane -> (row l%32, one 16-byte chunk);
//     f is a bijection on 16 consecutive rows, so 16 lanes cover all 16 chunk columns;
//   * transposed, with ds_read_b64_tr_b16: a 16-lane group touches 4 consecutive rows x
//     32 bytes; the (row & 3) << 2 term sends the four rows to four different 64-byte
//     column groups.
template <int D>
__device__ __forceinline__ int tile_off(int row, int chunk) {
  constexpr int CH = D / 8;
  const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & (CH - 1);
  return row * (2 * D) + ((chunk ^ f) << 4);
}

typedef __attribute__((address_space(3))) s16x4_t* lds_s16x4_ptr;

// Transposed LDS read: inside each group of 16 lanes, lane i supplies the address of
// 4 consecutive 16-bit columns of row i/4 (columns 4*(i%4)..+3 of a 4 x 16 patch) and
// receives the 4 rows of column i.
__device__ __forceinline__ u32x2_t lds_read_tr(const unsigned char* p) {
  s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
  return __builtin_bit_cast(u32x2_t, v);
}

// LDS access by byte address.  A kernel whose only LDS is its dynamic array sees that array at LDS
// address 0 (the direct global->LDS loads rely on the same fact), so offsets into it are LDS
// addresses.  Going through an integer keeps the compiler from adding the array's (zero) base to
// every address with a vector instruction.
typedef __attribute__((address_space(3))) u32x4_t* lds_u32x4_ptr;
typedef __attribute__((address_space(3))) float* lds_f32_ptr;
typedef __attribute__((address_space(3))) u32x2_t* lds_u32x2_ptr;
__device__ __forceinline__ u32x4_t lds_ld128(int addr) { return *(lds_u32x4_ptr)(uintptr_t)(uint32_t)addr; }
__device__ __forceinline__ void lds_st128(int addr, u32x4_t v) { *(lds_u32x4_ptr)(uintptr_t)(uint32_t)addr = v; }
__device__ __forceinline__ void lds_st32(int addr, float v) { *(lds_f32_ptr)(uintptr_t)(uint32_t)addr = v; }
__device__ __forceinline__ u32x2_t lds_ld_tr(int addr) {
  s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(uintptr_t)(uint32_t)addr);
  return __builtin_bit_cast(u32x2_t, v);
}

// Transposed fragment of a row-major tile (A operand, rows = 32 head dims of chunk dc,
// k = 16 tile rows of step j of the 32-row tile at LDS row base rb) in the row order of
// the C layout: register pair 0 holds rows 16j + 4h + {0..3}, pair 1 rows 16j + 8 + 4h + {0..3}.
template <int D>
__device__ __forceinline__ u32x4_t load_tr_frag(const unsigned char* vbuf, int rb, int j, int dc, int lane) {
  const int h = lane >> 5, i = lane & 15, g2 = (lane >> 4) & 1;
  const int col = 32 * dc + 16 * g2 + 4 * (i & 3);
  const int row0 = rb + 16 * j + 4 * h + (i >> 2);
  u32x2_t a = lds_read_tr(vbuf + tile_off<D>(row0, col >> 3) + ((col >> 2) & 1) * 8);
  u32x2_t b = lds_read_tr(vbuf + tile_off<D>(row0 + 8, col >> 3) + ((col >> 2) & 1) * 8);
  u32x4_t r = {a[0], a[1], b[0], b[1]};
  return r;
}

// Row fragment (A operand, rows = the 32 rows of the tile at LDS row base rb, k = head dims
// 16*ks + 8*(l/32) .. +7).
template <int D>
__device__ __forceinline__ u32x4_t load_row_frag(const unsigned char* kbuf, int rb, int ks, int lane) {
  const int row = rb + (lane & 31);
  return *(const u32x4_t*)(kbuf + tile_off<D>(row, 2 * ks + (lane >> 5)));
}

// Blocks of n tokens worked on in BS slots (n <= BS): slot s < n-1 of a complete block is its normal token s, the
// last slot its landmark (token n-1), the slots in between hold nothing; a partial last block (n_full = number of
// complete blocks) keeps its tokens in its first slots.  Slot row -> token row of the tensor, or -1.
template <int BS>
__device__ __forceinline__ int slot_to_token_row(int slot_row, int n, int n_full) {
  const int blk = slot_row / BS, s = slot_row % BS;
  int tok = s;
  if (blk < n_full) tok = (s == BS - 1) ? n - 1 : (s < n - 1 ? s : -1);
  return tok < 0 ? -1 : blk * n + tok;
}
// The same for loads whose result is masked afterwards: a slot without a token reads its block's first token.
template <int BS>
__device__ __forceinline__ int slot_to_token_row_clamped(int slot_row, int n, int n_full) {
  const int r = slot_to_token_row<BS>(slot_row, n, n_full);
  return r < 0 ? (slot_row / BS) * n : r;
}

// Blocks of unequal length (landmarks at irregular positions): seg[b] is the first token of block b and
// seg[b + 1] - seg[b] its length, at most BS; the first n_full blocks end in their landmark, a last block behind
// them has none.  `seg` points at the entry of the first block of the tensor whose rows are asked for (the queries
// of a call with history start n_prefix blocks into the keys' table).  Null: every block holds n tokens.
template <int BS>
__device__ __forceinline__ int slot_to_token_row(int slot_row, int n, int n_full, const int* seg) {
  if (seg == nullptr) return slot_to_token_row<BS>(slot_row, n, n_full);
  const int blk = slot_row / BS, s = slot_row % BS;
  const int first = seg[blk], len = seg[blk + 1] - first;
  int tok = s < len ? s : -1;
  if (blk < n_full) tok = (s == BS - 1) ? len - 1 : (s < len - 1 ? s : -1);
  return tok < 0 ? -1 : first - seg[0] + tok;
}
template <int BS>
__device__ __forceinline__ int slot_to_token_row_clamped(int slot_row, int n, int n_full, const int* seg) {
  if (seg == nullptr) return slot_to_token_row_clamped<BS>(slot_row, n, n_full);
  const int r = slot_to_token_row<BS>(slot_row, n, n_full, seg);
  return r < 0 ? seg[slot_row / BS] - seg[0] : r;
}
// normal keys of block blk of the keys (slots behind them, up to the landmark's, hold nothing)
template <int BS>
__device__ __forceinline__ int block_normal_keys(int blk, int n, int n_full, const int* seg) {
  if (seg == nullptr) return n - 1;
  return blk < n_full ? seg[blk + 1] - seg[blk] - 1 : BS - 1;
}

// A wave's 32 x (32 DC) accumulator tile in the MFMA C layout -- register 4 g + e of chunk dc holds (row ql,
// column 32 dc + 8 g + 4 h + e), ql = lane % 32, h = lane / 32 -- scaled per lane, rounded to T and stored as rows.
// Stored straight from the registers every store instruction touches 32 rows, 16 bytes each, and a workgroup's
// waves doing that together keep the compute unit's memory pipeline busy for microseconds; so each 32-column chunk
// goes through 2 KB of LDS that belong to this wave alone (at LDS byte address `xb`; the kernels' dynamic array
// starts at address 0) and leaves as 64-byte row segments, 16 rows per store instruction.  row_ptr(r): where row r of the tile (r = 0..31) starts in memory, or null to skip it.
// Everything per lane is formed here from the lane id: kept across a kernel's loops such values are spilled, and a
// reload's wait for the memory counter also waits for whatever the kernel has in flight.
// MAY_SKIP = false: row_ptr never returns null, and the tile's 2 DC store instructions are issued unconditionally
// (a caller that counts its memory operations needs that).
template <class T, int DC, bool MAY_SKIP = true, class RowPtr>
__device__ __forceinline__ void store_tile_rows(const f32x16_t* acc, float scl, int xb, RowPtr row_ptr) {
  int ln;                                                  // lane id without a long-lived register
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
  const int rk = ln >> 2, rq = ln & 3;
  const int wr = xb + (ln & 31) * 64 + 8 * (ln >> 5);
  char* out[2];
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    out[k] = row_ptr(rk + 16 * k);
    if (!MAY_SKIP || out[k] != nullptr) out[k] += 16 * rq;
  }
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const u32x2_t o2 = {pack2<T>(acc[dc][4 * g + 0] * scl, acc[dc][4 * g + 1] * scl),
                          pack2<T>(acc[dc][4 * g + 2] * scl, acc[dc][4 * g + 3] * scl)};
      *(lds_u32x2_ptr)(uintptr_t)(uint32_t)(wr + 16 * g) = o2;
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const u32x4_t v = lds_ld128(xb + (rk + 16 * k) * 64 + 16 * rq);
      if (!MAY_SKIP || out[k] != nullptr) *(u32x4_t*)(out[k] + 64 * dc) = v;
    }
  }
}

template <class T>
__device__ __forceinline__ float round_to(float x) {  // fp32 -> T (RNE) -> fp32
  return unpack_lo<T>(pack2<T>(x, 0.f));
}

// rotary on 8 consecutive head dims held as 4 packed dwords; `other` holds the chunk D/2 away
template <class T>
__device__ __forceinline__ void rotate_chunk(const u32x4_t x, const u32x4_t other, const u32x4_t c, const u32x4_t s,
                                             bool upper_half, float* out) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float x0 = unpack_lo<T>(x[i]), x1 = unpack_hi<T>(x[i]);
    float r0 = unpack_lo<T>(other[i]), r1 = unpack_hi<T>(other[i]);
    if (!upper_half) {  // rotate_half: first half gets -x[d + D/2], second half gets x[d - D/2]
      r0 = -r0;
      r1 = -r1;
    }
    float a0 = round_to<T>(x0 * unpack_lo<T>(c[i])), a1 = round_to<T>(x1 * unpack_hi<T>(c[i]));
    float b0 = round_to<T>(r0 * unpack_lo<T>(s[i])), b1 = round_to<T>(r1 * unpack_hi<T>(s[i]));
    // The rounded products are opaque to the compiler: with f16 it would otherwise turn
    // round(round(x*c) + round(r*s)) into a half-precision fused multiply-add, which skips a rounding.
    asm volatile("" : "+v"(a0), "+v"(a1), "+v"(b0), "+v"(b1));
    out[2 * i] = round_to<T>(a0 + b0);
    out[2 * i + 1] = round_to<T>(a1 + b1);
  }
}

// Rotary embedding of a wave's Q (or K) operand fragments in registers: fragment ks of a lane holds head dims
// 16 ks + 8 h .. + 7 of its row, whose rotary partners (D/2 away) sit in fragment ks ^ (KS/2) of the same lane.
// cos_row / sin_row: the row's table rows (D values each).  Same three roundings as rotate_chunk.
template <class T, int KS>
__device__ __forceinline__ void rotate_fragments(u32x4_t* f, const char* cos_row, const char* sin_row, int h) {
  u32x4_t raw[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) raw[ks] = f[ks];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const u32x4_t c = *(const u32x4_t*)(cos_row + 16 * (2 * ks + h));
    const u32x4_t s = *(const u32x4_t*)(sin_row + 16 * (2 * ks + h));
    float o[8];
    rotate_chunk<T>(raw[ks], raw[ks ^ (KS / 2)], c, s, ks >= KS / 2, o);
    const u32x4_t r = {pack2<T>(o[0], o[1]), pack2<T>(o[2], o[3]), pack2<T>(o[4], o[5]), pack2<T>(o[6], o[7])};
    f[ks] = r;
  }
}

}  // namespace lmk
