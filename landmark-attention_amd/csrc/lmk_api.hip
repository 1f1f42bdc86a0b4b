// C ABI of liblandmark_hip.so: argument validation on the host, then dispatch
// to the kernel launchers.  Declarations and the contract live in include/lmk.h.
#include <cmath>

#include <mutex>

#include "lmk_launch.hpp"

// Scratch memory of lmk_retrieve_topk_static: the selection's workspace (rotated landmark keys, their norms
// and the two score planes) for callers that may not allocate.  Every GPU the library runs on holds its own
// copy of this array, at its own address, until the process ends.  In host code the array's name is only a
// handle for hipGetSymbolAddress: kernels and copies get the device address that call returns.
#define LMK_STATIC_SCRATCH_BYTES (16u << 20)
static __device__ __align__(256) unsigned char scratch[LMK_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};          // device address of `scratch` on each device, looked up once

// Address of the current device's copy of `scratch`; *rc is 0 or a hipError_t.
void* static_scratch(int* rc) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    *rc = e != hipSuccess ? (int)e : (int)hipErrorInvalidDevice;
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));           // with device `dev` current
    if (e != hipSuccess || ptr == nullptr) {
      *rc = e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  *rc = 0;
  return g_scratch_ptr[dev];
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
bool stride_ok(int64_t s) { return (s & 7) == 0; }  // 8 elements x 2 bytes = 16 bytes

int check_tensor(const lmk_tensor4* t) {
  if (t == nullptr || t->ptr == nullptr) return LMK_ERR_NULL;
  if (!aligned16(t->ptr) || !stride_ok(t->stride_b) || !stride_ok(t->stride_h) || !stride_ok(t->stride_row))
    return LMK_ERR_ALIGN;
  if (t->stride_row <= 0) return LMK_ERR_SHAPE;   // rows are walked forwards
  return LMK_OK;
}

// The kernels address the rows of one (batch, head) slice with 32-bit byte offsets.
bool slice_fits_32bit(const lmk_tensor4* t, int rows) { return (int64_t)rows * t->stride_row * 2 < ((int64_t)1 << 32); }

int check_common(int B, int H, int Lq, int Lk, int D, float sm_scale, int block, int n_prefix, int dtype) {
  if (B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0 || n_prefix < 0) return LMK_ERR_SHAPE;
  if (!(D == 64 || D == 128)) return LMK_ERR_UNSUPPORTED;
  if (!(block == 32 || block == 64 || block == 128)) return LMK_ERR_UNSUPPORTED;
  if (!(dtype == LMK_DTYPE_BF16 || dtype == LMK_DTYPE_F16)) return LMK_ERR_UNSUPPORTED;
  if (Lk < Lq || (int64_t)Lk - Lq != (int64_t)n_prefix * block) return LMK_ERR_HISTORY;
  if (!std::isfinite(sm_scale) || !(sm_scale > 0.f)) return LMK_ERR_SCALE;
  return LMK_OK;
}

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

struct RetrLayout {
  size_t lk_rot, lk_norm, approx, exact, total;
};

RetrLayout retr_layout(int B, int H, int T, int S, int D, int block) {
  const size_t bh = (size_t)B * H, nm = (size_t)(S / block);
  RetrLayout l;
  l.lk_rot = 0;
  l.lk_norm = align256(l.lk_rot + bh * (size_t)lmk::lk_tiles((int)nm) * (size_t)lmk::lk_tile_bytes(D));   // whole tiles of 32 keys
  l.approx = align256(l.lk_norm + bh * nm * 4);
  l.exact = align256(l.approx + bh * T * nm * 4);
  l.total = align256(l.exact + bh * T * nm * 4);
  return l;
}

int check_retrieval(int B, int H, int T, int S, int D, int block, int top_k, int dtype, int64_t n_pos) {
  if (B <= 0 || H <= 0 || T <= 0 || S <= 0) return LMK_ERR_SHAPE;
  if (!(D == 64 || D == 128)) return LMK_ERR_UNSUPPORTED;
  if (block < 2 || block > 4096) return LMK_ERR_UNSUPPORTED;
  if (!(dtype == LMK_DTYPE_BF16 || dtype == LMK_DTYPE_F16)) return LMK_ERR_UNSUPPORTED;
  if (S < block) return LMK_ERR_CACHE;          // at least one complete block; a shorter tail behind it is fine
  if (top_k < 1 || top_k > 64) return LMK_ERR_TOPK;
  if (n_pos < S) return LMK_ERR_TABLE;
  return LMK_OK;
}

void fill_retr_common(lmk::RetrParams& p, int B, int H, int T, int S, int D, int block, int top_k) {
  p.B = B; p.H = H; p.T = T; p.S = S; p.block = block;
  p.num_mems = S / block;                         // complete blocks; the S % block newest tokens are the tail
  p.k = top_k < p.num_mems ? top_k : p.num_mems;
  p.prefix_len = (int64_t)p.num_mems * block - (int64_t)(p.k + 1) * block;   // llama_mem.py:361 with full_len
  p.sqrt_hd = (float)std::sqrt((double)D);
}

// Shared by lmk_local_window (idx == nullptr) and lmk_gather_window.
int window_impl(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache, const int64_t* idx,
                       const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table,
                       const void* sin_table, int64_t table_stride_row, int64_t n_pos, const lmk_tensor4* q_win,
                       const lmk_tensor4* k_win, const lmk_tensor4* v_win, int B, int H, int T, int S, int D,
                       int block, int top_k, int dtype, void* stream) {
  int rc;
  if ((rc = check_tensor(q)) || (rc = check_tensor(kcache)) || (rc = check_tensor(vcache)) ||
      (rc = check_tensor(k_loc)) || (rc = check_tensor(v_loc)) || (rc = check_tensor(k_win)) ||
      (rc = check_tensor(v_win)))
    return rc;
  if (cos_table == nullptr || sin_table == nullptr) return LMK_ERR_NULL;
  if (!aligned16(cos_table) || !aligned16(sin_table) || !stride_ok(table_stride_row)) return LMK_ERR_ALIGN;
  if ((rc = check_retrieval(B, H, T, S, D, block, idx ? top_k : 1, dtype, n_pos))) return rc;
  const int inc = S % block;
  if (idx == nullptr && inc == 0) return LMK_ERR_CACHE;   // no tail, no selection: the new chunk alone is the window
  if (inc > 0 && T + inc > block) return LMK_ERR_SHAPE;   // llama_mem.py:330
  if (inc > 0 || q_win != nullptr) {                      // without a tail the queries need no padding rows
    if ((rc = check_tensor(q_win))) return rc;
  }
  lmk::WindowParams p = {};
  p.q = q->ptr; p.kcache = kcache->ptr; p.vcache = vcache->ptr; p.k_loc = k_loc->ptr; p.v_loc = v_loc->ptr;
  p.cos = cos_table; p.sin = sin_table;
  p.q_win = q_win ? q_win->ptr : nullptr; p.k_win = k_win->ptr; p.v_win = v_win->ptr;
  p.B = B; p.H = H; p.T = T; p.inc = inc;
  p.full_len = (int64_t)S - inc;
  p.tail_pos = p.full_len;
  p.block = block;
  p.num_mems = S / block;
  if (idx != nullptr) {
    p.idx = idx;
    p.k = top_k < p.num_mems ? top_k : p.num_mems;
    p.n_sel = p.k * block;
    p.prefix_len = p.full_len - (int64_t)(p.k + 1) * block;        // llama_mem.py:361
  }
  p.qs_b = q->stride_b; p.qs_h = q->stride_h; p.qs_r = q->stride_row;
  p.kcs_b = kcache->stride_b; p.kcs_h = kcache->stride_h; p.kcs_r = kcache->stride_row;
  p.vcs_b = vcache->stride_b; p.vcs_h = vcache->stride_h; p.vcs_r = vcache->stride_row;
  p.kls_b = k_loc->stride_b; p.kls_h = k_loc->stride_h; p.kls_r = k_loc->stride_row;
  p.vls_b = v_loc->stride_b; p.vls_h = v_loc->stride_h; p.vls_r = v_loc->stride_row;
  if (q_win) { p.qws_b = q_win->stride_b; p.qws_h = q_win->stride_h; p.qws_r = q_win->stride_row; }
  p.kws_b = k_win->stride_b; p.kws_h = k_win->stride_h; p.kws_r = k_win->stride_row;
  p.vws_b = v_win->stride_b; p.vws_h = v_win->stride_h; p.vws_r = v_win->stride_row;
  p.cs_r = table_stride_row;
  return lmk::launch_local_window(p, D, dtype, (hipStream_t)stream);
}

}  // namespace

extern "C" {

const char* lmk_strerror(int code) {
  switch (code) {
    case LMK_OK: return "ok";
    case LMK_ERR_NULL: return "a required pointer is NULL";
    case LMK_ERR_SHAPE: return "non-positive or inconsistent sizes";
    case LMK_ERR_UNSUPPORTED:
      return "unsupported head dim (64,128), block size (32,64,128) or dtype (bf16,f16), or a (batch, head) slice of 4 GiB or more";
    case LMK_ERR_ALIGN: return "pointer or stride not 16-byte aligned";
    case LMK_ERR_HISTORY: return "Lk - Lq must equal n_prefix * block";
    case LMK_ERR_PARTIAL: return "backward supported only for full blocks";
    case LMK_ERR_SCALE: return "softmax scale must be finite and > 0";
    case LMK_ERR_WORKSPACE: return "workspace too small";
    case LMK_ERR_CACHE: return "cache must hold at least one whole block";
    case LMK_ERR_TOPK: return "top_k must be in 1..64";
    case LMK_ERR_TABLE: return "rotary tables shorter than the cached length";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "unknown error";
}

const char* lmk_version(void) { return "landmark_hip 0.1 gfx950"; }

// block_real: tokens of each stored block that exist (== block for the plain entry points)
static int check_block_real(int block, int block_real) {
  if (block_real == block) return LMK_OK;
  if (!(block == 64 || block == 128)) return LMK_ERR_UNSUPPORTED;      // the block-32 kernels carry no padding mask
  if (block_real < 2 || block_real > block) return LMK_ERR_SHAPE;
  return LMK_OK;
}

struct RopeArgs {
  const void *cos, *sin;
  int64_t stride_row, n_pos;
  const int64_t* pos;
  int64_t pos_stride_b;
};

// Lq_real, Lk_real > 0: the tensors are in token layout (rows = tokens of blocks of block_real), Lq and Lk count slots
// Blocks of unequal length: the device copy of the table the kernels read and the number of complete blocks among
// the keys' (validated on the host by the entry points that take one).
struct SegArgs {
  const int* seg_dev;
  int n_full_k;
};

static int attn_fwd_impl(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                         float* L, float* M, int B, int H, int Lq, int Lk, int D, float sm_scale, int block,
                         int block_real, int n_prefix, int dtype, void* stream, const RopeArgs* rope = nullptr,
                         int Lq_real = 0, int Lk_real = 0, const float* group_scale = nullptr,
                         lmk::FwdParams* params_out = nullptr, const SegArgs* segs = nullptr) {
  int rc;
  if ((rc = check_tensor(q)) || (rc = check_tensor(k)) || (rc = check_tensor(v)) || (rc = check_tensor(o))) return rc;
  if (L == nullptr || M == nullptr) return LMK_ERR_NULL;
  if ((rc = check_common(B, H, Lq, Lk, D, sm_scale, block, n_prefix, dtype))) return rc;
  if ((rc = check_block_real(block, block_real))) return rc;
  if (!slice_fits_32bit(q, Lq) || !slice_fits_32bit(o, Lq) || !slice_fits_32bit(k, Lk) || !slice_fits_32bit(v, Lk))
    return LMK_ERR_UNSUPPORTED;
  if (rope != nullptr) {
    if (rope->cos == nullptr || rope->sin == nullptr || rope->pos == nullptr) return LMK_ERR_NULL;
    if (!aligned16(rope->cos) || !aligned16(rope->sin) || !stride_ok(rope->stride_row)) return LMK_ERR_ALIGN;
    if (rope->pos_stride_b < 0) return LMK_ERR_SHAPE;
    if (rope->n_pos < 1) return LMK_ERR_TABLE;
  }
  lmk::FwdParams p = {};
  if (rope != nullptr) {
    p.rope_cos = rope->cos; p.rope_sin = rope->sin; p.rope_pos = rope->pos;
    p.rope_pos_stride_b = rope->pos_stride_b; p.rope_cs_r = rope->stride_row; p.rope_n_pos = rope->n_pos;
  }
  p.n_real = block_real;
  p.Lq_real = Lq_real; p.Lk_real = Lk_real;
  if (segs != nullptr) {
    if (Lq_real <= 0 || group_scale != nullptr) return LMK_ERR_UNSUPPORTED;
    p.seg = segs->seg_dev;
    p.n_full_k = segs->n_full_k;
    p.n_full_q = segs->n_full_k - n_prefix;
  } else if (Lq_real > 0) {
    p.n_full_q = Lq_real / block_real;
    p.n_full_k = Lk_real / block_real;
  }
  if (group_scale != nullptr) {                            // (B*H, Lk_real / block_real, Lq_real) floats
    if (Lq_real <= 0) return LMK_ERR_UNSUPPORTED;
    p.group_scale = group_scale;
    p.gs_blk = Lq_real;
    p.gs_bh = (int64_t)(Lk_real / block_real) * Lq_real;
  }
  p.q = q->ptr; p.k = k->ptr; p.v = v->ptr; p.o = o->ptr;
  p.L = L; p.M = M;
  p.B = B; p.H = H; p.Lq = Lq; p.Lk = Lk;
  p.n_prefix = n_prefix;
  p.n_qtiles = (Lq + 127) / 128;
  p.qs_b = q->stride_b; p.qs_h = q->stride_h; p.qs_r = q->stride_row;
  p.ks_b = k->stride_b; p.ks_h = k->stride_h; p.ks_r = k->stride_row;
  p.vs_b = v->stride_b; p.vs_h = v->stride_h; p.vs_r = v->stride_row;
  p.os_b = o->stride_b; p.os_h = o->stride_h; p.os_r = o->stride_row;
  p.scale_log2 = sm_scale * 1.4426950408889634f;
  if (params_out != nullptr) {                             // the caller launches (beside something else)
    *params_out = p;
    return LMK_OK;
  }
  return lmk::launch_fwd(p, D, block, dtype, (hipStream_t)stream);
}

int lmk_attn_fwd(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                 float* L, float* M, int B, int H, int Lq, int Lk, int D, float sm_scale, int block,
                 int n_prefix, int dtype, void* stream) {
  return attn_fwd_impl(q, k, v, o, L, M, B, H, Lq, Lk, D, sm_scale, block, block, n_prefix, dtype, stream);
}

int lmk_attn_fwd_padded(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                        float* L, float* M, int B, int H, int Lq, int Lk, int D, float sm_scale, int block,
                        int block_real, int n_prefix, int dtype, void* stream) {
  return attn_fwd_impl(q, k, v, o, L, M, B, H, Lq, Lk, D, sm_scale, block, block_real, n_prefix, dtype, stream);
}

int lmk_attn_fwd_rotary_q(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                          float* L, float* M, const void* cos_table, const void* sin_table, int64_t table_stride_row,
                          int64_t n_pos, const int64_t* position_ids, int64_t pos_stride_b, int B, int H, int Lq, int Lk,
                          int D, float sm_scale, int block, int n_prefix, int dtype, void* stream) {
  const RopeArgs rope = {cos_table, sin_table, table_stride_row, n_pos, position_ids, pos_stride_b};
  return attn_fwd_impl(q, k, v, o, L, M, B, H, Lq, Lk, D, sm_scale, block, block, n_prefix, dtype, stream, &rope);
}

int64_t lmk_padded_rows(int64_t rows, int block_real, int block) {
  if (rows < 0 || block_real < 2 || block < block_real) return -1;
  return rows / block_real * block + rows % block_real;
}

static int pad_impl(const lmk_tensor4* src, const lmk_tensor4* dst, int B, int H, int64_t rows, int D, int block_real,
                    int block, bool unpad, void* stream) {
  int rc;
  if ((rc = check_tensor(src)) || (rc = check_tensor(dst))) return rc;
  if (B <= 0 || H <= 0 || rows <= 0 || block_real < 2 || block < block_real) return LMK_ERR_SHAPE;
  if (!(D == 64 || D == 128)) return LMK_ERR_UNSUPPORTED;
  const int64_t rows_padded = lmk_padded_rows(rows, block_real, block);
  if (rows_padded >= ((int64_t)1 << 31)) return LMK_ERR_UNSUPPORTED;
  lmk::PadParams p;
  p.src = src->ptr; p.dst = dst->ptr;
  p.B = B; p.H = H; p.n_real = block_real; p.block = block;
  p.L_src = (int)(unpad ? rows_padded : rows);
  p.L_dst = (int)(unpad ? rows : rows_padded);
  p.ss_b = src->stride_b; p.ss_h = src->stride_h; p.ss_r = src->stride_row;
  p.ds_b = dst->stride_b; p.ds_h = dst->stride_h; p.ds_r = dst->stride_row;
  return lmk::launch_pad_blocks(p, D, unpad, (hipStream_t)stream);
}

int lmk_pad_blocks(const lmk_tensor4* src, const lmk_tensor4* dst, int B, int H, int64_t rows, int D, int block_real,
                   int block, void* stream) {
  return pad_impl(src, dst, B, H, rows, D, block_real, block, false, stream);
}

int lmk_unpad_blocks(const lmk_tensor4* src, const lmk_tensor4* dst, int B, int H, int64_t rows, int D, int block_real,
                     int block, void* stream) {
  return pad_impl(src, dst, B, H, rows, D, block_real, block, true, stream);
}

size_t lmk_attn_bwd_workspace_bytes(int B, int H, int Lq, int Lk, int block) {
  if (B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0 || block <= 0) return 0;
  const size_t rows = (size_t)B * H * Lq;
  const size_t nb = (size_t)(Lk / block);
  return sizeof(float) * (2 * rows + 3 * rows * nb);
}

// hand-over layout: delta, mhat (rows floats each), the `a` plane (rows * nb floats), then the dS tiles at the
// next multiple of 2 KB
static size_t handover_tiles_offset(size_t rows, size_t nb) {
  const size_t head = sizeof(float) * (2 * rows + rows * nb);
  return (head + 2047) & ~(size_t)2047;
}

size_t lmk_attn_bwd_handover_workspace_bytes(int B, int H, int Lq, int Lk, int block) {
  if (B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0 || block != 32 || Lq % 32 != 0 || Lk % 32 != 0 || Lk < Lq) return 0;
  const size_t rows = (size_t)B * H * Lq;
  const size_t nb = (size_t)(Lk / 32);
  const size_t tiles = (size_t)lmk::handover_tiles_per_head(Lq / 32, (Lk - Lq) / 32);
  return handover_tiles_offset(rows, nb) + (size_t)B * H * tiles * 2048;
}

int lmk_attn_bwd(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                 const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                 const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes, int B, int H,
                 int Lq, int Lk, int D, float sm_scale, int block, int n_prefix, int dtype, void* stream) {
  return lmk_attn_bwd_phases(q, k, v, o, dout, L, M, dq, dk, dv, workspace, workspace_bytes, B, H, Lq, Lk, D,
                             sm_scale, block, n_prefix, dtype, LMK_BWD_ALL, stream);
}

static int attn_bwd_impl(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                         const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                         const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes, int B,
                         int H, int Lq, int Lk, int D, float sm_scale, int block, int block_real, int n_prefix,
                         int dtype, int phases, void* stream, int Lq_real = 0, int Lk_real = 0,
                         const float* group_scale = nullptr, const SegArgs* segs = nullptr);

int lmk_attn_bwd_phases(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                        const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                        const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes, int B,
                        int H, int Lq, int Lk, int D, float sm_scale, int block, int n_prefix, int dtype, int phases,
                        void* stream) {
  return attn_bwd_impl(q, k, v, o, dout, L, M, dq, dk, dv, workspace, workspace_bytes, B, H, Lq, Lk, D, sm_scale,
                       block, block, n_prefix, dtype, phases, stream);
}

int lmk_attn_bwd_padded(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                        const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                        const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes, int B,
                        int H, int Lq, int Lk, int D, float sm_scale, int block, int block_real, int n_prefix,
                        int dtype, void* stream) {
  return attn_bwd_impl(q, k, v, o, dout, L, M, dq, dk, dv, workspace, workspace_bytes, B, H, Lq, Lk, D, sm_scale,
                       block, block_real, n_prefix, dtype, LMK_BWD_ALL, stream);
}

// ---- blocks of any size on tensors in token layout
static int slots_of(int block_tokens) {
  if (block_tokens == 32 || block_tokens == 64 || block_tokens == 128) return block_tokens;
  if (block_tokens < 2 || block_tokens > 128) return 0;
  return block_tokens <= 64 ? 64 : 128;
}

int lmk_attn_fwd_blocks(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                        float* L, float* M, int B, int H, int Lq, int Lk, int D, float sm_scale, int block_tokens,
                        int n_prefix, int dtype, void* stream) {
  const int slots = slots_of(block_tokens);
  if (slots == 0) return LMK_ERR_UNSUPPORTED;
  if (slots == block_tokens)
    return attn_fwd_impl(q, k, v, o, L, M, B, H, Lq, Lk, D, sm_scale, slots, slots, n_prefix, dtype, stream);
  if (Lq <= 0 || Lk < Lq || n_prefix < 0) return LMK_ERR_SHAPE;
  if ((int64_t)Lk - Lq != (int64_t)n_prefix * block_tokens) return LMK_ERR_HISTORY;
  const int64_t lq = lmk_padded_rows(Lq, block_tokens, slots), lk = (int64_t)n_prefix * slots + lq;
  if (lk >= ((int64_t)1 << 31)) return LMK_ERR_UNSUPPORTED;
  return attn_fwd_impl(q, k, v, o, L, M, B, H, (int)lq, (int)lk, D, sm_scale, slots, block_tokens, n_prefix, dtype, stream,
                       nullptr, Lq, Lk);
}

size_t lmk_attn_bwd_blocks_workspace_bytes(int B, int H, int Lq, int Lk, int block_tokens) {
  const int slots = slots_of(block_tokens);
  if (slots == 0 || Lq <= 0 || Lk <= 0) return 0;
  return lmk_attn_bwd_workspace_bytes(B, H, (int)lmk_padded_rows(Lq, block_tokens, slots),
                                      (int)lmk_padded_rows(Lk, block_tokens, slots), slots);
}

int lmk_attn_bwd_blocks(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                        const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                        const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes, int B,
                        int H, int Lq, int Lk, int D, float sm_scale, int block_tokens, int n_prefix, int dtype,
                        void* stream) {
  const int slots = slots_of(block_tokens);
  if (slots == 0) return LMK_ERR_UNSUPPORTED;
  if (slots == block_tokens)
    return attn_bwd_impl(q, k, v, o, dout, L, M, dq, dk, dv, workspace, workspace_bytes, B, H, Lq, Lk, D, sm_scale, slots,
                         slots, n_prefix, dtype, LMK_BWD_ALL, stream);
  if (Lq <= 0 || Lk < Lq || n_prefix < 0) return LMK_ERR_SHAPE;
  if (Lq % block_tokens != 0 || Lk % block_tokens != 0) return LMK_ERR_PARTIAL;
  if ((int64_t)Lk - Lq != (int64_t)n_prefix * block_tokens) return LMK_ERR_HISTORY;
  const int64_t lq = (int64_t)Lq / block_tokens * slots, lk = (int64_t)Lk / block_tokens * slots;
  if (lk >= ((int64_t)1 << 31)) return LMK_ERR_UNSUPPORTED;
  return attn_bwd_impl(q, k, v, o, dout, L, M, dq, dk, dv, workspace, workspace_bytes, B, H, (int)lq, (int)lk, D, sm_scale,
                       slots, block_tokens, n_prefix, dtype, LMK_BWD_ALL, stream, Lq, Lk);
}

// ---- group dropout: a caller-supplied factor per (query row, earlier block).  Always the slot kernels in token
// layout: blocks of up to 64 tokens in 64 slots (block 32 included: its own kernels carry no such factor), wider in 128.
static int slots_for_group_scale(int block_tokens) {
  if (block_tokens < 2 || block_tokens > 128) return 0;
  return block_tokens <= 64 ? 64 : 128;
}

// Host-side check of a table of blocks of unequal length and the geometry that follows from it: slots per block,
// rows of slots of the keys and of the queries.  `complete_only`: the backward's restriction.
struct SegGeometry {
  int slots, n_full_k;
  int64_t lq_slots, lk_slots;
};

static int check_segments(const int32_t* seg_host, const void* seg_dev, int n_blocks, int max_block_tokens, int n_prefix,
                          int Lq, int Lk, bool last_is_partial, bool complete_only, SegGeometry* g) {
  if (seg_host == nullptr || seg_dev == nullptr) return LMK_ERR_NULL;
  if (n_blocks <= 0 || n_prefix < 0 || n_prefix >= n_blocks || Lq <= 0 || Lk < Lq) return LMK_ERR_SHAPE;
  if (max_block_tokens < 2 || max_block_tokens > 128) return LMK_ERR_UNSUPPORTED;
  if (last_is_partial && complete_only) return LMK_ERR_PARTIAL;
  const int n_full = n_blocks - (last_is_partial ? 1 : 0);
  if (seg_host[0] != 0 || seg_host[n_blocks] != Lk) return LMK_ERR_SHAPE;
  for (int b = 0; b < n_blocks; ++b) {
    const int64_t len = (int64_t)seg_host[b + 1] - seg_host[b];
    // a complete block: a key and its landmark at least; the block without landmark must leave the last slot free
    if (len > max_block_tokens - (b < n_full ? 0 : 1) || len < (b < n_full ? 2 : 1)) return LMK_ERR_SHAPE;
  }
  if ((int64_t)Lk - Lq != seg_host[n_prefix]) return LMK_ERR_HISTORY;                 // the history is whole blocks
  g->slots = max_block_tokens <= 64 ? 64 : 128;
  g->n_full_k = n_full;
  g->lk_slots = (int64_t)n_full * g->slots + (last_is_partial ? seg_host[n_blocks] - seg_host[n_blocks - 1] : 0);
  g->lq_slots = g->lk_slots - (int64_t)n_prefix * g->slots;
  if (g->lk_slots >= ((int64_t)1 << 31) || g->lq_slots <= 0) return LMK_ERR_UNSUPPORTED;
  return LMK_OK;
}

int lmk_attn_fwd_segments(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                          float* L, float* M, const int32_t* seg_host, const int32_t* seg_dev, int n_blocks,
                          int max_block_tokens, int last_is_partial, int B, int H, int Lq, int Lk, int D,
                          float sm_scale, int n_prefix, int dtype, void* stream) {
  SegGeometry g;
  if (int rc = check_segments(seg_host, seg_dev, n_blocks, max_block_tokens, n_prefix, Lq, Lk, last_is_partial != 0, false, &g))
    return rc;
  const SegArgs segs = {seg_dev, g.n_full_k};
  return attn_fwd_impl(q, k, v, o, L, M, B, H, (int)g.lq_slots, (int)g.lk_slots, D, sm_scale, g.slots, g.slots, n_prefix,
                       dtype, stream, nullptr, Lq, Lk, nullptr, nullptr, &segs);
}

size_t lmk_attn_bwd_segments_workspace_bytes(int B, int H, int n_blocks, int n_prefix, int max_block_tokens) {
  if (n_blocks <= 0 || n_prefix < 0 || n_prefix >= n_blocks || max_block_tokens < 2 || max_block_tokens > 128) return 0;
  const int slots = max_block_tokens <= 64 ? 64 : 128;
  const int64_t lk = (int64_t)n_blocks * slots, lq = (int64_t)(n_blocks - n_prefix) * slots;
  if (lk >= ((int64_t)1 << 31)) return 0;
  return lmk_attn_bwd_workspace_bytes(B, H, (int)lq, (int)lk, slots);
}

int lmk_attn_bwd_segments(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                          const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                          const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes,
                          const int32_t* seg_host, const int32_t* seg_dev, int n_blocks, int max_block_tokens, int B,
                          int H, int Lq, int Lk, int D, float sm_scale, int n_prefix, int dtype, void* stream) {
  SegGeometry g;
  if (int rc = check_segments(seg_host, seg_dev, n_blocks, max_block_tokens, n_prefix, Lq, Lk, false, true, &g)) return rc;
  const SegArgs segs = {seg_dev, g.n_full_k};
  return attn_bwd_impl(q, k, v, o, dout, L, M, dq, dk, dv, workspace, workspace_bytes, B, H, (int)g.lq_slots,
                       (int)g.lk_slots, D, sm_scale, g.slots, g.slots, n_prefix, dtype, LMK_BWD_ALL, stream, Lq, Lk, nullptr,
                       &segs);
}

int lmk_attn_fwd_group_scale(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                             float* L, float* M, const float* group_scale, int B, int H, int Lq, int Lk, int D,
                             float sm_scale, int block_tokens, int n_prefix, int dtype, void* stream) {
  const int slots = slots_for_group_scale(block_tokens);
  if (slots == 0) return LMK_ERR_UNSUPPORTED;
  if (group_scale == nullptr) return LMK_ERR_NULL;
  if (Lq <= 0 || Lk < Lq || n_prefix < 0) return LMK_ERR_SHAPE;
  if ((int64_t)Lk - Lq != (int64_t)n_prefix * block_tokens) return LMK_ERR_HISTORY;
  const int64_t lq = lmk_padded_rows(Lq, block_tokens, slots), lk = (int64_t)n_prefix * slots + lq;
  if (lk >= ((int64_t)1 << 31)) return LMK_ERR_UNSUPPORTED;
  return attn_fwd_impl(q, k, v, o, L, M, B, H, (int)lq, (int)lk, D, sm_scale, slots, block_tokens, n_prefix, dtype, stream,
                       nullptr, Lq, Lk, group_scale);
}

size_t lmk_attn_bwd_group_scale_workspace_bytes(int B, int H, int Lq, int Lk, int block_tokens) {
  const int slots = slots_for_group_scale(block_tokens);
  if (slots == 0 || Lq <= 0 || Lk <= 0) return 0;
  return lmk_attn_bwd_workspace_bytes(B, H, (int)lmk_padded_rows(Lq, block_tokens, slots),
                                      (int)lmk_padded_rows(Lk, block_tokens, slots), slots);
}

int lmk_attn_bwd_group_scale(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                             const lmk_tensor4* dout, const float* L, const float* M, const float* group_scale,
                             const lmk_tensor4* dq, const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace,
                             size_t workspace_bytes, int B, int H, int Lq, int Lk, int D, float sm_scale,
                             int block_tokens, int n_prefix, int dtype, void* stream) {
  const int slots = slots_for_group_scale(block_tokens);
  if (slots == 0) return LMK_ERR_UNSUPPORTED;
  if (group_scale == nullptr) return LMK_ERR_NULL;
  if (Lq <= 0 || Lk < Lq || n_prefix < 0) return LMK_ERR_SHAPE;
  if (Lq % block_tokens != 0 || Lk % block_tokens != 0) return LMK_ERR_PARTIAL;
  if ((int64_t)Lk - Lq != (int64_t)n_prefix * block_tokens) return LMK_ERR_HISTORY;
  const int64_t lq = (int64_t)Lq / block_tokens * slots, lk = (int64_t)Lk / block_tokens * slots;
  if (lk >= ((int64_t)1 << 31)) return LMK_ERR_UNSUPPORTED;
  return attn_bwd_impl(q, k, v, o, dout, L, M, dq, dk, dv, workspace, workspace_bytes, B, H, (int)lq, (int)lk, D, sm_scale,
                       slots, block_tokens, n_prefix, dtype, LMK_BWD_ALL, stream, Lq, Lk, group_scale);
}

static int attn_bwd_impl(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                         const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                         const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes, int B,
                         int H, int Lq, int Lk, int D, float sm_scale, int block, int block_real, int n_prefix,
                         int dtype, int phases, void* stream, int Lq_real, int Lk_real, const float* group_scale,
                         const SegArgs* segs) {
  int rc;
  if (phases <= 0 || phases > LMK_BWD_ALL) return LMK_ERR_SHAPE;
  if ((rc = check_tensor(q)) || (rc = check_tensor(k)) || (rc = check_tensor(v)) || (rc = check_tensor(o)) ||
      (rc = check_tensor(dout)) || (rc = check_tensor(dq)) || (rc = check_tensor(dk)) || (rc = check_tensor(dv)))
    return rc;
  if (L == nullptr || M == nullptr || workspace == nullptr) return LMK_ERR_NULL;
  if ((rc = check_common(B, H, Lq, Lk, D, sm_scale, block, n_prefix, dtype))) return rc;
  if ((rc = check_block_real(block, block_real))) return rc;
  if (Lq % block != 0 || Lk % block != 0) return LMK_ERR_PARTIAL;
  if (!slice_fits_32bit(q, Lq) || !slice_fits_32bit(o, Lq) || !slice_fits_32bit(dout, Lq) || !slice_fits_32bit(dq, Lq) ||
      !slice_fits_32bit(k, Lk) || !slice_fits_32bit(v, Lk) || !slice_fits_32bit(dk, Lk) || !slice_fits_32bit(dv, Lk))
    return LMK_ERR_UNSUPPORTED;
  if (!aligned16(workspace)) return LMK_ERR_ALIGN;
  if (workspace_bytes < lmk_attn_bwd_workspace_bytes(B, H, Lq, Lk, block)) return LMK_ERR_WORKSPACE;
  lmk::BwdParams p;
  p.q = q->ptr; p.k = k->ptr; p.v = v->ptr; p.o = o->ptr; p.dout = dout->ptr;
  p.dq = dq->ptr; p.dk = dk->ptr; p.dv = dv->ptr;
  p.L = L; p.M = M;
  const size_t rows = (size_t)B * H * Lq;
  const size_t nb = (size_t)(Lk / block);
  float* w = static_cast<float*>(workspace);
  p.delta = w;
  p.mhat = w + rows;
  p.stat_a = w + 2 * rows;
  p.stat_n = w + 2 * rows + rows * nb;
  p.stat_l = w + 2 * rows + 2 * rows * nb;
  // a workspace large enough for the dS tiles selects the hand-over backward (block 32, unpadded)
  const size_t ho_bytes = (block_real == block) ? lmk_attn_bwd_handover_workspace_bytes(B, H, Lq, Lk, block) : 0;
  p.ds_tiles = nullptr;
  if (ho_bytes != 0 && workspace_bytes >= ho_bytes) {
    p.ds_tiles = static_cast<char*>(workspace) + handover_tiles_offset(rows, nb);
    p.stat_n = p.stat_l = nullptr;
  }
  p.B = B; p.H = H; p.Lq = Lq; p.Lk = Lk;
  p.n_prefix = n_prefix; p.n_blocks = (int)nb;
  p.n_real = block_real;
  p.Lq_real = Lq_real; p.Lk_real = Lk_real;
  p.seg = nullptr; p.n_full_q = p.n_full_k = 0;
  if (segs != nullptr) {
    if (Lq_real <= 0 || group_scale != nullptr) return LMK_ERR_UNSUPPORTED;
    p.seg = segs->seg_dev;
    p.n_full_k = segs->n_full_k;
    p.n_full_q = segs->n_full_k - n_prefix;
  } else if (Lq_real > 0) {
    p.n_full_q = Lq_real / block_real;
    p.n_full_k = Lk_real / block_real;
  }
  p.group_scale = nullptr; p.gs_bh = p.gs_blk = 0;
  if (group_scale != nullptr) {
    if (Lq_real <= 0) return LMK_ERR_UNSUPPORTED;
    p.group_scale = group_scale;
    p.gs_blk = Lq_real;
    p.gs_bh = (int64_t)(Lk_real / block_real) * Lq_real;
  }
  p.n_qtiles = (Lq + 127) / 128; p.n_kvtiles = (Lk + 127) / 128;
  p.qs_b = q->stride_b; p.qs_h = q->stride_h; p.qs_r = q->stride_row;
  p.ks_b = k->stride_b; p.ks_h = k->stride_h; p.ks_r = k->stride_row;
  p.vs_b = v->stride_b; p.vs_h = v->stride_h; p.vs_r = v->stride_row;
  p.os_b = o->stride_b; p.os_h = o->stride_h; p.os_r = o->stride_row;
  p.dos_b = dout->stride_b; p.dos_h = dout->stride_h; p.dos_r = dout->stride_row;
  p.dqs_b = dq->stride_b; p.dqs_h = dq->stride_h; p.dqs_r = dq->stride_row;
  p.dks_b = dk->stride_b; p.dks_h = dk->stride_h; p.dks_r = dk->stride_row;
  p.dvs_b = dv->stride_b; p.dvs_h = dv->stride_h; p.dvs_r = dv->stride_row;
  p.scale = sm_scale;
  p.scale_log2 = sm_scale * 1.4426950408889634f;
  return lmk::launch_bwd(p, D, block, dtype, phases, (hipStream_t)stream);
}

size_t lmk_retrieve_workspace_bytes(int B, int H, int T, int S, int D, int block) {
  if (B <= 0 || H <= 0 || T <= 0 || S <= 0 || D <= 0 || block <= 0) return 0;
  return retr_layout(B, H, T, S, D, block).total;
}

// The host-side checks of the selection, everything but the workspace.
static int retrieve_topk_check(const lmk_tensor4* q, const lmk_tensor4* kcache, const void* cos_table,
                               const void* sin_table, int64_t table_stride_row, int64_t n_pos, const int64_t* idx_out,
                               int B, int H, int T, int S, int D, int block, int top_k, int dtype) {
  int rc;
  if ((rc = check_tensor(q)) || (rc = check_tensor(kcache))) return rc;
  if (cos_table == nullptr || sin_table == nullptr || idx_out == nullptr) return LMK_ERR_NULL;
  if (!aligned16(cos_table) || !aligned16(sin_table) || !stride_ok(table_stride_row)) return LMK_ERR_ALIGN;
  return check_retrieval(B, H, T, S, D, block, top_k, dtype, n_pos);
}

static int retrieve_topk_impl(bool reuse_landmark_keys, const lmk_tensor4* q, const lmk_tensor4* kcache,
                              const void* cos_table, const void* sin_table, int64_t table_stride_row, int64_t n_pos,
                              int64_t* idx_out, void* workspace, size_t workspace_bytes, int B, int H, int T, int S,
                              int D, int block, int top_k, int dtype, void* stream,
                              lmk::RetrParams* params_out = nullptr) {
  if (int rc = retrieve_topk_check(q, kcache, cos_table, sin_table, table_stride_row, n_pos, idx_out, B, H, T, S, D,
                                   block, top_k, dtype))
    return rc;
  if (workspace == nullptr) return LMK_ERR_NULL;
  if (!aligned16(workspace)) return LMK_ERR_ALIGN;
  const RetrLayout l = retr_layout(B, H, T, S, D, block);
  if (workspace_bytes < l.total) return LMK_ERR_WORKSPACE;
  lmk::RetrParams p = {};
  fill_retr_common(p, B, H, T, S, D, block, top_k);
  p.q = q->ptr; p.kcache = kcache->ptr; p.cos = cos_table; p.sin = sin_table; p.idx = idx_out;
  char* w = static_cast<char*>(workspace);
  p.lk_rot = w + l.lk_rot;
  p.lk_norm = reinterpret_cast<float*>(w + l.lk_norm);
  p.approx = reinterpret_cast<float*>(w + l.approx);
  p.exact = reinterpret_cast<float*>(w + l.exact);
  p.qs_b = q->stride_b; p.qs_h = q->stride_h; p.qs_r = q->stride_row;
  p.kcs_b = kcache->stride_b; p.kcs_h = kcache->stride_h; p.kcs_r = kcache->stride_row;
  p.cs_r = table_stride_row;
  if (params_out != nullptr) {                             // the caller launches
    *params_out = p;
    return LMK_OK;
  }
  return lmk::launch_retrieve_topk(p, D, dtype, reuse_landmark_keys, (hipStream_t)stream);
}

int lmk_retrieve_topk(const lmk_tensor4* q, const lmk_tensor4* kcache, const void* cos_table, const void* sin_table,
                      int64_t table_stride_row, int64_t n_pos, int64_t* idx_out, void* workspace,
                      size_t workspace_bytes, int B, int H, int T, int S, int D, int block, int top_k, int dtype,
                      void* stream) {
  return retrieve_topk_impl(false, q, kcache, cos_table, sin_table, table_stride_row, n_pos, idx_out, workspace,
                            workspace_bytes, B, H, T, S, D, block, top_k, dtype, stream);
}

int lmk_retrieve_topk_reuse(const lmk_tensor4* q, const lmk_tensor4* kcache, const void* cos_table,
                            const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                            void* workspace, size_t workspace_bytes, int B, int H, int T, int S, int D, int block,
                            int top_k, int dtype, void* stream) {
  return retrieve_topk_impl(true, q, kcache, cos_table, sin_table, table_stride_row, n_pos, idx_out, workspace,
                            workspace_bytes, B, H, T, S, D, block, top_k, dtype, stream);
}

size_t lmk_retrieve_static_max_bytes(void) { return LMK_STATIC_SCRATCH_BYTES; }

int lmk_retrieve_static_init(void) {
  int rc = 0;
  return static_scratch(&rc) != nullptr ? LMK_OK : rc;
}

int lmk_retrieve_topk_static(const lmk_tensor4* q, const lmk_tensor4* kcache, const void* cos_table,
                             const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out, int B,
                             int H, int T, int S, int D, int block, int top_k, int dtype, void* stream) {
  // every argument check runs on the host first, the size limit of the array among them
  int rc = retrieve_topk_check(q, kcache, cos_table, sin_table, table_stride_row, n_pos, idx_out, B, H, T, S, D, block,
                               top_k, dtype);
  if (rc) return rc;
  if (retr_layout(B, H, T, S, D, block).total > LMK_STATIC_SCRATCH_BYTES) return LMK_ERR_WORKSPACE;
  void* ptr = static_scratch(&rc);
  if (ptr == nullptr) return rc;
  // same kernels, same layout: the device address of the array takes the place of the caller's workspace
  return retrieve_topk_impl(false, q, kcache, cos_table, sin_table, table_stride_row, n_pos, idx_out, ptr,
                            LMK_STATIC_SCRATCH_BYTES, B, H, T, S, D, block, top_k, dtype, stream);
}

// `candidates`: the selection has stopped after its slice step (lmk::launch_fwd32_topk_slices) and the gather picks
// a row's k best from what that step left, writing them to idx on the way; else idx holds the indices already.
static int gather_attend_impl(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache, const int64_t* idx,
                              const void* cos_table, const void* sin_table, int64_t table_stride_row, int64_t n_pos,
                              const lmk_tensor4* o_loc, const float* L_loc, const float* M_loc, int64_t stat_stride,
                              const lmk_tensor4* out, int B, int H, int T, int S, int D, float sm_scale, int block,
                              int top_k, int dtype, void* stream, const lmk::RetrParams* candidates,
                              const lmk_tensor4* k_new = nullptr, const lmk_tensor4* v_new = nullptr) {
  // k_new, v_new: the gather kernel attends to the rows' local window itself (gather_takes_local_window) and
  // o_loc, L_loc, M_loc are not read
  const bool local = k_new != nullptr;
  int rc;
  if ((rc = check_tensor(q)) || (rc = check_tensor(kcache)) || (rc = check_tensor(vcache)) || (rc = check_tensor(out)))
    return rc;
  if (local ? ((rc = check_tensor(k_new)) || (rc = check_tensor(v_new))) : (rc = check_tensor(o_loc))) return rc;
  if (cos_table == nullptr || sin_table == nullptr || idx == nullptr || (!local && (L_loc == nullptr || M_loc == nullptr)))
    return LMK_ERR_NULL;
  if (!aligned16(cos_table) || !aligned16(sin_table) || !stride_ok(table_stride_row)) return LMK_ERR_ALIGN;
  if ((rc = check_retrieval(B, H, T, S, D, block, top_k, dtype, n_pos))) return rc;
  if (!(block == 32 || block == 64 || block == 128)) return LMK_ERR_UNSUPPORTED;
  if (!local && stat_stride < T) return LMK_ERR_SHAPE;
  if (local && !lmk::gather_takes_local_window(T, S, block)) return LMK_ERR_UNSUPPORTED;
  if (!std::isfinite(sm_scale) || !(sm_scale > 0.f)) return LMK_ERR_SCALE;
  lmk::RetrParams p = {};
  fill_retr_common(p, B, H, T, S, D, block, top_k);
  p.q = q->ptr; p.kcache = kcache->ptr; p.vcache = vcache->ptr; p.cos = cos_table; p.sin = sin_table;
  p.idx = const_cast<int64_t*>(idx);
  p.idx_st = p.k; p.idx_sh = (int64_t)T * p.k; p.idx_sb = (int64_t)H * T * p.k;
  p.out = out->ptr;
  if (local) {
    p.local = 1;
    p.local_inc = S % block;
    p.local_row0 = S - S % block;                               // the cache's rows are its positions (llama_mem.py:336-338)
    p.local_pos0 = p.local_row0;
    p.k_new = k_new->ptr; p.kns_b = k_new->stride_b; p.kns_h = k_new->stride_h; p.kns_r = k_new->stride_row;
    p.v_new = v_new->ptr; p.vns_b = v_new->stride_b; p.vns_h = v_new->stride_h; p.vns_r = v_new->stride_row;
  } else {
    p.o_loc = o_loc->ptr; p.L_loc = L_loc; p.M_loc = M_loc; p.stat_stride = stat_stride;
    p.ols_b = o_loc->stride_b; p.ols_h = o_loc->stride_h; p.ols_r = o_loc->stride_row;
  }
  p.qs_b = q->stride_b; p.qs_h = q->stride_h; p.qs_r = q->stride_row;
  p.kcs_b = kcache->stride_b; p.kcs_h = kcache->stride_h; p.kcs_r = kcache->stride_row;
  p.vcs_b = vcache->stride_b; p.vcs_h = vcache->stride_h; p.vcs_r = vcache->stride_row;
  p.outs_b = out->stride_b; p.outs_h = out->stride_h; p.outs_r = out->stride_row;
  p.cs_r = table_stride_row;
  p.scale_log2 = sm_scale * 1.4426950408889634f;
  if (candidates != nullptr) {
    p.merge_slices = lmk::topk_slices(*candidates);
    p.approx = candidates->approx;
    p.exact = candidates->exact;
  }
  return lmk::launch_gather_attend(p, D, block, dtype, (hipStream_t)stream);
}

int lmk_gather_attend(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache, const int64_t* idx,
                      const void* cos_table, const void* sin_table, int64_t table_stride_row, int64_t n_pos,
                      const lmk_tensor4* o_loc, const float* L_loc, const float* M_loc, int64_t stat_stride,
                      const lmk_tensor4* out, int B, int H, int T, int S, int D, float sm_scale, int block, int top_k,
                      int dtype, void* stream) {
  return gather_attend_impl(q, kcache, vcache, idx, cos_table, sin_table, table_stride_row, n_pos, o_loc, L_loc, M_loc,
                            stat_stride, out, B, H, T, S, D, sm_scale, block, top_k, dtype, stream, nullptr);
}

static int retrieve_topk_shared_impl(const lmk_tensor4* q, const lmk_tensor4* kcache, const void* cos_table,
                                     const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                                     void* block_prob_out, void* workspace, size_t workspace_bytes, int B, int H, int T,
                                     int S, int D, int block, int top_k, int dtype, void* stream, bool lm_dense);

int lmk_retrieve_topk_shared(const lmk_tensor4* q, const lmk_tensor4* kcache, const void* cos_table,
                             const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                             void* block_prob_out, void* workspace, size_t workspace_bytes, int B, int H, int T, int S,
                             int D, int block, int top_k, int dtype, void* stream) {
  return retrieve_topk_shared_impl(q, kcache, cos_table, sin_table, table_stride_row, n_pos, idx_out, block_prob_out,
                                   workspace, workspace_bytes, B, H, T, S, D, block, top_k, dtype, stream, false);
}

int lmk_retrieve_topk_shared_landmarks(const lmk_tensor4* q, const lmk_tensor4* landmark_keys, const void* cos_table,
                                       const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                                       void* block_prob_out, void* workspace, size_t workspace_bytes, int B, int H, int T,
                                       int n_blocks, int D, int block, int top_k, int dtype, void* stream) {
  if (n_blocks <= 0) return LMK_ERR_CACHE;
  if (block < 2 || (int64_t)n_blocks * block >= ((int64_t)1 << 31)) return LMK_ERR_UNSUPPORTED;
  return retrieve_topk_shared_impl(q, landmark_keys, cos_table, sin_table, table_stride_row, n_pos, idx_out,
                                   block_prob_out, workspace, workspace_bytes, B, H, T, n_blocks * block, D, block, top_k,
                                   dtype, stream, true);
}

static int retrieve_topk_shared_impl(const lmk_tensor4* q, const lmk_tensor4* kcache, const void* cos_table,
                                     const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                                     void* block_prob_out, void* workspace, size_t workspace_bytes, int B, int H, int T,
                                     int S, int D, int block, int top_k, int dtype, void* stream, bool lm_dense) {
  int rc;
  if ((rc = check_tensor(q)) || (rc = check_tensor(kcache))) return rc;
  if (cos_table == nullptr || sin_table == nullptr || idx_out == nullptr || workspace == nullptr) return LMK_ERR_NULL;
  if (!aligned16(cos_table) || !aligned16(sin_table) || !stride_ok(table_stride_row) || !aligned16(workspace))
    return LMK_ERR_ALIGN;
  if ((rc = check_retrieval(B, H, T, S, D, block, top_k, dtype, n_pos))) return rc;
  const RetrLayout l = retr_layout(B, H, T, S, D, block);
  if (workspace_bytes < l.total) return LMK_ERR_WORKSPACE;
  lmk::RetrParams p = {};
  fill_retr_common(p, B, H, T, S, D, block, top_k);
  p.q = q->ptr; p.kcache = kcache->ptr; p.cos = cos_table; p.sin = sin_table; p.idx = idx_out;
  char* w = static_cast<char*>(workspace);
  p.lk_rot = w + l.lk_rot;
  p.lk_norm = reinterpret_cast<float*>(w + l.lk_norm);
  p.approx = reinterpret_cast<float*>(w + l.approx);              // every query's scores, then exponentials
  p.agg = reinterpret_cast<uint32_t*>(w + l.exact);               // B*H*num_mems words: fits, T >= 1
  p.agg_out = static_cast<uint16_t*>(block_prob_out);
  p.lm_dense = lm_dense ? 1 : 0;
  p.qs_b = q->stride_b; p.qs_h = q->stride_h; p.qs_r = q->stride_row;
  p.kcs_b = kcache->stride_b; p.kcs_h = kcache->stride_h; p.kcs_r = kcache->stride_row;
  p.cs_r = table_stride_row;
  return lmk::launch_retrieve_topk_shared(p, D, dtype, (hipStream_t)stream);
}

int lmk_ring_retrieve_topk(const lmk_tensor4* q, const lmk_tensor4* kring, const void* cos_table,
                           const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                           void* workspace, size_t workspace_bytes, int B, int H, int T, int n_blocks, int D, int block,
                           int top_k, int ring_start, int method, int dtype, void* stream) {
  int rc;
  if ((rc = check_tensor(q)) || (rc = check_tensor(kring))) return rc;
  if (cos_table == nullptr || sin_table == nullptr || idx_out == nullptr || workspace == nullptr) return LMK_ERR_NULL;
  if (!aligned16(cos_table) || !aligned16(sin_table) || !stride_ok(table_stride_row) || !aligned16(workspace))
    return LMK_ERR_ALIGN;
  if (B <= 0 || H <= 0 || T <= 0) return LMK_ERR_SHAPE;
  if (n_blocks <= 0) return LMK_ERR_CACHE;
  if (!(D == 64 || D == 128)) return LMK_ERR_UNSUPPORTED;
  if (block < 2 || block > 4096 || (int64_t)n_blocks * block >= ((int64_t)1 << 31)) return LMK_ERR_UNSUPPORTED;
  if (!(dtype == LMK_DTYPE_BF16 || dtype == LMK_DTYPE_F16)) return LMK_ERR_UNSUPPORTED;
  if (method < LMK_SELECT_PER_TOKEN_AND_HEAD || method > LMK_SELECT_MAX_OVER_TOKENS) return LMK_ERR_UNSUPPORTED;
  if (top_k < 1 || top_k > 64 || top_k > n_blocks) return LMK_ERR_TOPK;      // torch.topk raises for k > n (mem_cache.py:72)
  if (ring_start < 0 || ring_start >= n_blocks) return LMK_ERR_SHAPE;
  if (n_pos < (int64_t)(top_k + 1) * block) return LMK_ERR_TABLE;            // landmark positions end at top_k*block + block-1
  const int S = n_blocks * block;
  const RetrLayout l = retr_layout(B, H, T, S, D, block);
  if (workspace_bytes < l.total) return LMK_ERR_WORKSPACE;
  lmk::RetrParams p = {};
  fill_retr_common(p, B, H, T, S, D, block, top_k);
  p.prefix_len = 0;                                                          // mem_cache.py:60: slot * block + block - 1
  p.ring_start = ring_start;
  p.q = q->ptr; p.kcache = kring->ptr; p.cos = cos_table; p.sin = sin_table; p.idx = idx_out;
  char* w = static_cast<char*>(workspace);
  p.lk_rot = w + l.lk_rot;
  p.lk_norm = reinterpret_cast<float*>(w + l.lk_norm);
  p.approx = reinterpret_cast<float*>(w + l.approx);
  p.exact = reinterpret_cast<float*>(w + l.exact);
  p.qs_b = q->stride_b; p.qs_h = q->stride_h; p.qs_r = q->stride_row;
  p.kcs_b = kring->stride_b; p.kcs_h = kring->stride_h; p.kcs_r = kring->stride_row;
  p.cs_r = table_stride_row;
  if (method == LMK_SELECT_PER_TOKEN_AND_HEAD) return lmk::launch_retrieve_topk(p, D, dtype, false, (hipStream_t)stream);
  p.agg = reinterpret_cast<uint32_t*>(w + l.exact);                          // B*T or B*H vectors of n_blocks words: fits
  p.agg_over_heads = method == LMK_SELECT_MAX_OVER_HEADS;
  p.prob32 = 1;                                                              // softmax output stays fp32 under autocast
  return lmk::launch_retrieve_topk_shared(p, D, dtype, (hipStream_t)stream);
}

int lmk_ring_gather_attend(const lmk_tensor4* q, const lmk_tensor4* kring, const lmk_tensor4* vring, const int64_t* idx,
                           const void* cos_table, const void* sin_table, int64_t table_stride_row, int64_t n_pos,
                           const lmk_tensor4* o_loc, const float* L_loc, const float* M_loc, int64_t stat_stride,
                           const lmk_tensor4* out, int B, int H, int T, int n_blocks, int D, float sm_scale, int block,
                           int top_k, int ring_start, int method, int dtype, void* stream) {
  int rc;
  if ((rc = check_tensor(q)) || (rc = check_tensor(kring)) || (rc = check_tensor(vring)) || (rc = check_tensor(o_loc)) ||
      (rc = check_tensor(out)))
    return rc;
  if (cos_table == nullptr || sin_table == nullptr || idx == nullptr || L_loc == nullptr || M_loc == nullptr)
    return LMK_ERR_NULL;
  if (!aligned16(cos_table) || !aligned16(sin_table) || !stride_ok(table_stride_row)) return LMK_ERR_ALIGN;
  if (B <= 0 || H <= 0 || T <= 0 || stat_stride < T) return LMK_ERR_SHAPE;
  if (n_blocks <= 0) return LMK_ERR_CACHE;
  if (!(D == 64 || D == 128)) return LMK_ERR_UNSUPPORTED;
  if (block < 2 || block > 128) return LMK_ERR_UNSUPPORTED;
  if (!(dtype == LMK_DTYPE_BF16 || dtype == LMK_DTYPE_F16)) return LMK_ERR_UNSUPPORTED;
  if (method < LMK_SELECT_PER_TOKEN_AND_HEAD || method > LMK_SELECT_MAX_OVER_TOKENS) return LMK_ERR_UNSUPPORTED;
  if (top_k < 1 || top_k > 64 || top_k > n_blocks) return LMK_ERR_TOPK;
  if (ring_start < 0 || ring_start >= n_blocks) return LMK_ERR_SHAPE;
  if (n_pos < (int64_t)(top_k + 1) * block) return LMK_ERR_TABLE;            // key positions end at (top_k + 1) * block - 1
  if (!std::isfinite(sm_scale) || !(sm_scale > 0.f)) return LMK_ERR_SCALE;
  lmk::RetrParams p = {};
  fill_retr_common(p, B, H, T, n_blocks * block, D, block, top_k);
  p.prefix_len = 0;                                                          // mem_cache.py:95-97: k_indices start at 0
  p.ring_start = ring_start;
  p.q = q->ptr; p.kcache = kring->ptr; p.vcache = vring->ptr; p.cos = cos_table; p.sin = sin_table;
  p.idx = const_cast<int64_t*>(idx);
  const int64_t k = p.k;
  if (method == LMK_SELECT_PER_TOKEN_AND_HEAD) { p.idx_st = k; p.idx_sh = T * k; p.idx_sb = (int64_t)H * T * k; }
  else if (method == LMK_SELECT_MAX_OVER_HEADS) { p.idx_st = k; p.idx_sh = 0; p.idx_sb = T * k; }
  else { p.idx_st = 0; p.idx_sh = k; p.idx_sb = H * k; }
  p.o_loc = o_loc->ptr; p.L_loc = L_loc; p.M_loc = M_loc; p.stat_stride = stat_stride; p.out = out->ptr;
  p.qs_b = q->stride_b; p.qs_h = q->stride_h; p.qs_r = q->stride_row;
  p.kcs_b = kring->stride_b; p.kcs_h = kring->stride_h; p.kcs_r = kring->stride_row;
  p.vcs_b = vring->stride_b; p.vcs_h = vring->stride_h; p.vcs_r = vring->stride_row;
  p.ols_b = o_loc->stride_b; p.ols_h = o_loc->stride_h; p.ols_r = o_loc->stride_row;
  p.outs_b = out->stride_b; p.outs_h = out->stride_h; p.outs_r = out->stride_row;
  p.cs_r = table_stride_row;
  p.scale_log2 = sm_scale * 1.4426950408889634f;
  const int slots = block == 32 ? 32 : (block <= 64 ? 64 : 128);
  return lmk::launch_gather_attend(p, D, slots, dtype, (hipStream_t)stream);
}

int lmk_local_window(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache,
                     const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table, const void* sin_table,
                     int64_t table_stride_row, int64_t n_pos, const lmk_tensor4* q_win, const lmk_tensor4* k_win,
                     const lmk_tensor4* v_win, int B, int H, int T, int S, int D, int block, int dtype, void* stream) {
  if (q_win == nullptr) return LMK_ERR_NULL;
  return window_impl(q, kcache, vcache, nullptr, k_loc, v_loc, cos_table, sin_table, table_stride_row, n_pos, q_win,
                     k_win, v_win, B, H, T, S, D, block, 1, dtype, stream);
}

int lmk_ring_local_window(const lmk_tensor4* q, const lmk_tensor4* k_tail, const lmk_tensor4* v_tail,
                          const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table,
                          const void* sin_table, int64_t table_stride_row, int64_t n_pos, const lmk_tensor4* q_win,
                          const lmk_tensor4* k_win, const lmk_tensor4* v_win, int B, int H, int T, int tail,
                          int64_t tail_position, int D, int dtype, void* stream) {
  int rc;
  if ((rc = check_tensor(q)) || (rc = check_tensor(k_tail)) || (rc = check_tensor(v_tail)) ||
      (rc = check_tensor(k_loc)) || (rc = check_tensor(v_loc)) || (rc = check_tensor(q_win)) ||
      (rc = check_tensor(k_win)) || (rc = check_tensor(v_win)))
    return rc;
  if (cos_table == nullptr || sin_table == nullptr) return LMK_ERR_NULL;
  if (!aligned16(cos_table) || !aligned16(sin_table) || !stride_ok(table_stride_row)) return LMK_ERR_ALIGN;
  if (B <= 0 || H <= 0 || T <= 0 || tail <= 0) return LMK_ERR_SHAPE;
  if (!(D == 64 || D == 128)) return LMK_ERR_UNSUPPORTED;
  if (!(dtype == LMK_DTYPE_BF16 || dtype == LMK_DTYPE_F16)) return LMK_ERR_UNSUPPORTED;
  if (tail_position < 0 || tail_position + tail > n_pos) return LMK_ERR_TABLE;
  lmk::WindowParams p = {};
  p.q = q->ptr; p.kcache = k_tail->ptr; p.vcache = v_tail->ptr; p.k_loc = k_loc->ptr; p.v_loc = v_loc->ptr;
  p.cos = cos_table; p.sin = sin_table;
  p.q_win = q_win->ptr; p.k_win = k_win->ptr; p.v_win = v_win->ptr;
  p.B = B; p.H = H; p.T = T; p.inc = tail;
  p.full_len = 0;                                          // the tail's rows are rows 0 .. tail-1 of k_tail, v_tail
  p.tail_pos = tail_position;
  p.block = 1; p.num_mems = 0;
  p.qs_b = q->stride_b; p.qs_h = q->stride_h; p.qs_r = q->stride_row;
  p.kcs_b = k_tail->stride_b; p.kcs_h = k_tail->stride_h; p.kcs_r = k_tail->stride_row;
  p.vcs_b = v_tail->stride_b; p.vcs_h = v_tail->stride_h; p.vcs_r = v_tail->stride_row;
  p.kls_b = k_loc->stride_b; p.kls_h = k_loc->stride_h; p.kls_r = k_loc->stride_row;
  p.vls_b = v_loc->stride_b; p.vls_h = v_loc->stride_h; p.vls_r = v_loc->stride_row;
  p.qws_b = q_win->stride_b; p.qws_h = q_win->stride_h; p.qws_r = q_win->stride_row;
  p.kws_b = k_win->stride_b; p.kws_h = k_win->stride_h; p.kws_r = k_win->stride_row;
  p.vws_b = v_win->stride_b; p.vws_h = v_win->stride_h; p.vws_r = v_win->stride_row;
  p.cs_r = table_stride_row;
  return lmk::launch_local_window(p, D, dtype, (hipStream_t)stream);
}

int lmk_gather_window(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache, const int64_t* idx,
                      const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table, const void* sin_table,
                      int64_t table_stride_row, int64_t n_pos, const lmk_tensor4* q_win, const lmk_tensor4* k_win,
                      const lmk_tensor4* v_win, int B, int H, int T, int S, int D, int block, int top_k, int dtype,
                      void* stream) {
  if (idx == nullptr) return LMK_ERR_NULL;
  return window_impl(q, kcache, vcache, idx, k_loc, v_loc, cos_table, sin_table, table_stride_row, n_pos, q_win,
                     k_win, v_win, B, H, T, S, D, block, top_k, dtype, stream);
}

int lmk_apply_rotary(const lmk_tensor4* x, const lmk_tensor4* out, const void* cos_table, const void* sin_table,
                     int64_t table_stride_row, int64_t n_pos, const int64_t* position_ids, int64_t pos_stride_b, int B,
                     int H, int L, int D, int dtype, void* stream) {
  int rc;
  if ((rc = check_tensor(x)) || (rc = check_tensor(out))) return rc;
  if (cos_table == nullptr || sin_table == nullptr || position_ids == nullptr) return LMK_ERR_NULL;
  if (!aligned16(cos_table) || !aligned16(sin_table) || !stride_ok(table_stride_row)) return LMK_ERR_ALIGN;
  if (B <= 0 || H <= 0 || L <= 0 || pos_stride_b < 0) return LMK_ERR_SHAPE;
  if (!(D == 64 || D == 128)) return LMK_ERR_UNSUPPORTED;
  if (!(dtype == LMK_DTYPE_BF16 || dtype == LMK_DTYPE_F16)) return LMK_ERR_UNSUPPORTED;
  if (n_pos < 1) return LMK_ERR_TABLE;
  lmk::RotaryParams p = {};
  p.x = x->ptr; p.out = out->ptr; p.cos = cos_table; p.sin = sin_table;
  p.pos = position_ids; p.pos_stride_b = pos_stride_b; p.n_pos = n_pos;
  p.B = B; p.H = H; p.L = L;
  p.xs_b = x->stride_b; p.xs_h = x->stride_h; p.xs_r = x->stride_row;
  p.os_b = out->stride_b; p.os_h = out->stride_h; p.os_r = out->stride_row;
  p.cs_r = table_stride_row;
  return lmk::launch_rotary(p, D, dtype, (hipStream_t)stream);
}

int lmk_apply_rotary_qk(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* q_out, const lmk_tensor4* k_out,
                        const void* cos_table, const void* sin_table, int64_t table_stride_row, int64_t n_pos,
                        const int64_t* position_ids, int64_t pos_stride_b, int B, int H, int L, int D, int dtype,
                        void* stream) {
  int rc;
  if ((rc = check_tensor(q)) || (rc = check_tensor(k)) || (rc = check_tensor(q_out)) || (rc = check_tensor(k_out))) return rc;
  if (cos_table == nullptr || sin_table == nullptr || position_ids == nullptr) return LMK_ERR_NULL;
  if (!aligned16(cos_table) || !aligned16(sin_table) || !stride_ok(table_stride_row)) return LMK_ERR_ALIGN;
  if (B <= 0 || H <= 0 || L <= 0 || pos_stride_b < 0) return LMK_ERR_SHAPE;
  if (!(D == 64 || D == 128)) return LMK_ERR_UNSUPPORTED;
  if (!(dtype == LMK_DTYPE_BF16 || dtype == LMK_DTYPE_F16)) return LMK_ERR_UNSUPPORTED;
  if (n_pos < 1) return LMK_ERR_TABLE;
  lmk::RotaryParams p = {};
  p.x = q->ptr; p.out = q_out->ptr; p.x2 = k->ptr; p.out2 = k_out->ptr; p.cos = cos_table; p.sin = sin_table;
  p.pos = position_ids; p.pos_stride_b = pos_stride_b; p.n_pos = n_pos;
  p.B = B; p.H = H; p.L = L;
  p.xs_b = q->stride_b; p.xs_h = q->stride_h; p.xs_r = q->stride_row;
  p.os_b = q_out->stride_b; p.os_h = q_out->stride_h; p.os_r = q_out->stride_row;
  p.x2s_b = k->stride_b; p.x2s_h = k->stride_h; p.x2s_r = k->stride_row;
  p.o2s_b = k_out->stride_b; p.o2s_h = k_out->stride_h; p.o2s_r = k_out->stride_row;
  p.cs_r = table_stride_row;
  return lmk::launch_rotary(p, D, dtype, (hipStream_t)stream);
}

// ---- the attend step as one call: local window, fused forward on it, gather + attend ----
namespace {
struct AttendLayout {
  size_t q_win, k_win, v_win, o_win, L, M, total;
  int W;   // rows of the local window: inc + T
};
AttendLayout attend_layout(int B, int H, int T, int S, int D, int block) {
  AttendLayout l;
  const int inc = S % block;
  l.W = inc + T;
  const size_t rows = (size_t)B * H * l.W, tile = align256(rows * D * 2), stat = align256(rows * 4);
  l.q_win = 0;
  l.k_win = inc ? tile : 0;                  // without a tail the new chunk is the window: only o, L, M are needed
  l.v_win = inc ? 2 * tile : 0;
  l.o_win = inc ? 3 * tile : 0;
  l.L = l.o_win + tile;
  l.M = l.L + stat;
  l.total = l.M + stat;
  return l;
}

// Every argument check of the attend step's three stages (local window, fused forward on it, gather +
// attend), run before the first of them is enqueued: a rejected call has launched nothing.
int attend_precheck(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache, const int64_t* idx,
                    const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table, const void* sin_table,
                    int64_t table_stride_row, int64_t n_pos, const lmk_tensor4* out, const void* workspace, int B,
                    int H, int T, int S, int D, float sm_scale, int block, int top_k, int dtype, bool need_idx) {
  int rc;
  if ((rc = check_tensor(q)) || (rc = check_tensor(kcache)) || (rc = check_tensor(vcache)) ||
      (rc = check_tensor(k_loc)) || (rc = check_tensor(v_loc)) || (rc = check_tensor(out)))
    return rc;
  if (cos_table == nullptr || sin_table == nullptr || workspace == nullptr || (need_idx && idx == nullptr))
    return LMK_ERR_NULL;
  if (!aligned16(cos_table) || !aligned16(sin_table) || !stride_ok(table_stride_row) || !aligned16(workspace))
    return LMK_ERR_ALIGN;
  if ((rc = check_retrieval(B, H, T, S, D, block, top_k, dtype, n_pos))) return rc;
  if (!(block == 32 || block == 64 || block == 128)) return LMK_ERR_UNSUPPORTED;   // gather + attend, fused forward
  if (!std::isfinite(sm_scale) || !(sm_scale > 0.f)) return LMK_ERR_SCALE;
  const int inc = S % block;
  if (inc && T + inc > block) return LMK_ERR_SHAPE;             // llama_mem.py:330
  if (!slice_fits_32bit(q, T) || !slice_fits_32bit(k_loc, T) || !slice_fits_32bit(v_loc, T)) return LMK_ERR_UNSUPPORTED;
  return LMK_OK;
}
}  // namespace

size_t lmk_attend_workspace_bytes(int B, int H, int T, int S, int D, int block) {
  if (B <= 0 || H <= 0 || T <= 0 || S <= 0 || D <= 0 || block <= 0) return 0;
  return attend_layout(B, H, T, S, D, block).total;
}

int lmk_attend(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache, const int64_t* idx,
               const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table, const void* sin_table,
               int64_t table_stride_row, int64_t n_pos, const lmk_tensor4* out, void* workspace,
               size_t workspace_bytes, int B, int H, int T, int S, int D, float sm_scale, int block, int top_k,
               int dtype, void* stream) {
  if (int rc = attend_precheck(q, kcache, vcache, idx, k_loc, v_loc, cos_table, sin_table, table_stride_row, n_pos, out,
                               workspace, B, H, T, S, D, sm_scale, block, top_k, dtype, true))
    return rc;
  const int inc = S % block;
  const AttendLayout l = attend_layout(B, H, T, S, D, block);
  if (workspace_bytes < l.total) return LMK_ERR_WORKSPACE;
  if (lmk::gather_takes_local_window(T, S, block))             // a handful of new tokens: one launch, nothing staged
    return gather_attend_impl(q, kcache, vcache, idx, cos_table, sin_table, table_stride_row, n_pos, nullptr, nullptr,
                              nullptr, 0, out, B, H, T, S, D, sm_scale, block, top_k, dtype, stream, nullptr, k_loc, v_loc);
  char* w = static_cast<char*>(workspace);
  const int64_t W = l.W;
  auto win = [&](size_t off) { return lmk_tensor4{w + off, (int64_t)H * W * D, W * D, (int64_t)D}; };
  const lmk_tensor4 q_win = win(l.q_win), k_win = win(l.k_win), v_win = win(l.v_win), o_win = win(l.o_win);
  float* L = reinterpret_cast<float*>(w + l.L);
  float* M = reinterpret_cast<float*>(w + l.M);
  int rc;
  if (inc) {
    if ((rc = lmk_local_window(q, kcache, vcache, k_loc, v_loc, cos_table, sin_table, table_stride_row, n_pos, &q_win,
                               &k_win, &v_win, B, H, T, S, D, block, dtype, stream)))
      return rc;
    if ((rc = lmk_attn_fwd(&q_win, &k_win, &v_win, &o_win, L, M, B, H, (int)W, (int)W, D, sm_scale, block, 0, dtype, stream)))
      return rc;
  } else if ((rc = lmk_attn_fwd(q, k_loc, v_loc, &o_win, L, M, B, H, T, T, D, sm_scale, block, 0, dtype, stream))) {
    return rc;
  }
  // the window's last T rows, read in place
  const lmk_tensor4 o_loc = {w + l.o_win + (size_t)inc * D * 2, o_win.stride_b, o_win.stride_h, o_win.stride_row};
  return lmk_gather_attend(q, kcache, vcache, idx, cos_table, sin_table, table_stride_row, n_pos, &o_loc, L + inc,
                           M + inc, W, out, B, H, T, S, D, sm_scale, block, top_k, dtype, stream);
}

int lmk_retrieve_and_attend(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache,
                            const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table,
                            const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                            const lmk_tensor4* out, void* retrieve_workspace, size_t retrieve_workspace_bytes,
                            int reuse_landmark_keys, void* attend_workspace, size_t attend_workspace_bytes, int B,
                            int H, int T, int S, int D, float sm_scale, int block, int top_k, int dtype, void* stream) {
  // everything the attend step would reject is rejected here, before the selection is enqueued
  if (int rc = attend_precheck(q, kcache, vcache, idx_out, k_loc, v_loc, cos_table, sin_table, table_stride_row, n_pos,
                               out, attend_workspace, B, H, T, S, D, sm_scale, block, top_k, dtype, true))
    return rc;
  if (attend_workspace_bytes < attend_layout(B, H, T, S, D, block).total) return LMK_ERR_WORKSPACE;
  if (retrieve_workspace == nullptr) return LMK_ERR_NULL;
  if (!aligned16(retrieve_workspace)) return LMK_ERR_ALIGN;
  if (retrieve_workspace_bytes < retr_layout(B, H, T, S, D, block).total) return LMK_ERR_WORKSPACE;
  if (lmk::gather_takes_local_window(T, S, block)) {
    // decode: the selection (slice step where it serves, else the fused top-k), then a gather that merges the
    // slices' candidates and attends to the local window itself -- no window, no forward launch
    int rc;
    lmk::RetrParams pr;
    if ((rc = retrieve_topk_impl(false, q, kcache, cos_table, sin_table, table_stride_row, n_pos, idx_out, retrieve_workspace,
                                 retrieve_workspace_bytes, B, H, T, S, D, block, top_k, dtype, stream, &pr)))
      return rc;
    if (lmk::topk_slices(pr) > 0) {
      if (!reuse_landmark_keys && (rc = lmk::launch_landmark_keys(pr, D, dtype, (hipStream_t)stream))) return rc;
      if ((rc = lmk::launch_topk_slices(pr, D, dtype, (hipStream_t)stream))) return rc;
      return gather_attend_impl(q, kcache, vcache, idx_out, cos_table, sin_table, table_stride_row, n_pos, nullptr, nullptr,
                                nullptr, 0, out, B, H, T, S, D, sm_scale, block, top_k, dtype, stream, &pr, k_loc, v_loc);
    }
    if ((rc = lmk::launch_retrieve_topk(pr, D, dtype, reuse_landmark_keys != 0, (hipStream_t)stream))) return rc;
    return gather_attend_impl(q, kcache, vcache, idx_out, cos_table, sin_table, table_stride_row, n_pos, nullptr, nullptr,
                              nullptr, 0, out, B, H, T, S, D, sm_scale, block, top_k, dtype, stream, nullptr, k_loc, v_loc);
  }
  if (block == 32) {
    // The forward over the local window needs nothing from the selection and alone fills a fraction of the chip, so
    // it shares a launch with a step of the selection that is as small:
    //   many query rows   window, forward || rotation of the landmark keys, fused top-k, gather
    //   up to 1024 rows   window, [rotation,] forward || slice step of the selection, gather that first picks a row's
    //                     k best from the slices' candidates
    int rc;
    const int inc = S % block;
    const AttendLayout l = attend_layout(B, H, T, S, D, block);
    char* w = static_cast<char*>(attend_workspace);
    const int64_t W = l.W;
    auto win = [&](size_t off) { return lmk_tensor4{w + off, (int64_t)H * W * D, W * D, (int64_t)D}; };
    const lmk_tensor4 q_win = win(l.q_win), k_win = win(l.k_win), v_win = win(l.v_win), o_win = win(l.o_win);
    float* L = reinterpret_cast<float*>(w + l.L);
    float* M = reinterpret_cast<float*>(w + l.M);
    lmk::RetrParams pr;
    if ((rc = retrieve_topk_impl(false, q, kcache, cos_table, sin_table, table_stride_row, n_pos, idx_out, retrieve_workspace,
                                 retrieve_workspace_bytes, B, H, T, S, D, block, top_k, dtype, stream, &pr)))
      return rc;
    lmk::FwdParams pf;
    if (inc) {
      if ((rc = attn_fwd_impl(&q_win, &k_win, &v_win, &o_win, L, M, B, H, (int)W, (int)W, D, sm_scale, block, block, 0, dtype,
                              stream, nullptr, 0, 0, nullptr, &pf)))
        return rc;
      if ((rc = lmk_local_window(q, kcache, vcache, k_loc, v_loc, cos_table, sin_table, table_stride_row, n_pos, &q_win,
                                 &k_win, &v_win, B, H, T, S, D, block, dtype, stream)))
        return rc;
    } else if ((rc = attn_fwd_impl(q, k_loc, v_loc, &o_win, L, M, B, H, T, T, D, sm_scale, block, block, 0, dtype, stream,
                                   nullptr, 0, 0, nullptr, &pf))) {
      return rc;
    }
    const bool by_slices = lmk::topk_slices(pr) > 0;
    if (by_slices) {
      if (!reuse_landmark_keys && (rc = lmk::launch_landmark_keys(pr, D, dtype, (hipStream_t)stream))) return rc;
      if ((rc = lmk::launch_fwd32_topk_slices(pf, pr, D, dtype, (hipStream_t)stream))) return rc;
    } else {
      if (reuse_landmark_keys) rc = lmk::launch_fwd(pf, D, block, dtype, (hipStream_t)stream);
      else rc = lmk::launch_fwd32_landmark_keys(pf, pr, D, dtype, (hipStream_t)stream);
      if (rc) return rc;
      if ((rc = lmk::launch_retrieve_topk(pr, D, dtype, true, (hipStream_t)stream))) return rc;   // keys are rotated already
    }
    const lmk_tensor4 o_loc = {w + l.o_win + (size_t)inc * D * 2, o_win.stride_b, o_win.stride_h, o_win.stride_row};
    return gather_attend_impl(q, kcache, vcache, idx_out, cos_table, sin_table, table_stride_row, n_pos, &o_loc, L + inc,
                              M + inc, W, out, B, H, T, S, D, sm_scale, block, top_k, dtype, stream,
                              by_slices ? &pr : nullptr);
  }
  if (int rc = retrieve_topk_impl(reuse_landmark_keys != 0, q, kcache, cos_table, sin_table, table_stride_row, n_pos,
                                  idx_out, retrieve_workspace, retrieve_workspace_bytes, B, H, T, S, D, block, top_k,
                                  dtype, stream))
    return rc;
  return lmk_attend(q, kcache, vcache, idx_out, k_loc, v_loc, cos_table, sin_table, table_stride_row, n_pos, out,
                    attend_workspace, attend_workspace_bytes, B, H, T, S, D, sm_scale, block, top_k, dtype, stream);
}

}  // extern "C"
