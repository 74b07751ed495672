// Block-sparse attention forward for gfx950 (MI355X): pre-pass + flash-style main kernel.
//
// Replaces the reference's Triton launchers and kernels
//   hbsattn/fwd_triton_auto_tile_size.py:76-310, hbsattn/fwd_triton_fix_tile_size.py:30-276
// with one kernel family that does not tile per k block.  Semantics follow the
// reference's golden implementation hbsattn/reference.py:23-107.
//
// Data flow
//   prep kernel : block_mask bytes + sequence boundaries -> one bit per in-sequence
//                 k block (causally unreachable blocks already cleared) and one
//                 geometry record per q block.
//   main kernel : one workgroup (4 wavefronts) per (kv head, q block, group of 4
//                 "wave slots"); a wave slot is 32 query rows of one q head, so the
//                 q heads of a GQA group and the 32-row slices of a q block share the
//                 K/V tiles one workgroup stages in LDS.  Kept k blocks that are
//                 adjacent merge into key runs which are walked in 64-key tiles.
//
// Matrix-core mapping (v_mfma_f32_32x32x16, 64-lane wavefronts)
//   S^T[key, query] = K[key, :] . Q[query, :]     A = K tile (LDS, ds_read_b128)
//                                                  B = Q^T   (registers, whole kernel)
//   The accumulator then holds, per lane, 16 keys of ONE query (query = lane % 32),
//   so row max / row sum are in-lane reductions plus one lane<->lane+32 exchange
//   (v_permlane32_swap), and the online-softmax state (m, l) is one scalar per lane.
//   O^T[d, query] += V^T[d, key] . P^T[key, query]  A = V^T (LDS, ds_read_b64_tr_b16)
//                                                  B = P^T = the S^T accumulator
//                                                      converted in place, no shuffle.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <type_traits>

#include "hbsattn_amd.h"

namespace {

typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define HBSA_AS1(p) ((const __attribute__((address_space(1))) void *)(p))
#define HBSA_AS3(p) ((__attribute__((address_space(3))) void *)(p))

constexpr int kThreads = 256;   // 4 wavefronts
constexpr int kWaveRows = 32;   // query rows per wavefront (the MFMA N dimension)
constexpr int kTileKeys = 64;   // keys per main-loop step
constexpr int kWalkReportTiles = 8;   // an item adds its progress to its walk clock every so many tiles (a power of two)
constexpr float kLog2e = 1.4426950408889634f;
constexpr int kMaxDevices = 64;            // devices of one process the launch caches cover
constexpr float kLazyRescaleLog2 = 8.0f;  // running max may lag the true max by 2^8

// Geometry of one q block, written by the pre-pass (48 bytes).
struct QBlockInfo {
  int32_t row_begin;   // token row of the block's first query
  int32_t rows;        // queries in the block (ragged last block of a sequence)
  int32_t key_begin;   // token row of the sequence's first key
  int32_t klen;        // keys in the sequence
  int32_t q_pos;       // in-sequence position of the block's first query
  int32_t shift;       // k_len - q_len: bottom-right causal alignment
  int32_t nkblk;       // k blocks in the sequence
  int32_t kmax;        // exclusive in-sequence bound of keys any row of the block may see
  int32_t seq;         // first q block of the block's sequence: identifies the sequence by a number below num_q_block
                       // (the batch index can exceed it when the batch holds sequences without queries)
  int32_t flags;       // 1: the block's sequence did not fit the tensors; it has no keys (and perhaps no rows)
  int32_t pad[2];
};
static_assert(sizeof(QBlockInfo) == 48, "QBlockInfo is read as twelve 32-bit words");

struct Sched;

struct PrepParams {
  const int32_t *cu_q, *cu_k, *q_block_to_batch, *cu_num_q_block, *cu_num_k_block;
  const uint8_t *mask;
  int64_t ms_h, ms_q, ms_k;
  QBlockInfo *info;
  uint32_t *bits;
  struct Sched *sched;
  unsigned long long *clock;
  int32_t nqb, qbs, kbs, wpr, causal;
  int32_t batch, nkb, total_q, total_k;   // bounds the sequences' boundaries are checked against
};

// Division by a launch constant d, exact for 0 <= n < 2^31: n / d == (n * m) >> s with
// s = 31 + ceil(log2 d), m = ceil(2^s / d) (which fits 32 bits).  Three scalar instructions where
// a hardware-less integer division takes about forty.
struct FastDiv {
  uint32_t m, s;
};
__host__ __device__ inline uint32_t fast_div(uint32_t n, FastDiv f) { return (uint32_t)(((uint64_t)n * f.m) >> f.s); }
inline FastDiv make_fast_div(uint32_t d) {
  uint32_t l = 0;
  while (((uint64_t)1 << l) < d) ++l;
  FastDiv f;
  f.s = 31 + l;
  f.m = (uint32_t)((((uint64_t)1 << f.s) + d - 1) / d);
  return f;
}

// (Fields are appended at the end, never inserted: the compiler fetches the kernel arguments in aligned groups,
// and a layout that splits the fields the tile loop uses makes it fetch some of them again inside that loop,
// where a scalar load's wait also waits for every hand-issued LDS read; measured, 0.8 % of T for one such shift.)
struct FwdParams {
  const char *q, *k, *v;
  char *out;
  const QBlockInfo *info;
  const uint32_t *bits;
  int64_t q_s, q_h, k_s, k_h, v_s, v_h, o_s, o_h;  // bytes
  int32_t nqb, ratio, kbs, wpr, causal;
  int32_t wps;    // wave slots per q head = ceil(q_block_size / 32)
  int32_t nw;     // wavefronts per workgroup (4 or 8)
  int32_t nsub;   // workgroups per (kv head, q block) = ceil(ratio * wps / nw)
  uint32_t q_sign;  // 0x80008000 when softmax_scale < 0 (Q is negated, |scale| used)
  float c;        // |softmax_scale| * log2(e)
  float lag;      // kLazyRescaleLog2 / c: how far the running max may lag, in raw score units
  FastDiv div_nsub, div_nqb, div_kbs;   // divisions on the scheduler's path
  int32_t f32;    // fp32 inputs staged as fp16: the softmax constants come from the launch record, where
                  // the setup kernel derived them from the tensors' maxima
  int32_t nhead_k;
  int32_t one_each;   // > 0: the number of work items, handed out without queues: workgroup i of G takes items i, 2G - 1 - i, 2G + i, ...
  struct Sched *sched;
  // Walk order of the kept k blocks (see the kernel's comment).  walk != 0: the workgroups that work on
  // one (kv head, sequence) keep near each other in key space through a shared clock, so that they find
  // each other's K/V blocks in the L2; the summation order, and with it the last bits of the result,
  // then depend on timing.  walk == 0: every item walks its blocks in ascending order (deterministic).
  unsigned long long *clock;   // [nhead_k, num_q_block]: clock of (kv head, first q block of the sequence)
  int32_t walk;
  float *lse;             // optional [total_q, nhead_q] log-sum-exp output (nullptr: none)
  int64_t lse_s, lse_h;   // its strides in elements
  // Split over key blocks (few, long work items): every (kv head, q block, slot group) becomes
  // nparts items, part i sees the bit row copy i (its share of the k blocks) and stores a
  // normalised fp32 partial result and its log-sum-exp; hbsa_merge_kernel combines them.
  int32_t nparts;         // 1: no split
  FastDiv div_nparts;
  float *part_out;        // [nparts, total_q, nhead_q, D]
  float *part_lse;        // [nparts, total_q, nhead_q]
  int32_t total_q, nhead_q;
  // One-launch form (the kernel instantiated with FUSED): no pre-pass has run, `info` and `bits` are unused,
  // and the scheduler derives every item's geometry and bit row itself from the caller's arrays.
  const int32_t *cu_q, *cu_k, *cu_nqb, *cu_nkb;   // int32[batch + 1] each
  const uint8_t *mask;                            // block_mask bytes, innermost (k block) stride 1
  int64_t ms_h, ms_q;                             // its head and q block strides
  int32_t batch, nkb_total, total_k, qbs;
  int32_t pack;   // host side only: the launch uses the kernel whose wave slots are packed across the q heads of a GQA group
  FastDiv div_nhk;   // division by nhead_k (items handed out without queues)
};

// Boundaries of one sequence of the packed batch, as read from the caller's device arrays.
struct SeqBounds {
  int32_t q0, q1;     // cu_q_seqlens[b], [b + 1]
  int32_t k0, k1;     // cu_k_seqlens[b], [b + 1]
  int32_t kb0, kb1;   // cu_num_k_block[b], [b + 1]
  int32_t qb0;        // cu_num_q_block[b]
};

// Geometry record of q block g.  The sequence boundaries are device data the host cannot check, so they
// are checked here against the token counts of q and k/v and the block counts.  A sequence that does
// not fit (a wrong cu_seqlens, q/k/v shorter than it says, inconsistent block metadata) gets no keys:
// nothing of k, v or the mask is read for it, and those of its query rows that lie inside q and out are
// written as zeros, like any row that sees no key (flags = 1 marks such a block).  When not even the
// query side makes sense (have == false: the block's sequence index is outside the batch) the block
// has no rows and nothing is written for it.  kb0: first global k block of the sequence.
__host__ __device__ inline QBlockInfo q_block_geometry(int g, bool have, SeqBounds s, int qbs, int kbs, int causal,
                                                      int nkb_total, int total_q, int total_k, int &kb0) {
  const int qlen = s.q1 - s.q0, klen_in = s.k1 - s.k0, nkb_in = s.kb1 - s.kb0;
  const int q_pos = (g - s.qb0) * qbs;
  const bool q_ok = have && s.q0 >= 0 && qlen > 0 && s.qb0 >= 0 && g >= s.qb0 && q_pos >= 0 && q_pos < qlen &&
                    (int64_t)s.q0 + q_pos < total_q;
  const bool ok = q_ok && (int64_t)s.q0 + qlen <= total_q && s.k0 >= 0 && klen_in >= 0 && (int64_t)s.k0 + klen_in <= total_k &&
                  s.kb0 >= 0 && nkb_in >= 0 && (int64_t)s.kb0 + nkb_in <= nkb_total && (int64_t)nkb_in * kbs >= klen_in;
  QBlockInfo r;
  r.row_begin = q_ok ? s.q0 + q_pos : 0;
  int rows = 0;
  if (q_ok) {
    rows = qlen - q_pos < qbs ? qlen - q_pos : qbs;
    if (rows > total_q - r.row_begin) rows = total_q - r.row_begin;
  }
  r.rows = rows;
  r.key_begin = ok ? s.k0 : 0;
  r.klen = ok ? klen_in : 0;
  r.q_pos = q_ok ? q_pos : 0;
  r.shift = ok ? klen_in - qlen : 0;
  r.nkblk = ok ? nkb_in : 0;
  int kmax = 0;
  if (ok) {
    kmax = klen_in;
    if (causal && q_pos + rows + r.shift < kmax) kmax = q_pos + rows + r.shift;
    if (kmax < 0) kmax = 0;
  }
  r.kmax = kmax;
  r.seq = q_ok ? s.qb0 : 0;
  r.flags = ok ? 0 : 1;
  r.pad[0] = r.pad[1] = 0;
  kb0 = ok ? s.kb0 : 0;
  return r;
}

// --------------------------------------------------------------------------------------
// Pre-pass: one wavefront per (kv head, q block).
// --------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void hbsa_prep_kernel(PrepParams p) {
  const int lane = threadIdx.x & 63;
  const int g = blockIdx.x * 4 + (threadIdx.x >> 6);
  // the work-queue counters of the launch record start at zero; every attention launch leaves them so
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x < 9) ((uint32_t *)p.sched)[threadIdx.x] = 0;
  if (g >= p.nqb) return;
  const int hk = blockIdx.y;
  const int b = p.q_block_to_batch[g];
  SeqBounds sb = {0, 0, 0, 0, 0, 0, 0};
  const bool have = b >= 0 && b < p.batch;
  if (have) {
    sb.q0 = p.cu_q[b]; sb.q1 = p.cu_q[b + 1];
    sb.k0 = p.cu_k[b]; sb.k1 = p.cu_k[b + 1];
    sb.kb0 = p.cu_num_k_block[b]; sb.kb1 = p.cu_num_k_block[b + 1];
    sb.qb0 = p.cu_num_q_block[b];
  }
  int kb0;
  const QBlockInfo r = q_block_geometry(g, have, sb, p.qbs, p.kbs, p.causal, p.nkb, p.total_q, p.total_k, kb0);
  const int nkb = r.nkblk;
  const int nvis = min(nkb, (r.kmax + p.kbs - 1) / p.kbs);
  if (hk == 0 && lane == 0) p.info[g] = r;
  if (lane == 0) p.clock[(size_t)hk * p.nqb + g] = 0ull;   // the walk clocks start at zero (and every launch leaves them so)
  uint32_t *row = p.bits + ((size_t)hk * p.nqb + g) * p.wpr;
  const uint8_t *m = p.mask + hk * p.ms_h + g * p.ms_q + kb0 * p.ms_k;
  const int nw64 = (nkb + 63) >> 6;
  for (int w = 0; w < nw64; ++w) {
    const int j = w * 64 + lane;
    const bool keep = j < nvis && m[j * p.ms_k] != 0;
    const uint64_t bal = __ballot(keep);
    if (lane < 2) row[2 * w + lane] = lane ? (uint32_t)(bal >> 32) : (uint32_t)bal;
  }
}

// --------------------------------------------------------------------------------------
// Element-type policies.
// --------------------------------------------------------------------------------------
struct ElemBF16 {
  static __device__ __forceinline__ f32x16 mfma(short8v a, short8v b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
  static __device__ __forceinline__ uint32_t scale_packed(uint32_t w, float f) { return pack2(lo(w) * f, hi(w) * f); }
  // acc + lo + hi of a packed pair (v_dot2c_f32_bf16 with a vector of ones)
  static __device__ __forceinline__ float dot2_ones(uint32_t packed, float acc) {
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed), ones, acc, false);
  }
};
struct ElemF16 {
  static __device__ __forceinline__ f32x16 mfma(short8v a, short8v b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  static __device__ __forceinline__ float lo(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w).x; }
  static __device__ __forceinline__ float hi(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w).y; }
  static __device__ __forceinline__ uint32_t scale_packed(uint32_t w, float f) { return pack2(lo(w) * f, hi(w) * f); }
  static __device__ __forceinline__ float dot2_ones(uint32_t packed, float acc) {
    const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, packed), ones, acc, false);
  }
};

// exchange-and-combine between lane i and lane i^32
__device__ __forceinline__ float half_max(float x) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
__device__ __forceinline__ float half_sum(float x) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

// --------------------------------------------------------------------------------------
// Main kernel (persistent).  D = head dim (32, 64, 128 or 256); rows of K/V tiles are D*2 bytes.  At D = 256 a
// wavefront's output accumulator and query operand alone are 192 registers, so a CU runs one workgroup of four
// wavefronts, each with the 512 registers of a SIMD (accumulators in the AGPR half), and its two 128 KB of K/V
// tile buffers take most of the LDS.
//
// Scheduling.  The grid is as many workgroups as fit the device at once and every workgroup
// loops over work items it claims from eight queues, one per XCD (the chip's eight dies, each
// with its own L2).  Queue v holds, head-major, the items of the kv heads h with h % 8 == v:
// for each such head every q block of the packed batch from the last to the first (under a
// causal mask the heaviest blocks of each sequence come first), and for each q block its
// groups of four wave slots.  The queues need no storage: entry idx of queue v decodes
// arithmetically, and one atomic counter per queue hands entries out.  A workgroup reads the
// id of the XCD it runs on from the hardware and drains that XCD's queue, so at any time the
// workgroups that share an L2 walk the K/V of one (or few) kv heads; when its queue is empty it
// takes from the other queues, which balances the tail.  A workgroup ends after at most eight
// consecutive failed claims, one per queue.
//
// Division of labour.  Wavefront 0 is also the workgroup's scheduler: one item ahead it
// claims a queue entry, fetches that item's geometry record and mask bits, and expands the
// bits into a list of 64-key tiles in LDS (adjacent kept k blocks merge into key runs).  The
// main loop of every wavefront then only steps through that list: no mask logic, no global
// metadata loads and no divergent control flow remain on the per-tile path.
//
// Pipelining.  K/V tiles stream through two LDS buffers without a bubble at item borders:
// while the last tile of an item is being computed the first tile of the next item is
// already on its way and the next item's Q rows are being fetched.
//
// LDS: K[2][64][D] then V[2][64][D] (double-buffered 64-key tiles), 16-byte chunks of
// every row XOR-swizzled so that both the K reads (16 rows x one chunk per 16 lanes) and
// the transposing V reads (4 rows x 64 bytes per 32 lanes) spread over all banks; then two
// item headers and two tile lists.
// --------------------------------------------------------------------------------------
struct Sched {
  uint32_t qnext[8];   // next unclaimed entry of each queue
  uint32_t done;       // workgroups of the running attention launch that have made their last claim
  // fp32 inputs staged as fp16 only (written by hbsa_setup_kernel, read by the attention kernel at its start):
  float c;             // |softmax_scale| * log2(e), divided by the q and k staging multipliers
  float lag;           // kLazyRescaleLog2 / c, in raw score units
  float out_mul;       // 1 / (v staging multiplier)
  // bit patterns of max|x| over q, k, v and the power-of-two staging multipliers
  uint32_t amax[3];
  float in_mul[3];
  uint32_t pad[46];
};
static_assert(sizeof(Sched) == 256, "Sched is one 256-byte slot of the workspace");

// Softmax constants of an attention launch on fp32 inputs staged as fp16: they follow from the maxima
// the absmax kernels left in s->amax.  (Launches on 16-bit inputs carry their constants as kernel
// arguments and need no such step.)
__global__ void hbsa_setup_kernel(Sched *s, float c, int f32) {
  if (threadIdx.x != 0) return;
  float out_mul = 1.f;
  if (f32) {
    // Each tensor is staged as fp16 after multiplication by a power of two that brings its largest
    // magnitude into [2^14, 2^15): exact, and as far from fp16's overflow and underflow as possible.
    float mul[3];
    for (int i = 0; i < 3; ++i) {
      const int e = (int)((s->amax[i] >> 23) & 255u);   // biased exponent of max|x|
      int sh = 14 - (e - 127);
      if (e == 0 || e == 255) sh = 0;                   // all zero (or denormal), inf or nan: leave as is
      sh = sh > 126 ? 126 : (sh < -126 ? -126 : sh);    // 2^sh and its reciprocal stay normal numbers
      mul[i] = __builtin_ldexpf(1.f, sh);
      s->in_mul[i] = mul[i];
    }
    c = c / mul[0] / mul[1];
    if (!(c >= 1.2e-38f)) c = 1.2e-38f;                 // keep -inf * c == -inf
    if (c > 3e38f) c = 3e38f;
    out_mul = 1.f / mul[2];
  }
  s->c = c;
  s->lag = kLazyRescaleLog2 / c;
  s->out_mul = out_mul;
}

__global__ void hbsa_f32_begin_kernel(Sched *s) {
  if (threadIdx.x < 3) s->amax[threadIdx.x] = 0;
}

// fp32 staging.  A tensor is [tokens, heads, D] with element strides (tok_s, head_s), rows of D
// contiguous floats, 16-byte aligned; one thread handles 4 consecutive floats.
struct F32Tensor {
  const float *x;
  int64_t tok_s, head_s;
  int32_t heads, dshift;   // dshift = log2(D / 4)
  int64_t quads;           // tokens * heads * D / 4
};
__device__ __forceinline__ const float *f32_quad_ptr(const F32Tensor &t, int64_t i) {
  const int64_t row = i >> t.dshift;
  const int dq = (int)(i & ((1 << t.dshift) - 1));
  return t.x + (row / t.heads) * t.tok_s + (row % t.heads) * t.head_s + dq * 4;
}
// max |x| as a bit pattern (for non-negative floats the integer order is the float order)
__global__ __launch_bounds__(256) void hbsa_f32_absmax_kernel(F32Tensor t, uint32_t *amax) {
  uint32_t m = 0;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < t.quads; i += (int64_t)gridDim.x * 256) {
    const u32x4 v = *(const u32x4 *)f32_quad_ptr(t, i);
    m = max(max(m, v.x & 0x7fffffffu), max(max(v.y & 0x7fffffffu, v.z & 0x7fffffffu), v.w & 0x7fffffffu));
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off));
  if ((threadIdx.x & 63) == 0 && m != 0) atomicMax(amax, m);
}
// fp16 copy, contiguous [tokens, heads, D], of x * *mul
__global__ __launch_bounds__(256) void hbsa_f32_stage_kernel(F32Tensor t, const float *mul, uint32_t *dst) {
  const float m = *mul;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < t.quads; i += (int64_t)gridDim.x * 256) {
    const float *src = f32_quad_ptr(t, i);
    u32x2 w;
    w.x = ElemF16::pack2(src[0] * m, src[1] * m);
    w.y = ElemF16::pack2(src[2] * m, src[3] * m);
    *(u32x2 *)(dst + 2 * i) = w;
  }
}

constexpr int kListCap = 1024;   // tile entries per list; longer items are expanded in chunks
// Up to this many items per resident workgroup are handed out without the per-XCD work queues, in a fixed order
// (see claim() in the kernel).  Measured against the queues: 8 x 512 tokens 71 -> 45 us, 8 x 1024 113 -> 99,
// 8 x 2048 causal 200 -> 189, C5 0.33 -> 0.245 ms; at sixteen per workgroup 8 x 4096 tokens lose 5 % and at 64
// C2 and C3 lose 5-8 % (the queues keep one head's K/V in one XCD's L2).
constexpr int kStaticShare = 8;
// One-launch form: sequences whose boundaries the scheduler keeps in LDS (batch + 1 entries of four arrays),
// and bytes of its staging area for one row of block_mask bytes (2048 blocks and the alignment slack)
constexpr int kSeqCap = 128;
constexpr int kMaskWindow = 2048;
constexpr int kMaskStage = kMaskWindow + 256;

// Item header in LDS (16 ints).
enum { H_HK = 0, H_QB, H_SUB, H_TOTAL, H_ROW_BEGIN, H_ROWS, H_KEY_BEGIN, H_Q_POS, H_SHIFT, H_PART, H_T0, H_SEQ, H_NKBLK, H_WORDS = 16 };

__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// A tile entry packs the in-sequence position of the tile's first key (a multiple of 16) and
// the number of valid keys (1..64).
__device__ __forceinline__ int pack_tile(int pos, int valid) { return ((pos >> 4) << 6) | (valid - 1); }

// Expands one item's kept-block bits into tile entries [chunk_base, chunk_base + kListCap) of
// the item's tile sequence, written to list[0..); returns the item's total tile count.
// Executed by one whole wavefront; `first_words`: lane i holds bit word i of the row.  Rows longer than
// 2048 blocks ask `more_words(window)` for the words window * 64 + lane (lane i: word window * 64 + i, zero
// past the row's end), arrived and ready to use.
template <typename MoreWords>
__device__ __forceinline__ int build_tile_list(int *list, int chunk_base, MoreWords &&more_words, int nwords, int kbs,
                                                FastDiv div_kbs, int kmax, uint32_t first_words, int lane) {
  if (kmax <= 0 || nwords <= 0) return 0;
  int total = 0;
  if ((kbs & 63) == 0) {
    // Blocks are whole tiles: every kept block yields kbs/64 tiles (those starting at or past
    // kmax are dropped; they would be the last of the list).  Two bit words are expanded per
    // step: lane l looks at bit (l & 31) of word 2*step + (l >> 5), and its tiles go right after
    // the tiles of the kept blocks below it.
    const int tpb = kbs >> 6;
    const int half = lane >> 5, bit = lane & 31;
    const int j_last = (int)fast_div((uint32_t)(kmax - 1), div_kbs);   // no bit above this block is set
    int window = 0;
    uint32_t held = lane < nwords ? first_words : 0u;
    for (int w2 = 0; w2 < nwords; w2 += 2) {
      if ((w2 >> 6) != window) {   // rows longer than 2048 blocks only
        window = w2 >> 6;
        held = more_words(window);
      }
      const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)held, w2 & 63);
      const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)held, (w2 + 1) & 63);   // nwords is even
      if ((lo | hi) == 0) continue;
      const uint32_t mine = half ? hi : lo;
      if ((mine >> bit) & 1u) {
        const int below = __builtin_popcount(mine & ((1u << bit) - 1u)) + (half ? __builtin_popcount(lo) : 0);
        const int j = (w2 + half) * 32 + bit;
        int off = total + below * tpb - chunk_base;
        for (int t = 0; t < tpb; ++t, ++off) {
          const int pos = j * kbs + 64 * t;
          if (pos < kmax && off >= 0 && off < kListCap) list[off] = pack_tile(pos, min(kTileKeys, kmax - pos));
        }
      }
      total += (__builtin_popcount(lo) + __builtin_popcount(hi)) * tpb;
      if ((j_last >> 6) == (w2 >> 1)) {   // tiles dropped at the end of the last visible block
        const uint32_t wsel = (j_last & 32) ? hi : lo;
        if ((wsel >> (j_last & 31)) & 1u) total -= tpb - ((kmax - j_last * kbs + 63) >> 6);
      }
    }
  } else {
    // General block sizes: walk the runs of adjacent kept blocks serially (wavefront-uniform).
    int window = 0;
    uint32_t held = lane < nwords ? first_words : 0u;
    auto word = [&](int w) -> uint32_t {
      if ((w >> 6) != window) {   // rows longer than 2048 blocks only
        window = w >> 6;
        held = more_words(window);
      }
      return (uint32_t)__builtin_amdgcn_readlane((int)held, w & 63);
    };
    int blk = 0;
    for (;;) {
      int w = blk >> 5;
      if (w >= nwords) break;
      uint32_t cur = word(w) & (~0u << (blk & 31));
      while (cur == 0) {
        if (++w >= nwords) break;
        cur = word(w);
      }
      if (w >= nwords) break;
      const int first = w * 32 + __builtin_ctz(cur);
      uint32_t inv = ~word(w) & (~0u << (first & 31));
      while (inv == 0) {
        if (++w >= nwords) break;
        inv = ~word(w);
      }
      const int stop = (w >= nwords) ? nwords * 32 : w * 32 + __builtin_ctz(inv);
      blk = stop;
      const int end = min(stop * kbs, kmax);
      for (int pos = first * kbs; pos < end; pos += kTileKeys) {
        const int off = total - chunk_base;
        if (lane == 0 && off >= 0 && off < kListCap) list[off] = pack_tile(pos, min(kTileKeys, end - pos));
        ++total;
      }
      if (end >= kmax) break;
    }
  }
  return total;
}


// ---- LDS reads issued by hand.  The compiler neither waits for these nor knows they touch LDS,
// so each result must pass through lds_wait<N>() before it is used: LDS operations of a
// wavefront complete in order, and lds_wait<N> returns once at most N of them are outstanding.
// (The transposing read is issued this way because the compiler otherwise waits for every
// outstanding global->LDS load before it; the K reads so that their issue distance is fixed.)
// HAND = false gives the same reads as ordinary loads the compiler schedules and waits for itself (the
// lds_wait calls then do nothing): the form for instantiations that spill registers, where a register with
// a hand-issued read in flight could be saved before its data arrives.
template <int OFF, bool HAND = true>
__device__ __forceinline__ short8v lds_read_b128(uint32_t addr) {
  if constexpr (HAND) {
    short8v r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(r) : "v"(addr), "n"(OFF));
    return r;
  } else {
    return *(const __attribute__((address_space(3))) short8v *)(uintptr_t)(addr + (uint32_t)OFF);
  }
}
template <int OFF, bool HAND = true>
__device__ __forceinline__ short4v lds_read_tr16_b64(uint32_t addr) {
  if constexpr (HAND) {
    short4v r;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=&v"(r) : "v"(addr), "n"(OFF));
    return r;
  } else {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(uintptr_t)(addr + (uint32_t)OFF));
  }
}
template <int N>
__device__ __forceinline__ void lds_wait1(short8v &a) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(a) : "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_wait(short8v &a, short8v &b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_wait(short4v &a, short4v &b, short4v &c, short4v &d, short4v &e, short4v &f, short4v &g,
                                         short4v &h) {
  asm volatile("s_waitcnt lgkmcnt(%8)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f), "+v"(g), "+v"(h) : "n"(N));
}

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

template <int D, typename E, bool OUT32, int NW, bool EXTRAS, bool FUSED, bool PACK>
__global__ __launch_bounds__(NW * 64, D > 128 ? 1 : 8 / NW) void hbsa_fwd_kernel(FwdParams p) {
  // OUT32: fp32 output (the fp32-input path; q/k/v are then fp16 staging copies)
  // EXTRAS: the clocked walk, the split over key blocks and the log-sum-exp output are compiled in.  The
  // plain call uses none of them, and its kernel is a tenth shorter without them (1-2 % faster: eight
  // wavefronts in different parts of a long kernel share one instruction cache).
  // FUSED: the one-launch form.  No pre-pass has run: wavefront 0 derives an item's geometry from the
  // sequence boundaries (kept in LDS) and its bit row from the item's own block_mask bytes, which it
  // fetches into an LDS staging area one item ahead, where the other form fetches the prepared records.
  // PACK: wave slots packed across the q heads of a GQA group (see slot_of below); instantiated for the
  // one-launch form only, since either placement of the queries gives the same results bit for bit.
  // NW: wavefronts (wave slots) of a workgroup, 4 or 8.  Eight are used when the q heads of a GQA group
  // and the 32-row slices of a q block give an item more than four wave slots: one workgroup per CU then
  // stages every K/V tile once for all of them instead of two workgroups staging it each.
  constexpr int RB = D * 2;            // row bytes
  constexpr int CPR = RB / 16;         // 16-byte chunks per row
  constexpr int RPG = 16 / CPR > 0 ? 16 / CPR : 1;  // rows per 256-byte bank sweep
  constexpr int TILE_BYTES = kTileKeys * RB;
  constexpr int LOADS = CPR / NW;      // 16-byte loads per thread per tile per operand
  static_assert(LOADS >= 1, "a tile row has fewer 16-byte chunks than the workgroup has wavefronts");
  constexpr int KSTEPS = D / 16;       // MFMA k-steps of Q.K^T
  constexpr int DT = D / 32;           // 32-row tiles of O^T
  constexpr bool HAND = D <= 128;      // operand reads from LDS issued and waited for by hand (see lds_read_b128)

  extern __shared__ __attribute__((aligned(1024))) char lds[];
  char *lds_k = lds;
  int *lds_hdr = (int *)(lds + 4 * TILE_BYTES);     // [2][H_WORDS]
  int *lds_list = lds_hdr + 2 * H_WORDS;            // [2][kListCap]
  int *lds_seq = lds_list + 2 * kListCap;           // FUSED: [4][kSeqCap] cu_q, cu_k, cu_num_q_block, cu_num_k_block
  uint8_t *lds_mask = (uint8_t *)(lds_seq + 4 * kSeqCap);   // FUSED: [kMaskStage] block_mask bytes of the staged item
  auto hdr_word = [&](int c_, int i) { return __builtin_amdgcn_readfirstlane(lds_hdr[c_ * H_WORDS + i]); };

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g32 = lane >> 5;   // which half of the wavefront
  const int l32 = lane & 31;   // query within the wave slot / key row within a sub-tile

  // softmax constants of this launch (uniform): kernel arguments, or for fp32 inputs staged as fp16 what
  // the setup kernel that precedes this launch derived on the device
  float sm_c = p.c, sm_lag = p.lag, sm_out_mul = 1.f;
  if (p.f32) {
    sm_c = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, p.sched->c)));
    sm_lag = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, p.sched->lag)));
    sm_out_mul = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, p.sched->out_mul)));
  }
  // Leaving: wavefront 0 makes every claim of its workgroup.  Once its last claim has been performed it
  // counts the workgroup as done, and the workgroup that completes the count puts the queue counters
  // back to zero, so the next launch on this work description needs no preparation of its own.
  auto leave = [&]() {
    if (wave != 0 || p.one_each) return;   // (items without queues: no counter was touched)
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this workgroup's last claim has returned
    if (lane == 0) {
      const uint32_t before = atomicAdd(&p.sched->done, 1u);
      if (before + 1 == gridDim.x) {
#pragma unroll
        for (int i = 0; i < 8; ++i) atomicExch(&p.sched->qnext[i], 0u);
        atomicExch(&p.sched->done, 0u);
      }
    }
  };

  // ------------------------------------------------------------------ scheduler (wavefront 0)
  const int nq = p.nhead_k < 8 ? p.nhead_k : 8;                       // queues that hold work
  const int home = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 7;    // HW_REG_XCC_ID
  const int first_queue = home < nq ? home : home % nq;
  int tries = 0;                    // queues found empty so far
  uint32_t pending = 0xffffffffu;   // queue index claimed for the item after the staged one
  int st_hk = -1, st_qb = 0, st_sub = 0, st_part = 0;   // staged item: claimed, records fetched, list not built
  uint32_t st_info = 0, st_bits = 0;       // lane i: word i of its QBlockInfo / of its bit row

  auto queue_len = [&](int v) -> uint32_t {
    const int heads = v < p.nhead_k ? (p.nhead_k - v + 7) / 8 : 0;
    return (uint32_t)heads * (uint32_t)p.nqb * (uint32_t)p.nsub * (uint32_t)p.nparts;
  };
  // Without queues (few items per workgroup).  The items are numbered last q blocks first, the heads of a q block
  // next to each other (decode_free_entry), so under a causal mask their weights fall with the number.  Workgroup
  // i of G takes item i, then 2G - 1 - i, 2G + i, 4G - 1 - i, ...: every second round runs backwards, so the
  // lightest item of a round goes to the workgroup that got the heaviest of the round before, and the
  // workgroups (those of one CU, too) end at about the same time.  Nothing is claimed: measured against a shared
  // counter for the later rounds, 8 x 1024 tokens 106 -> 99 us and C5 0.258 -> 0.241 ms.
  int own_claims = 0;
  auto claim = [&]() -> uint32_t {   // the value is looked at an item later, so its latency is hidden
    uint32_t r = 0xffffffffu;
    if (p.one_each) {
      r = (own_claims & 1) ? (uint32_t)(own_claims + 1) * gridDim.x - 1u - blockIdx.x : (uint32_t)own_claims * gridDim.x + blockIdx.x;
      ++own_claims;
    } else if (tries < 8) {
      if (lane == 0) r = atomicAdd(&p.sched->qnext[(first_queue + tries) & 7], 1u);
    }
    return r;
  };
  // (kv head, q block, slot group, part) of entry `claimed` of a head-major list that starts at kv head
  // `head0` and holds every `head_step`-th head
  auto decode_entry = [&](uint32_t claimed, int head0, int head_step) {
    const uint32_t whole = fast_div(claimed, p.div_nparts);   // parts of one item are neighbours
    st_part = (int)(claimed - whole * (uint32_t)p.nparts);
    const uint32_t t = fast_div(whole, p.div_nsub);
    st_sub = (int)(whole - t * (uint32_t)p.nsub);
    const uint32_t h = fast_div(t, p.div_nqb);
    st_hk = head0 + head_step * (int)h;
    st_qb = p.nqb - 1 - (int)(t - h * (uint32_t)p.nqb);
  };
  // (kv head, q block, slot group, part) of item `claimed` of the numbering without queues: parts, slot groups and
  // kv heads of a q block are neighbours, the last q block comes first
  auto decode_free_entry = [&](uint32_t claimed) {
    const uint32_t whole = fast_div(claimed, p.div_nparts);
    st_part = (int)(claimed - whole * (uint32_t)p.nparts);
    const uint32_t t = fast_div(whole, p.div_nsub);
    st_sub = (int)(whole - t * (uint32_t)p.nsub);
    const uint32_t b = fast_div(t, p.div_nhk);
    st_hk = (int)(t - b * (uint32_t)p.nhead_k);
    st_qb = p.nqb - 1 - (int)b;
  };
  // ---- one-launch form: geometry and mask bits without a pre-pass (wavefront 0)
  const uint8_t *st_mrow = nullptr;   // staged item: address of the mask byte of its sequence's first k block
  int st_nvis = 0, st_ms = 0;         // its k blocks below the causal bound; offset of the first one's byte in the staging area
  // geometry of q block qb from the boundaries in LDS (uniform values); kb0: first global k block of its sequence.
  // Consecutive items of a queue mostly belong to one sequence, so the last sequence's boundaries are kept.
  SeqBounds seq_sb = {0, 0, 0, 0, 0, 0, 0};
  int seq_qb_end = -1;      // q blocks [seq_sb.qb0, seq_qb_end) belong to the kept sequence (none at first)
  bool seq_have = false;
  auto fused_geometry = [&](int qb, int &kb0) -> QBlockInfo {
    if (!(qb >= seq_sb.qb0 && qb < seq_qb_end)) {
      int b = 0;   // sequences that start at or before qb, minus one
      for (int base = 0; base < p.batch; base += 64) {
        const int i = base + lane + 1;
        const int first_qb = i <= p.batch ? lds_seq[2 * kSeqCap + i] : 0x7fffffff;
        b += __builtin_popcountll(__builtin_amdgcn_ballot_w64(first_qb <= qb));
      }
      seq_have = b < p.batch;
      seq_sb = SeqBounds{0, 0, 0, 0, 0, 0, 0};
      seq_qb_end = -1;
      if (seq_have) {
        auto at = [&](int arr, int i) { return __builtin_amdgcn_readfirstlane(lds_seq[arr * kSeqCap + i]); };
        seq_sb.q0 = at(0, b); seq_sb.q1 = at(0, b + 1);
        seq_sb.k0 = at(1, b); seq_sb.k1 = at(1, b + 1);
        seq_sb.qb0 = at(2, b); seq_qb_end = at(2, b + 1);
        seq_sb.kb0 = at(3, b); seq_sb.kb1 = at(3, b + 1);
      }
    }
    return q_block_geometry(qb, seq_have, seq_sb, p.qbs, p.kbs, p.causal, p.nkb_total, p.total_q, p.total_k, kb0);
  };
  const uint32_t lds_mask_addr = (uint32_t)(uintptr_t)HBSA_AS3(lds_mask);
  // Requests the mask bytes of blocks [first, first + count), count <= kMaskWindow, of the row at `mrow`: whole
  // aligned dwords, four bytes per lane, straight into the staging area (a dword that holds a byte of the
  // row lies inside the mask's allocation).  Returns the offset of block `first`'s byte in the staging area.
  auto mask_dma = [&](const uint8_t *mrow, int first, int count) -> int {
    const uintptr_t a = (uintptr_t)(mrow + first);
    const int sh = (int)(a & 3);
    const char *base = (const char *)(a - sh);
    const uint32_t last = (uint32_t)(sh + count - 1) & ~3u;   // offset of the last dword needed
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");        // what was read from the staging area before has arrived
    for (uint32_t i = 0; i <= last; i += 256) {
      const uint32_t off = min(i + 4u * (uint32_t)lane, last);   // every lane loads: lanes past the end repeat the last dword
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                   :
                   : "s"(lds_mask_addr + i), "v"(off), "s"(base)
                   : "memory", "m0");
    }
    return sh;
  };
  // bit words of the staged bytes: lane i gets word i (blocks 32 * i .. + 31 of the window; zero from `count` on)
  auto staged_words = [&](int sh, int count) -> uint32_t {
    uint32_t words = 0;
    for (int w64 = 0; w64 * 64 < count; ++w64) {
      const int j = w64 * 64 + lane;
      const bool keep = j < count && lds_mask[sh + j] != 0;
      const uint64_t bal = __builtin_amdgcn_ballot_w64(keep);
      if (lane == 2 * w64) words = (uint32_t)bal;
      if (lane == 2 * w64 + 1) words = (uint32_t)(bal >> 32);
    }
    return words;
  };
  // words of a later window of a row (rows longer than kMaskWindow blocks): fetched and waited for on the spot
  auto fused_more_words = [&](const uint8_t *mrow, int nvis) {
    return [&, mrow, nvis](int window) -> uint32_t {
      const int first = window * kMaskWindow;
      const int count = min(kMaskWindow, nvis - first);
      if (count <= 0) return 0u;
      const int sh = mask_dma(mrow, first, count);
      __builtin_amdgcn_s_waitcnt(0x0F70);
      return staged_words(sh, count);
    };
  };
  // the same for a prepared bit row in the workspace
  auto prepared_more_words = [&](const uint32_t *row, int nwords) {
    return [=](int window) -> uint32_t {
      const int i = window * 64 + lane;
      uint32_t held = i < nwords ? row[i] : 0u;
      __builtin_amdgcn_s_waitcnt(0x0F70);   // wait here, not (for everything in flight) on the common path
      asm volatile("" : "+v"(held));
      return held;
    };
  };

  // turn `pending` into the staged item (claiming again from the next queues when the one it
  // came from is exhausted) and start fetching the item's records
  auto stage = [&]() {
    uint32_t claimed = (uint32_t)__builtin_amdgcn_readfirstlane((int)pending);
    st_hk = -1;
    if (p.one_each) {
      if (claimed < (uint32_t)p.one_each) decode_free_entry(claimed);
    } else {
      while (tries < 8) {
        const int v = (first_queue + tries) & 7;
        if (claimed < queue_len(v)) {
          decode_entry(claimed, v, 8);
          break;
        }
        // This queue has run dry (the tail of the kernel).  Look at the other queues' counters first, all at
        // once, and claim only from one that still shows work: a workgroup then ends after one load instead
        // of seven failed claims in a row, each a round trip to a counter every other workgroup is hitting.
        uint32_t seen = 0xffffffffu;
        if (lane < 8) seen = __hip_atomic_load(&p.sched->qnext[(first_queue + lane) & 7], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        asm volatile("" : "+v"(seen));
        const bool open = lane > tries && lane < 8 && seen < queue_len((first_queue + lane) & 7);
        const uint64_t open_mask = __builtin_amdgcn_ballot_w64(open);
        if (open_mask == 0) {
          tries = 8;
          break;
        }
        tries = __builtin_ctzll(open_mask);
        uint32_t r = 0;
        if (lane == 0) r = atomicAdd(&p.sched->qnext[(first_queue + tries) & 7], 1u);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        asm volatile("" : "+v"(r));
        claimed = (uint32_t)__builtin_amdgcn_readfirstlane((int)r);
      }
    }
    if (st_hk >= 0) {
      if constexpr (FUSED) {
        int kb0;
        const QBlockInfo r = fused_geometry(st_qb, kb0);
        st_info = (uint32_t)(lane == 0 ? r.row_begin : lane == 1 ? r.rows : lane == 2 ? r.key_begin : lane == 3 ? r.klen
                             : lane == 4 ? r.q_pos : lane == 5 ? r.shift : lane == 6 ? r.nkblk : lane == 7 ? r.kmax
                             : lane == 8 ? r.seq : 0);
        st_nvis = min(r.nkblk, (int)fast_div((uint32_t)(r.kmax + p.kbs - 1), p.div_kbs));
        st_mrow = p.mask + (int64_t)st_hk * p.ms_h + (int64_t)st_qb * p.ms_q + kb0;
        st_ms = st_nvis > 0 ? mask_dma(st_mrow, 0, min(st_nvis, kMaskWindow)) : 0;
      } else {
        st_info = lane < 12 ? ((const uint32_t *)(p.info + st_qb))[lane] : 0u;
        st_bits = lane < p.wpr ? p.bits[(((size_t)st_part * p.nhead_k + st_hk) * p.nqb + st_qb) * p.wpr + lane] : 0u;
      }
    }
  };
  // expand the staged item into list `c` and write its header
  auto build = [&](int c) {
    int *hdr = lds_hdr + c * H_WORDS;
    int total = 0;
    if (st_hk >= 0) {
      const int nkblk = __builtin_amdgcn_readlane((int)st_info, 6);
      const int kmax = __builtin_amdgcn_readlane((int)st_info, 7);
      if constexpr (FUSED) {
        // the staged bytes arrived with the wait of a tile (or of the kernel's first lines) since stage()
        st_bits = st_nvis > 0 ? staged_words(st_ms, min(st_nvis, kMaskWindow)) : 0u;
        total = build_tile_list(lds_list + c * kListCap, 0, fused_more_words(st_mrow, st_nvis), 2 * ((st_nvis + 63) >> 6),
                                p.kbs, p.div_kbs, kmax, st_bits, lane);
      } else {
        const int nwords = 2 * ((nkblk + 63) >> 6);
        total = build_tile_list(lds_list + c * kListCap, 0,
                                prepared_more_words(p.bits + (((size_t)st_part * p.nhead_k + st_hk) * p.nqb + st_qb) * p.wpr, nwords),
                                nwords, p.kbs, p.div_kbs, kmax, st_bits, lane);
      }
    }
    if (lane == 0) {
      hdr[H_HK] = st_hk; hdr[H_QB] = st_qb; hdr[H_SUB] = st_sub; hdr[H_TOTAL] = total; hdr[H_PART] = st_part;
      hdr[H_T0] = 0;   // the item's walk starts at its first tile unless next_start() decides otherwise
    }
    if (lane < 9) {   // QBlockInfo words: row_begin, rows, key_begin, klen, q_pos, shift, nkblk, kmax, seq
      const int dst = lane == 0 ? H_ROW_BEGIN : lane == 1 ? H_ROWS : lane == 2 ? H_KEY_BEGIN : lane == 4 ? H_Q_POS
                      : lane == 5 ? H_SHIFT : lane == 6 ? H_NKBLK : lane == 8 ? H_SEQ : -1;
      if (dst >= 0) hdr[dst] = (int)st_info;
    }
  };

  // ---- the walk clock (wavefront 0; p.walk != 0 only).  The online softmax does not care in which
  // order an item's tiles are taken, and the workgroups that share an L2 (one XCD) work on items of
  // one (kv head, sequence) at a time.  They keep near each other in key space, so that a K/V tile one
  // of them fetched is still in the L2 when the others ask for it: every (kv head, sequence) has a
  // clock word that holds, for the workgroups inside its items, their number (low 16 bits) and the sum
  // of their positions (upper 48 bits; a position counts 64-key tiles of the sequence's key space and
  // keeps growing over laps); one 64-bit atomic add updates both and returns both.  An item starts its
  // walk at the first of its tiles at or after the clock's mean position, walks upwards, wraps to its
  // first tile and ends where it began; it adds every step to the clock.  The start is decided two
  // tiles before the item begins (its first tile is requested one tile before).
  unsigned long long w_clk = 0;          // lane 0: the next item's clock as read three tiles before this item's end
  unsigned long long *w_ptr = nullptr;   // this item's clock word, nullptr when it takes no part
  int w_lap = 0, w_told = 0;             // the lap this item started in; the position its clock holds for it
  int w_next_lap = 0;                    // lap the next item starts in (-1: it takes no part); the workgroup's
                                         // first item finds the clocks empty: lap 0, first tile
  int w_lt = 1;                          // 64-key tiles of this item's sequence (the length of a lap)
  // what wavefront 0 remembers of the two items whose lists are in LDS (slot c_): clock word, lap length,
  // and whether the item may take part (its tile list is a single chunk of at least three tiles)
  unsigned long long *w_clock_of[2] = {nullptr, nullptr};
  int w_tiles_of[2] = {1, 1};
  bool w_part_of[2] = {false, false};
  auto note_item = [&](int c_, int total_) {   // right after build(c_), from the staged records
    const int nkblk = __builtin_amdgcn_readlane((int)st_info, 6);
    const int seq = __builtin_amdgcn_readlane((int)st_info, 8);
    w_part_of[c_] = EXTRAS && p.walk != 0 && st_hk >= 0 && total_ >= 3 && total_ <= kListCap;
    w_clock_of[c_] = p.clock + (size_t)(st_hk < 0 ? 0 : st_hk) * p.nqb + seq;
    w_tiles_of[c_] = (nkblk * p.kbs + kTileKeys - 1) >> 6;
  };
  // three tiles before this item ends: read the next item's clock (a load that bypasses the CU's own
  // cache; the clock words live in the XCD's L2, where the atomics on them are performed)
  auto peek_next = [&](int cn) {
    w_next_lap = -1;
    if (!w_part_of[cn]) return;
    if (lane == 0) w_clk = __hip_atomic_load(w_clock_of[cn], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    w_next_lap = 0;
  };
  // two tiles before it ends: the next item's start, from the clock's mean position
  auto next_start = [&](int cn) {
    if (w_next_lap < 0) return;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)w_clk);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(w_clk >> 32));
    const uint32_t members = lo & 0xffffu;
    if (members == 0) return;   // nobody there: start at the first tile, in lap 0
    const float sum = (float)hi * 65536.f + (float)(lo >> 16);
    int mean = __builtin_amdgcn_readfirstlane((int)(sum * __builtin_amdgcn_rcpf((float)members)));
    const int lt = w_tiles_of[cn];
    int lap = __builtin_amdgcn_readfirstlane((int)((float)mean * __builtin_amdgcn_rcpf((float)lt)));
    int pos = mean - lap * lt;
    while (pos < 0) { pos += lt; --lap; }
    while (pos >= lt) { pos -= lt; ++lap; }
    // entries of the (ascending) list below that position
    const int n = hdr_word(cn, H_TOTAL);
    int below = 0;
    for (int i = 0; i < n; i += 64) {
      const bool less = i + lane < n && (lds_list[cn * kListCap + i + lane] >> 8) < pos;   // entry >> 6 = key >> 4
      below += __builtin_popcountll(__builtin_amdgcn_ballot_w64(less));
    }
    if (below >= n) {   // every tile of the item lies below: it starts the next lap at its first tile
      below = 0;
      ++lap;
    }
    if (lane == 0) lds_hdr[cn * H_WORDS + H_T0] = below;
    w_next_lap = lap;
  };
  // first tile of an item: join its clock; later: add the progress since the last report (the atomics
  // return nothing).  wraps: how often the walk has passed the end of the list (0 or 1).
  auto report = [&](int c_, int kpos, bool first, int wraps) {
    if (first) {
      w_ptr = nullptr;
      const int lap0 = w_next_lap;
      w_next_lap = -1;   // the item after this one takes part only if peek_next() says so
      if (lap0 < 0 || !w_part_of[c_]) return;
      w_ptr = w_clock_of[c_];
      w_lt = w_tiles_of[c_];
      w_lap = lap0;
      w_told = w_lap * w_lt + (kpos >> 6);
      if (lane == 0) atomicAdd(w_ptr, ((unsigned long long)(uint32_t)w_told << 16) + 1ull);
      return;
    }
    if (w_ptr == nullptr) return;
    const int now = (w_lap + wraps) * w_lt + (kpos >> 6);
    if (now != w_told && lane == 0) atomicAdd(w_ptr, (unsigned long long)(uint32_t)(now - w_told) << 16);
    w_told = now;
  };
  auto leave_clock = [&]() {
    if (w_ptr == nullptr) return;
    if (lane == 0) atomicAdd(w_ptr, 0ull - (((unsigned long long)(uint32_t)w_told << 16) + 1ull));
    w_ptr = nullptr;
  };

  if (wave == 0) {
    if constexpr (FUSED) {   // the sequences' boundaries, for fused_geometry()
      for (int i = lane; i <= p.batch; i += 64) {
        lds_seq[i] = p.cu_q[i];
        lds_seq[kSeqCap + i] = p.cu_k[i];
        lds_seq[2 * kSeqCap + i] = p.cu_nqb[i];
        lds_seq[3 * kSeqCap + i] = p.cu_nkb[i];
      }
    }
    pending = claim();
    stage();
    if constexpr (FUSED) __builtin_amdgcn_s_waitcnt(0x0F70);   // the first item's mask bytes
    build(0);
    note_item(0, hdr_word(0, H_TOTAL));
    pending = claim();
    stage();
    pending = claim();
  }
  __syncthreads();

  // ------------------------------------------------------------------ per-thread constants
  // tile loads: thread -> (row, 16-byte chunk) of the tile, same for every tile
  uint32_t ld_koff[LOADS], ld_voff[LOADS];   // byte offset of the thread's chunk from the tile's first row
  const uint32_t ks32 = (uint32_t)p.k_s, vs32 = (uint32_t)p.v_s;   // row strides in bytes (the host checks they fit)
  auto ld_place = [&](int i, int &r, uint32_t &kchunk, uint32_t &vchunk) {
    const int c = (i * NW + wave) * 64 + lane;
    const int pc = c % CPR;
    r = c / CPR;
    kchunk = (uint32_t)((pc ^ ((r / RPG) % CPR)) * 16);
    vchunk = (uint32_t)((pc ^ ((CPR >= 8) ? (((r / RPG) % (CPR / 4)) << 2) : 0)) * 16);
  };
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    int r; uint32_t kc, vc;
    ld_place(i, r, kc, vc);
    ld_koff[i] = (uint32_t)r * ks32 + kc;
    ld_voff[i] = (uint32_t)r * vs32 + vc;
  }
  const uint32_t lds_k_addr = (uint32_t)(uintptr_t)HBSA_AS3(lds_k);
  // kbase / vbase: wavefront-uniform address of the tile's first key row (for this kv head).
  // 16 bytes per lane go straight from global memory into LDS at (M0 + 16 * lane); the global
  // address is a scalar base plus a 32-bit per-lane offset.  The V buffers follow the K buffers.
  auto dma16 = [&](auto off_, const char *sbase, uint32_t voff, uint32_t lds_addr) {
    constexpr int off = decltype(off_)::value;
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(sbase), "n"(off)
                 : "memory", "m0", "scc");
  };
  auto tile_ptr = [&](const char *base, int tok, uint32_t stride) {   // tok >= 0
    return base + (uint64_t)(uint32_t)tok * (uint64_t)stride;
  };
  // One operand's half of a tile's loads.  V_PART selects the V buffers (which follow the K buffers).
  auto issue_part = [&](auto v_part_, int buf, const char *base, int valid) {
    constexpr bool V_PART = decltype(v_part_)::value;
    constexpr int lds_off = V_PART ? 2 * TILE_BYTES : 0;
    const uint32_t l0 = lds_k_addr + (uint32_t)(buf * TILE_BYTES) + (uint32_t)wave * 1024u;
    if (valid == kTileKeys) {
      static_for<0, LOADS>([&](auto i_) {
        constexpr int i = decltype(i_)::value;
        dma16(std::integral_constant<int, lds_off + i * NW * 1024>{}, base, V_PART ? ld_voff[i] : ld_koff[i], l0);
      });
    } else {   // ragged tail of a run: rows past the end re-read the last valid row (masked later)
      static_for<0, LOADS>([&](auto i_) {
        constexpr int i = decltype(i_)::value;
        int r; uint32_t kc, vc;
        ld_place(i, r, kc, vc);
        r = min(r, valid - 1);
        dma16(std::integral_constant<int, lds_off + i * NW * 1024>{}, base, (uint32_t)r * (V_PART ? vs32 : ks32) + (V_PART ? vc : kc), l0);
      });
    }
  };
  auto issue_k = [&](int buf, const char *kbase, int valid) { issue_part(std::false_type{}, buf, kbase, valid); };
  auto issue_v = [&](int buf, const char *vbase, int valid) { issue_part(std::true_type{}, buf, vbase, valid); };
  auto issue_loads = [&](int buf, const char *kbase, const char *vbase, int valid) {
    issue_k(buf, kbase, valid);
    issue_v(buf, vbase, valid);
  };

  // per-lane LDS read addresses
  // K (A operand of S^T): row l32 (+32), chunk (2*ks + g32) ^ swz(row)
  const int k_rd = l32 * RB + ((g32 ^ ((l32 / RPG) % CPR)) << 4);
  // V^T (A operand of O^T) through ds_read_b64_tr_b16: within a group of 16 lanes, lane r
  // supplies the address of key (r / 4), dims 4*(r % 4) .. +3 and receives dim r of 4 keys.
  const int v_key = 4 * g32 + ((lane & 15) >> 2);
  const int v_lc = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
  const int v_swz = (CPR >= 8) ? (((v_key / RPG) % (CPR / 4)) << 2) : 0;
  const int v_rd = v_key * RB + ((v_lc | v_swz) << 4) + 8 * (lane & 1);

  // Absolute LDS addresses of this lane's operand reads in the CURRENT tile buffer: one per k-step
  // for K, one per 32-dim block for V.  flip_buffers() moves them to the other buffer with one add
  // each (the two buffers of K, and of V, are TILE_BYTES apart), so the per-tile path has no
  // address arithmetic besides that.
  uint32_t k_addr[KSTEPS], v_addr[DT];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) k_addr[ks] = lds_k_addr + (uint32_t)(k_rd ^ (ks * 32));
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) v_addr[dt] = lds_k_addr + 2 * TILE_BYTES + (uint32_t)(v_rd ^ (dt * 64));
  int buf = 0;
  auto flip_buffers = [&]() {
    buf ^= 1;
    const uint32_t step = buf ? (uint32_t)TILE_BYTES : (uint32_t)-TILE_BYTES;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      k_addr[ks] += step;
      asm volatile("" : "+v"(k_addr[ks]));   // keep it in its register instead of recomputing it per read
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      v_addr[dt] += step;
      asm volatile("" : "+v"(v_addr[dt]));
    }
  };

  // This wavefront's slot of an item.  A wave slot holds up to 32 (q head of the GQA group, query row of the
  // q block) entries.  Plain form: the 32-row slices of one head after another (slot = head * wps + slice), a
  // q block of 80 rows filling 32 + 32 + 16 entries per head.  Packed form (PACK: q_block_size no multiple
  // of 32 and several q heads per kv head): entry number = head * rows + row, every slot takes the next 32
  // numbers, so a slot may hold the last rows of one head and the first rows of the next and only an item's
  // last slot is partly empty.  Every lane works on one query with its own pointers and causal limit, and
  // all heads of the group see the same K/V tiles, so nothing else changes.
  struct Slot {
    int first;          // first entry number (packed) / first row of the slice (plain)
    int n;              // entries held, <= 0: none
    int min_r, max_r;   // smallest and largest query row among them
    int hq;             // plain form: the slot's q head; packed form: the group's first q head
  };
  auto quotient = [](int a, int b) {   // a / b for 0 <= a < 2^20, 0 < b < 2^12
    return (int)(((float)a + 0.5f) * __builtin_amdgcn_rcpf((float)b));
  };
  auto slot_of = [&](int hk, int sub, int rows) -> Slot {
    const int slot = sub * NW + wave;
    Slot sl;
    if constexpr (PACK) {
      sl.hq = hk * p.ratio;
      sl.first = slot * kWaveRows;
      sl.n = min(kWaveRows, p.ratio * rows - sl.first);
      sl.min_r = 0;
      sl.max_r = rows - 1;
      if (sl.n > 0) {
        const int h0 = __builtin_amdgcn_readfirstlane(quotient(sl.first, rows));
        const int h1 = __builtin_amdgcn_readfirstlane(quotient(sl.first + sl.n - 1, rows));
        if (h0 == h1) {   // all entries belong to one head
          sl.min_r = sl.first - h0 * rows;
          sl.max_r = sl.min_r + sl.n - 1;
        }
      }
    } else {
      const int head = slot / p.wps;
      sl.hq = hk * p.ratio + head;
      sl.first = (slot % p.wps) * kWaveRows;
      sl.n = head < p.ratio ? min(kWaveRows, rows - sl.first) : 0;
      sl.min_r = sl.first;
      sl.max_r = sl.first + sl.n - 1;
    }
    return sl;
  };
  // q head and row (inside the q block) of entry idx of a slot with entries; idx past the last entry repeats it.
  // (The plain form needs nothing but the slot: what stays live through an item's tiles is as little as it can be.)
  auto slot_entry = [&](const Slot &sl, int idx, int rows, int &hq, int &r) {
    const int e = sl.first + min(idx, sl.n - 1);
    if constexpr (PACK) {
      const int h = quotient(e, rows);
      hq = sl.hq + h;
      r = e - h * rows;
    } else {
      hq = sl.hq;
      r = e;
    }
  };

  // Q^T fragments (B operand) of one item: lane (l32, g32) ends up with, per k-step ks, the 16 bytes
  // d = 16*ks + 8*g32 .. +7 of query row l32.  Fetched so that four lanes read 64 contiguous bytes
  // of a row (16 rows per instruction instead of 32, half the memory requests): with h = bit 4 of
  // the lane, load A_k takes row (lane % 16), load B_k row 16 + (lane % 16), both at bytes
  // 64*k + 32*h + 16*g32; then the h = 1 lanes of A_k and the h = 0 lanes of B_k trade places
  // (v_permlane16_swap), which leaves k-step 2k in A_k and k-step 2k+1 in B_k.
  short8v qf[KSTEPS];
  auto load_q = [&](int hk, int sub, int row_begin, int rows) {
    const Slot sl = slot_of(hk, sub, rows);
    if (sl.n <= 0) return;   // this wavefront has no rows: qf is never used
    const int l16 = lane & 15;
    int hq_a, r_a, hq_b, r_b;
    slot_entry(sl, l16, rows, hq_a, r_a);
    slot_entry(sl, 16 + l16, rows, hq_b, r_b);
    const char *base = p.q + (lane & 16) * 2 + g32 * 16;
    const char *ra = base + (int64_t)(row_begin + r_a) * p.q_s + (int64_t)hq_a * p.q_h;
    const char *rb = base + (int64_t)(row_begin + r_b) * p.q_s + (int64_t)hq_b * p.q_h;
    if constexpr (KSTEPS >= 2) {
#pragma unroll
      for (int k = 0; k < KSTEPS / 2; ++k) {
        u32x4 a = *(const u32x4 *)(ra + 64 * k), b = *(const u32x4 *)(rb + 64 * k);
        a ^= p.q_sign;
        b ^= p.q_sign;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const auto r = __builtin_amdgcn_permlane16_swap(a[j], b[j], false, false);
          a[j] = r[0];
          b[j] = r[1];
        }
        qf[2 * k] = __builtin_bit_cast(short8v, a);
        qf[2 * k + 1] = __builtin_bit_cast(short8v, b);
      }
    }
  };

  // ------------------------------------------------------------------ first item
  int c = 0;   // list / header of the current item
  if (hdr_word(0, H_HK) < 0) {
    leave();
    return;
  }
  {
    const int total0 = hdr_word(0, H_TOTAL);
    if (total0 > 0) {
      const int e = __builtin_amdgcn_readfirstlane(lds_list[0]);
      const int tok = hdr_word(0, H_KEY_BEGIN) + ((e >> 6) << 4);
      const int hk = hdr_word(0, H_HK);
      issue_loads(0, tile_ptr(p.k + (int64_t)hk * p.k_h, tok, ks32), tile_ptr(p.v + (int64_t)hk * p.v_h, tok, vs32), (e & 63) + 1);
    }
  }
  load_q(hdr_word(0, H_HK), hdr_word(0, H_SUB), hdr_word(0, H_ROW_BEGIN), hdr_word(0, H_ROWS));

  for (;;) {   // ------------------------------------------------------ one iteration per work item
    const int cur_hk = hdr_word(c, H_HK);
    const int cur_sub = hdr_word(c, H_SUB);
    const int cur_part = hdr_word(c, H_PART);   // read now: wavefront 0 rewrites the header while others finish this item
    const int total = hdr_word(c, H_TOTAL);
    const int row_begin = hdr_word(c, H_ROW_BEGIN);
    const int rows = hdr_word(c, H_ROWS);
    const int key_begin = hdr_word(c, H_KEY_BEGIN);
    const int q_pos = hdr_word(c, H_Q_POS);
    const int shift = hdr_word(c, H_SHIFT);

    if (wave == 0) {   // stay one item ahead: expand the staged item, stage the one after it
      build(c ^ 1);
      if (EXTRAS && p.walk) note_item(c ^ 1, hdr_word(c ^ 1, H_TOTAL));
      stage();
      pending = claim();
    }

    const Slot slot = slot_of(cur_hk, cur_sub, rows);
    const int nrows = slot.n;   // lanes l32 < nrows hold a query
    // last key position this lane's query / any query of the wavefront sees (causal): key position <= q_pos + row + shift
    int lane_kvis;
    if constexpr (PACK) {
      int hq_mine, r_mine = 0;
      if (nrows > 0) slot_entry(slot, l32, rows, hq_mine, r_mine);
      lane_kvis = q_pos + r_mine + shift;
    } else {
      lane_kvis = q_pos + slot.first + min(l32, nrows - 1) + shift;   // (a wavefront without queries never looks at it)
    }
    const int wave_kvis_min = q_pos + slot.min_r + shift;
    const int wave_kvis_max = q_pos + slot.max_r + shift;
    const bool active = nrows > 0;

    f32x16 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
    float m_run = -INFINITY;  // running reference max, raw (unscaled) score units
    float l_run = 0.f;        // this lane's share of the row sum

    const char *kg = p.k + (int64_t)cur_hk * p.k_h + (int64_t)key_begin * p.k_s;
    const char *vg = p.v + (int64_t)cur_hk * p.v_h + (int64_t)key_begin * p.v_s;

    int nxt_hk = -1;          // known once the last tile is reached
    int chunk_base = 0;
    // the walk starts at entry t0 of the (ascending) list and wraps: step t takes entry rot(t)
    const int t0 = total <= kListCap ? hdr_word(c, H_T0) : 0;
    for (;;) {   // ---------------------------------------------------- chunks of the tile list (usually one)
      const int n = min(kListCap, total - chunk_base);
      auto rot = [&](int x) { return x + t0 >= n ? x + t0 - n : x + t0; };   // x < n
      int held = 0;           // lane i: entry of step (window * 64 + i) of the current chunk
      for (int t = 0; t < n; ++t) {   // ---------------------------------- one iteration per 64-key tile
        if ((t & 63) == 0) held = (t + lane < n) ? lds_list[c * kListCap + rot(t + lane)] : 0;
        const int e = __builtin_amdgcn_readlane(held, t & 63);
        const int kpos = (e >> 6) << 4, valid = (e & 63) + 1;

        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the current tile has landed in LDS
        // Everything fetched so far has arrived, the scheduler's records included: tell the
        // compiler here, or it waits for ALL outstanding memory traffic where they are first read.
        asm volatile("" : "+v"(st_info), "+v"(st_bits), "+v"(pending), "+v"(w_clk));
        __syncthreads();                     // ... for every wave, and the other buffers are free

        const bool last = chunk_base + t + 1 == total;
        // The clock is dealt with on few tiles only (wavefront 0; any work it does alone on every tile
        // makes the other three wait at the next barrier): the item's first tile, every eighth, and
        // the last three.
        if (EXTRAS && p.walk && wave == 0 && ((t & (kWalkReportTiles - 1)) == 0 || chunk_base + t + 3 >= total)) {
          report(c, kpos, chunk_base + t == 0, t + t0 >= n ? 1 : 0);
          if (chunk_base + t + 3 == total) peek_next(c ^ 1);
          if (chunk_base + t + 2 == total) next_start(c ^ 1);
          if (last) leave_clock();
        }
        int nx_valid = 0;                 // > 0: a next tile exists and its loads go out during this tile
        const char *nx_vbase = nullptr, *nx_kbase = nullptr;
        if (t + 1 < n) {
          int e1;
          if (((t + 1) & 63) == 0) {
            const int h1 = (t + 1 + lane < n) ? lds_list[c * kListCap + rot(t + 1 + lane)] : 0;
            e1 = __builtin_amdgcn_readlane(h1, 0);
          } else {
            e1 = __builtin_amdgcn_readlane(held, (t + 1) & 63);
          }
          const int tok = (e1 >> 6) << 4;
          nx_valid = (e1 & 63) + 1;
          nx_vbase = tile_ptr(vg, tok, vs32);
          nx_kbase = tile_ptr(kg, tok, ks32);
        } else if (last) {
          nxt_hk = hdr_word(c ^ 1, H_HK);
          if (nxt_hk >= 0 && hdr_word(c ^ 1, H_TOTAL) > 0) {
            const int e1 = __builtin_amdgcn_readfirstlane(lds_list[(c ^ 1) * kListCap + hdr_word(c ^ 1, H_T0)]);
            const int tok = hdr_word(c ^ 1, H_KEY_BEGIN) + ((e1 >> 6) << 4);
            nx_valid = (e1 & 63) + 1;
            nx_vbase = tile_ptr(p.v + (int64_t)nxt_hk * p.v_h, tok, vs32);
            nx_kbase = tile_ptr(p.k + (int64_t)nxt_hk * p.k_h, tok, ks32);
          }
        }
        // The next tile's K is requested right after this tile's first operand reads, its V only after
        // the first MFMA block: the wavefronts then do not all queue at the load unit at once.

        const bool compute = active && (!p.causal || kpos <= wave_kvis_max);
        if (!compute && nx_valid > 0) {
          issue_k(buf ^ 1, nx_kbase, nx_valid);
          issue_v(buf ^ 1, nx_vbase, nx_valid);
        }
        if (compute) {
          // The tile is processed as two halves of 32 keys so that, inside one wavefront, the
          // matrix cores always have work queued while the vector ALU does the softmax of the
          // other half:   S0, max(S0) | S1 + exp(S0) | PV0 + max(S1), exp(S1) | PV1.
          const bool edge = valid < kTileKeys || (p.causal && kpos + valid - 1 > wave_kvis_min);
          int lim = valid;                      // keys (of this lane's query) below lim are visible
          if (p.causal) lim = min(lim, lane_kvis - kpos + 1);
          lim -= 4 * g32;

          f32x16 s0, s1;
#pragma unroll
          for (int i = 0; i < 16; ++i) { s0[i] = 0.f; s1[i] = 0.f; }

          // ---- K operand reads: 2 * KSTEPS reads (all k-steps of the first 32 keys, then of the
          // second 32), PF of them in flight, each consumed by one MFMA
          constexpr int PF = 4;
          constexpr int NK = 2 * KSTEPS;
          short8v kb[PF];
          auto read_k = [&](auto i_) {
            constexpr int i = decltype(i_)::value;
            constexpr int ks = i % KSTEPS;
            if constexpr (i < KSTEPS) kb[i % PF] = lds_read_b128<0, HAND>(k_addr[ks]);
            else kb[i % PF] = lds_read_b128<32 * RB, HAND>(k_addr[ks]);
          };
          static_for<0, PF>(read_k);
          // the next tile's K is requested while this tile's first operands are on their way from LDS
          if (nx_valid > 0) issue_k(buf ^ 1, nx_kbase, nx_valid);
          // ---- S0 = K[0:32] . Q^T
          static_for<0, KSTEPS>([&](auto i_) {
            constexpr int i = decltype(i_)::value;
            constexpr int ahead = (NK - 1 - i) < (PF - 1) ? (NK - 1 - i) : (PF - 1);
            if constexpr (HAND) lds_wait1<ahead>(kb[i % PF]);
            s0 = E::mfma(kb[i % PF], qf[i % KSTEPS], s0);
            if constexpr (i + PF < NK) read_k(std::integral_constant<int, i + PF>{});
          });

          if (nx_valid > 0) issue_v(buf ^ 1, nx_vbase, nx_valid);

          // row max of one half, merged into the running max; O and l are rescaled (rarely:
          // the running max may lag the true one by 2^kLazyRescaleLog2)
          auto half_rowmax = [&](f32x16 &sh, int key0) {
            if (edge) {
#pragma unroll
              for (int i = 0; i < 16; ++i)
                if (key0 + 8 * (i >> 2) + (i & 3) >= lim) sh[i] = -INFINITY;
            }
            // The first reduction step is an instruction the compiler knows, so that it inserts
            // the wait states an MFMA result needs before the vector ALU may read it; the
            // hand-written v_max3 steps all depend on that first result.
            float mx = __builtin_amdgcn_fmed3f(sh[0], sh[1], INFINITY);   // = max(sh[0], sh[1])
#pragma unroll
            for (int i = 2; i < 16; i += 2) mx = max3(mx, sh[i], sh[i + 1]);
            mx = half_max(mx);
            const bool grow = mx > m_run + sm_lag;
            if (__builtin_amdgcn_ballot_w64(grow) != 0) {
              const float m_new = grow ? mx : m_run;
              const float alpha = grow ? __builtin_amdgcn_exp2f((m_run - m_new) * sm_c) : 1.f;
              l_run *= alpha;
#pragma unroll
              for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
              m_run = m_new;
            }
          };
          // exponentials of one half, packed to the element type (two groups of 16 keys), row sum
          auto half_exp = [&](const f32x16 &sh, short8v &p_lo, short8v &p_hi) {
            const float mc = (m_run == -INFINITY) ? 0.f : m_run * sm_c;
            u32x4 w[2];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
              for (int q4 = 0; q4 < 4; ++q4) {
                const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sh[8 * j + 2 * q4], sm_c, -mc));
                const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sh[8 * j + 2 * q4 + 1], sm_c, -mc));
                w[j][q4] = E::pack2(e0, e1);
                // fp32 adds, not v_dot2c: the dot instructions share the matrix pipeline and would
                // stall the MFMAs of the wavefront's neighbour on the SIMD
                l_run += e0 + e1;
              }
            p_lo = __builtin_bit_cast(short8v, w[0]);
            p_hi = __builtin_bit_cast(short8v, w[1]);
          };
          auto read_vgroup = [&](auto g_, short4v *dst) {   // V^T operands of keys 16*g .. 16*g+15
            constexpr int g = decltype(g_)::value;
            static_for<0, DT>([&](auto dt_) {
              constexpr int dt = decltype(dt_)::value;
              dst[2 * dt] = lds_read_tr16_b64<g * 16 * RB, HAND>(v_addr[dt]);
              dst[2 * dt + 1] = lds_read_tr16_b64<g * 16 * RB + 8 * RB, HAND>(v_addr[dt]);
            });
          };
          auto wait_vgroup = [&](auto n_, short4v *v) {
            constexpr int n = decltype(n_)::value;
            if constexpr (!HAND) {
              (void)v;   // the compiler waits for its own reads
            } else if constexpr (DT == 4) {
              lds_wait<n>(v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7]);
            } else if constexpr (DT == 2) {
              asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]) : "n"(n));
            } else {
              asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(v[0]), "+v"(v[1]) : "n"(n));
            }
          };
          auto pv_group = [&](const short8v &pb, const short4v *v) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
              const short8v va = __builtin_shufflevector(v[2 * dt], v[2 * dt + 1], 0, 1, 2, 3, 4, 5, 6, 7);
              o[dt] = E::mfma(va, pb, o[dt]);
            }
          };

          half_rowmax(s0, 0);

          // ---- S1 = K[32:64] . Q^T   interleaved with   P0 = exp(S0)
          short8v p0a, p0b, p1a, p1b;
          static_for<KSTEPS, NK>([&](auto i_) {
            constexpr int i = decltype(i_)::value;
            constexpr int ahead = (NK - 1 - i) < (PF - 1) ? (NK - 1 - i) : (PF - 1);
            if constexpr (HAND) lds_wait1<ahead>(kb[i % PF]);
            s1 = E::mfma(kb[i % PF], qf[i % KSTEPS], s1);
            if constexpr (i + PF < NK) read_k(std::integral_constant<int, i + PF>{});
          });
          short4v vb[2][2 * DT];
          read_vgroup(std::integral_constant<int, 0>{}, vb[0]);
          read_vgroup(std::integral_constant<int, 1>{}, vb[1]);
          half_exp(s0, p0a, p0b);

          // ---- row max of S1.  P0 was formed under the running max as it stood after S0 and is not
          // accumulated yet, so if that max has to move now (rare), P0 is rescaled along with O and l.
          {
            if (edge) {
#pragma unroll
              for (int i = 0; i < 16; ++i)
                if (32 + 8 * (i >> 2) + (i & 3) >= lim) s1[i] = -INFINITY;
            }
            float mx = __builtin_amdgcn_fmed3f(s1[0], s1[1], INFINITY);
#pragma unroll
            for (int i = 2; i < 16; i += 2) mx = max3(mx, s1[i], s1[i + 1]);
            mx = half_max(mx);
            const bool grow = mx > m_run + sm_lag;
            if (__builtin_amdgcn_ballot_w64(grow) != 0) {
              const float m_new = grow ? mx : m_run;
              const float alpha = grow ? __builtin_amdgcn_exp2f((m_run - m_new) * sm_c) : 1.f;
              l_run *= alpha;
#pragma unroll
              for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
              u32x4 wa = __builtin_bit_cast(u32x4, p0a), wb = __builtin_bit_cast(u32x4, p0b);
#pragma unroll
              for (int q4 = 0; q4 < 4; ++q4) {
                wa[q4] = E::scale_packed(wa[q4], alpha);
                wb[q4] = E::scale_packed(wb[q4], alpha);
              }
              p0a = __builtin_bit_cast(short8v, wa);
              p0b = __builtin_bit_cast(short8v, wb);
              m_run = m_new;
            }
          }

          // ---- O^T += V^T[:, 0:32] . P0   interleaved with   P1 = exp(S1)
          wait_vgroup(std::integral_constant<int, 2 * DT>{}, vb[0]);
          pv_group(p0a, vb[0]);
          read_vgroup(std::integral_constant<int, 2>{}, vb[0]);
          wait_vgroup(std::integral_constant<int, 2 * DT>{}, vb[1]);
          pv_group(p0b, vb[1]);
          read_vgroup(std::integral_constant<int, 3>{}, vb[1]);
          half_exp(s1, p1a, p1b);

          // ---- O^T += V^T[:, 32:64] . P1
          wait_vgroup(std::integral_constant<int, 2 * DT>{}, vb[0]);
          pv_group(p1a, vb[0]);
          wait_vgroup(std::integral_constant<int, 0>{}, vb[1]);
          pv_group(p1b, vb[1]);
        }
        if (last && nxt_hk >= 0) {
          // Q of this item is no longer needed: fetch the next item's rows while the last MFMAs
          // drain and the epilogue runs
          load_q(nxt_hk, hdr_word(c ^ 1, H_SUB), hdr_word(c ^ 1, H_ROW_BEGIN), hdr_word(c ^ 1, H_ROWS));
        }
        flip_buffers();
      }
      chunk_base += n;
      if (chunk_base >= total) break;
      // a longer item: expand the next chunk of its tile list in place
      __syncthreads();
      if (wave == 0) {
        // (the staged records now belong to a later item, so this item's are fetched again)
        const int qb = hdr_word(c, H_QB);
        if constexpr (FUSED) {
          int kb0;
          const QBlockInfo inf = fused_geometry(qb, kb0);
          const int nvis = min(inf.nkblk, (int)fast_div((uint32_t)(inf.kmax + p.kbs - 1), p.div_kbs));
          auto more = fused_more_words(p.mask + (int64_t)cur_hk * p.ms_h + (int64_t)qb * p.ms_q + kb0, nvis);
          const uint32_t first = more(0);
          (void)build_tile_list(lds_list + c * kListCap, chunk_base, more, 2 * ((nvis + 63) >> 6), p.kbs, p.div_kbs, inf.kmax,
                                first, lane);
          // the staging area held the staged item's bytes: request them again (they arrive with the next tile's wait)
          if (st_hk >= 0 && st_nvis > 0) st_ms = mask_dma(st_mrow, 0, min(st_nvis, kMaskWindow));
        } else {
          const QBlockInfo inf = p.info[qb];
          const uint32_t *row = p.bits + (((size_t)cur_part * p.nhead_k + cur_hk) * p.nqb + qb) * p.wpr;
          const int nwords = 2 * ((inf.nkblk + 63) >> 6);
          (void)build_tile_list(lds_list + c * kListCap, chunk_base, prepared_more_words(row, nwords), nwords, p.kbs, p.div_kbs,
                                inf.kmax, lane < nwords ? row[lane] : 0u, lane);
        }
      }
      __syncthreads();
      {   // nothing is in flight here: fetch the chunk's first tile
        const int e = __builtin_amdgcn_readfirstlane(lds_list[c * kListCap]);
        const int tok = (e >> 6) << 4;
        issue_loads(buf, tile_ptr(kg, tok, ks32), tile_ptr(vg, tok, vs32), (e & 63) + 1);
      }
    }

    // ---- epilogue: normalise, convert, store (rows with no visible key store exact zeros)
    if (active) {
      int hq, my_r;   // this lane's query (lanes l32 >= nrows repeat the last one and store nothing)
      slot_entry(slot, l32, rows, hq, my_r);
      const float l_tot = half_sum(l_run);
      const float inv = l_tot > 0.f ? __builtin_amdgcn_rcpf(l_tot) : 0.f;   // 1 ulp; a full division is ten instructions
      if (EXTRAS && p.nparts > 1) {
        // split over key blocks: this part's normalised result and log-sum-exp, for the merge kernel
        if (l32 < nrows) {
          const int64_t rh = ((int64_t)cur_part * p.total_q + (row_begin + my_r)) * p.nhead_q + hq;
          if (g32 == 0)
            p.part_lse[rh] = l_tot > 0.f ? (m_run * sm_c + __builtin_amdgcn_logf(l_tot)) * 0.69314718055994531f : -INFINITY;
          float *dst = p.part_out + rh * D;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
              f32x4 w = {o[dt][4 * i4 + 0] * inv, o[dt][4 * i4 + 1] * inv, o[dt][4 * i4 + 2] * inv, o[dt][4 * i4 + 3] * inv};
              *(f32x4 *)(dst + dt * 32 + 8 * i4 + 4 * g32) = w;
            }
        }
      } else {
      if (EXTRAS && p.lse != nullptr && g32 == 0 && l32 < nrows) {
        // natural-log sum over the row's visible keys of exp(scale * q.k); m_run is the (possibly
        // lagging) reference maximum the row sum was accumulated under, which makes this exact
        const float lse = l_tot > 0.f ? (m_run * sm_c + __builtin_amdgcn_logf(l_tot)) * 0.69314718055994531f : -INFINITY;
        p.lse[(int64_t)(row_begin + my_r) * p.lse_s + (int64_t)hq * p.lse_h] = lse;
      }
      if constexpr (OUT32) {
        if (l32 < nrows) {
          char *orow = p.out + (int64_t)(row_begin + my_r) * p.o_s + (int64_t)hq * p.o_h;
          const float f = inv * sm_out_mul;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
              f32x4 w = {o[dt][4 * i4 + 0] * f, o[dt][4 * i4 + 1] * f, o[dt][4 * i4 + 2] * f, o[dt][4 * i4 + 3] * f};
              *(f32x4 *)(orow + (dt * 32 + 8 * i4 + 4 * g32) * 4) = w;
            }
        }
      } else {
        // A lane holds dims 8*i4 + 4*g32 .. +3 of row l32, per 32-dim block.  Two exchanges turn that
        // into 64 contiguous bytes of a row across four lanes, so that one store instruction covers
        // 16 rows instead of 32 and the memory system sees a quarter of the write requests:
        // lanes i and i+32 (same row) trade halves (16 contiguous bytes per lane), then lanes with
        // bit 4 clear / set (rows l and 16 + l) trade the two 16-dim halves of the block.
        const int l16 = lane & 15;
        int hq_x, r_x, hq_y, r_y;   // the slot's entries l16 and 16 + l16
        slot_entry(slot, l16, rows, hq_x, r_x);
        slot_entry(slot, 16 + l16, rows, hq_y, r_y);
        char *row_x = p.out + (int64_t)(row_begin + r_x) * p.o_s + (int64_t)hq_x * p.o_h + (lane & 16) * 2 + g32 * 16;
        char *row_y = PACK ? p.out + (int64_t)(row_begin + r_y) * p.o_s + (int64_t)hq_y * p.o_h + (lane & 16) * 2 + g32 * 16
                           : row_x + (int64_t)16 * p.o_s;   // (a row past the block's end is not stored)
        const bool st_x = l16 < nrows, st_y = 16 + l16 < nrows;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          u32x4 w[2];
#pragma unroll
          for (int m = 0; m < 2; ++m) {
            const uint32_t ax = E::pack2(o[dt][8 * m + 0] * inv, o[dt][8 * m + 1] * inv);
            const uint32_t ay = E::pack2(o[dt][8 * m + 2] * inv, o[dt][8 * m + 3] * inv);
            const uint32_t bx = E::pack2(o[dt][8 * m + 4] * inv, o[dt][8 * m + 5] * inv);
            const uint32_t by = E::pack2(o[dt][8 * m + 6] * inv, o[dt][8 * m + 7] * inv);
            const auto rx = __builtin_amdgcn_permlane32_swap(ax, bx, false, false);
            const auto ry = __builtin_amdgcn_permlane32_swap(ay, by, false, false);
            w[m] = u32x4{(uint32_t)rx[0], (uint32_t)ry[0], (uint32_t)rx[1], (uint32_t)ry[1]};
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const auto r = __builtin_amdgcn_permlane16_swap(w[0][j], w[1][j], false, false);
            w[0][j] = r[0];
            w[1][j] = r[1];
          }
          if (st_x) *(u32x4 *)(row_x + dt * 64) = w[0];
          if (st_y) *(u32x4 *)(row_y + dt * 64) = w[1];
        }
      }
      }
    }

    // ---- move on to the next item
    if (total == 0) {
      // No tile, hence no barrier since this item began: the next list may still be being written,
      // and nothing of the next item has been requested yet.
      w_next_lap = -1;   // (nor has its walk been given a start: it takes no part in the clock)
      __builtin_amdgcn_s_waitcnt(0x0F70);   // keeps "every fetch has arrived" true on every path
      __syncthreads();
      nxt_hk = hdr_word(c ^ 1, H_HK);
      if (nxt_hk >= 0) {
        if (hdr_word(c ^ 1, H_TOTAL) > 0) {
          const int e1 = __builtin_amdgcn_readfirstlane(lds_list[(c ^ 1) * kListCap]);
          const int tok = hdr_word(c ^ 1, H_KEY_BEGIN) + ((e1 >> 6) << 4);
          issue_loads(buf, tile_ptr(p.k + (int64_t)nxt_hk * p.k_h, tok, ks32), tile_ptr(p.v + (int64_t)nxt_hk * p.v_h, tok, vs32),
                      (e1 & 63) + 1);
        }
        load_q(nxt_hk, hdr_word(c ^ 1, H_SUB), hdr_word(c ^ 1, H_ROW_BEGIN), hdr_word(c ^ 1, H_ROWS));
      }
      __syncthreads();   // wave 0 rewrites this item's list next; every wave has read its header by now
    }
    if (nxt_hk < 0) break;
    c ^= 1;
  }
  leave();
}

// Split over key blocks: bit row copy `part` keeps the k blocks [part * n / nparts, (part + 1) * n / nparts)
// of a q block's own sequence (n = its k blocks).
__global__ __launch_bounds__(256) void hbsa_split_bits_kernel(const uint32_t *bits, uint32_t *out, const QBlockInfo *info,
                                                              int nhead_k, int nqb, int wpr, int nparts) {
  const int64_t per_part = (int64_t)nhead_k * nqb * wpr;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= per_part * nparts) return;
  const int part = (int)(i / per_part);
  const int64_t r = i % per_part;
  const int w = (int)(r % wpr), qb = (int)((r / wpr) % nqb);
  const int n = info[qb].nkblk;
  const int lo = (int)((int64_t)part * n / nparts), hi = (int)((int64_t)(part + 1) * n / nparts);
  uint32_t m = 0;
  for (int b = 0; b < 32; ++b) {
    const int j = w * 32 + b;
    if (j >= lo && j < hi) m |= 1u << b;
  }
  out[i] = bits[r] & m;
}

// out[row, head, :] = sum over parts of exp(lse_part - lse) * partial, lse = log sum exp(lse_part);
// rows whose parts all saw no key give 0 (and lse -inf).  One thread per 4 output elements.
template <typename E, bool OUT32>
__global__ __launch_bounds__(256) void hbsa_merge_kernel(const float *part_out, const float *part_lse, char *out, float *lse,
                                                         const Sched *sched, int nparts, int total_q, int nhead_q, int dshift,
                                                         int64_t o_s, int64_t o_h, int64_t lse_s, int64_t lse_h) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t rows = (int64_t)total_q * nhead_q;
  if (i >= rows << dshift) return;
  const int64_t rh = i >> dshift;
  const int dq = (int)(i & ((1 << dshift) - 1));
  float mx = -INFINITY;
  for (int pt = 0; pt < nparts; ++pt) mx = fmaxf(mx, part_lse[pt * rows + rh]);
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float den = 0.f;
  if (mx != -INFINITY) {
    for (int pt = 0; pt < nparts; ++pt) {
      const float l = part_lse[pt * rows + rh];
      if (l == -INFINITY) continue;
      const float w = __expf(l - mx);
      den += w;
      acc += *(const f32x4 *)(part_out + (((int64_t)pt * rows + rh) << (dshift + 2)) + dq * 4) * w;
    }
    acc *= 1.f / den;
  }
  const int64_t row = rh / nhead_q, h = rh % nhead_q;
  if (lse != nullptr && dq == 0) lse[row * lse_s + h * lse_h] = mx == -INFINITY ? -INFINITY : mx + __logf(den);
  char *dst = out + row * o_s + h * o_h;
  if constexpr (OUT32) {
    acc *= sched->out_mul;
    *(f32x4 *)(dst + dq * 16) = acc;
  } else {
    u32x2 w;
    w.x = E::pack2(acc[0], acc[1]);
    w.y = E::pack2(acc[2], acc[3]);
    *(u32x2 *)(dst + dq * 8) = w;
  }
}

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
inline int words_per_row(int num_k_block) { return 2 * ((num_k_block + 63) / 64); }
// workspace layout: QBlockInfo[num_q_block] | Sched | walk clocks [nhead_k, num_q_block] | bit words
inline size_t sched_offset(int num_q_block) { return align_up((size_t)num_q_block * sizeof(QBlockInfo), 256); }
inline size_t clock_offset(int num_q_block) { return sched_offset(num_q_block) + align_up(sizeof(Sched), 256); }
inline size_t bits_offset(int nhead_k, int num_q_block) {
  return clock_offset(num_q_block) + align_up((size_t)nhead_k * num_q_block * sizeof(unsigned long long), 256);
}

// Deterministic mode (the default, like the reference's ascending scan): every item walks its tiles in
// ascending order, so results are bitwise reproducible.  With it switched off (hbsa_set_deterministic(0) or
// the environment variable HBSATTN_AMD_DETERMINISTIC=0) very large problems use the clocked walk, and
// results then vary in their last bits from run to run.
int g_deterministic = [] {
  const char *e = std::getenv("HBSATTN_AMD_DETERMINISTIC");
  return e != nullptr && e[0] == '0' && e[1] == 0 ? 0 : 1;
}();
// K + V bytes of one kv head from which the clocked walk is used.  Measured on MI355X: at 64K-token
// sequences with 30 % of the blocks kept the walk takes a seventh off the HBM traffic and 5 % off the
// time; at 32K tokens and 10 % kept it takes 6 % off the traffic and nothing off the time.
long long g_walk_min_bytes = 192ll << 20;

// rows must be 16-byte aligned: strides (in elements) multiples of 8 for 16-bit types, of 4 for fp32
int check_strides(const int64_t *strides, bool f32) {
  const int unit = f32 ? 4 : 8;
  for (int i = 0; i < 8; ++i)
    if (strides[i] % unit != 0)
      return fail(HBSA_ERR_INVALID_ARGUMENT, "stride %d (%lld elements) is not a multiple of %d (16-byte rows)", i,
                  (long long)strides[i], unit);
  // 16-bit inputs: the tile loads address a 64-row tile with 32-bit byte offsets from its first row
  if (strides[2] < 0 || strides[4] < 0 || strides[2] > (1 << 24) || strides[4] > (1 << 24))
    return fail(HBSA_ERR_UNSUPPORTED, "k/v token stride (%lld, %lld elements) outside [0, 2^24]", (long long)strides[2],
                (long long)strides[4]);
  return 0;
}

// fp32 inputs: bytes of one fp16 staging copy [tokens, heads, D], placed after the bit words
inline size_t f32_stage_bytes(int64_t tokens, int64_t heads, int64_t d) { return align_up((size_t)(tokens * heads * d * 2), 256); }

// tensor i (0 q, 1 k, 2 v) of an fp32 call
F32Tensor f32_tensor(int i, const void *q, const void *k, const void *v, const int64_t *strides, int total_q, int total_k,
                     int nhead_q, int nhead_k, int headdim) {
  const int dshift = headdim == 32 ? 3 : headdim == 64 ? 4 : headdim == 128 ? 5 : 6;
  const void *x = i == 0 ? q : i == 1 ? k : v;
  const int64_t tokens = i == 0 ? total_q : total_k;
  const int heads = i == 0 ? nhead_q : nhead_k;
  return {(const float *)x, strides[2 * i], strides[2 * i + 1], heads, dshift, tokens * heads * headdim / 4};
}

// Wave slots of an item: 32-row slices of one q head after another, or (the one-launch form, when a q block
// is no whole number of slices and a kv head serves several q heads) packed across the q heads of the group.
inline bool fwd_packs(int ratio, int q_block_size) { return ratio > 1 && q_block_size % kWaveRows != 0; }
inline int fwd_slots(int ratio, int q_block_size, bool packed) {
  return packed ? (ratio * q_block_size + kWaveRows - 1) / kWaveRows : ratio * ((q_block_size + kWaveRows - 1) / kWaveRows);
}
// Wavefronts per workgroup of the 16-bit attention kernel for an item of `slots` wave slots: eight when the
// item has more than four slots, so that one workgroup stages its K/V tiles once (head dims 64 and 128; the
// fp32 kernel always has four), unless the item's last workgroup of eight would be at most half full: then
// workgroups of four, none of them with idle wavefronts (measured at 20 slots, head dim 64: 0.365 -> 0.33 ms).
inline int fwd_wavefronts(int slots, int headdim, bool f32_exact) {
  if (f32_exact || slots <= 4 || headdim < 64 || headdim > 128) return 4;
  const int in_last = slots % 8;
  return (in_last >= 1 && in_last <= 4) ? 4 : 8;
}

// Split over key blocks pays when the work items cannot fill the device: fewer than one per CU.
// Returns the number of parts (1 = no split) for the current device.
int split_parts(long long items, int num_k_block) {
  static thread_local int cus_of[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 1;
  if (cus_of[dev] == 0 && hipDeviceGetAttribute(&cus_of[dev], hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    return 1;
  const int cus = cus_of[dev];
  if (items <= 0 || items > cus) return 1;
  long long parts = std::min<long long>(32, (2LL * cus) / items);
  parts = std::min<long long>(parts, num_k_block / 8);     // a part should still have a few k blocks
  return parts < 2 ? 1 : (int)parts;
}
// split area: nparts bit row copies | nparts partial outputs | nparts partial log-sum-exps, each array packed
inline size_t split_bits_bytes(int parts, int nhead_k, int num_q_block, int num_k_block) {
  return align_up((size_t)parts * nhead_k * num_q_block * words_per_row(num_k_block) * sizeof(uint32_t), 256);
}
inline size_t split_out_bytes(int parts, int total_q, int nhead_q, int headdim) {
  return align_up((size_t)parts * total_q * nhead_q * headdim * 4, 256);
}
inline size_t split_bytes(int parts, int total_q, int nhead_q, int nhead_k, int headdim, int num_q_block, int num_k_block) {
  if (parts < 2) return 0;
  return split_bits_bytes(parts, nhead_k, num_q_block, num_k_block) + split_out_bytes(parts, total_q, nhead_q, headdim) +
         align_up((size_t)parts * total_q * nhead_q * 4, 256);
}

int persistent_grid(const void *kernel, int lds_bytes, int threads) {
  int dev = 0, cus = 0, per_cu = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, lds_bytes) != hipSuccess) return 0;
  if (per_cu < 1) return 0;
  if (per_cu > 4) per_cu = 4;
  return cus * per_cu;
}

// The fields of FwdParams that follow from the call's shape and softmax_scale alone.
void fill_shape(FwdParams &fp, int nhead_q, int nhead_k, int headdim, int num_q_block, int num_k_block, int q_block_size,
                int k_block_size, int causal, float softmax_scale, bool f32_exact, bool may_pack = false) {
  fp.nhead_k = nhead_k;
  fp.nqb = num_q_block; fp.ratio = nhead_q / nhead_k; fp.kbs = k_block_size; fp.wpr = words_per_row(num_k_block);
  fp.causal = causal ? 1 : 0;
  fp.wps = (q_block_size + kWaveRows - 1) / kWaveRows;
  fp.pack = may_pack && fwd_packs(fp.ratio, q_block_size) ? 1 : 0;
  const int slots = fwd_slots(fp.ratio, q_block_size, fp.pack != 0);
  fp.nw = fwd_wavefronts(slots, headdim, f32_exact);
  fp.nsub = (slots + fp.nw - 1) / fp.nw;
  fp.div_nsub = make_fast_div((uint32_t)fp.nsub);
  fp.div_nqb = make_fast_div((uint32_t)num_q_block);
  fp.div_nhk = make_fast_div((uint32_t)nhead_k);
  fp.div_kbs = make_fast_div((uint32_t)k_block_size);
  fp.q_sign = softmax_scale < 0.f ? 0x80008000u : 0u;
  float c = std::fabs(softmax_scale) * kLog2e;
  if (c < 1e-30f) c = 1e-30f;  // scale 0: uniform weights over the visible keys, and -inf * c stays -inf
  fp.c = c;
  fp.lag = kLazyRescaleLog2 / c;
}

template <int D, typename E, bool OUT32, int NW, bool EXTRAS, bool FUSED = false, bool PACK = false>
int launch_fwd_nw(const FwdParams &fp, long long items, hipStream_t stream) {
  constexpr int lds_bytes = 4 * kTileKeys * D * 2 + 2 * H_WORDS * 4 + 2 * kListCap * 4 + (FUSED ? 4 * kSeqCap * 4 + kMaskStage : 0);
  const void *kernel = reinterpret_cast<const void *>(&hbsa_fwd_kernel<D, E, OUT32, NW, EXTRAS, FUSED, PACK>);
  // workgroups that fit the current device at once; the attribute and the occupancy are per device
  static thread_local int resident_of[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(HBSA_ERR_UNSUPPORTED, "no current device, or device index above %d", kMaxDevices - 1);
  int &resident = resident_of[dev];
  if (resident == 0) {
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    resident = persistent_grid(kernel, lds_bytes, NW * 64);
    if (resident <= 0) return fail(HBSA_ERR_UNSUPPORTED, "could not size the persistent grid");
  }
  const int grid = (int)(items < resident ? items : resident);
  FwdParams launch = fp;
  // Few items per workgroup: a fixed order instead of the per-XCD queues, whose round trips (and, with few kv
  // heads, the crowd at few counters) would be a good part of such a launch.
  launch.one_each = items <= (long long)kStaticShare * resident ? (int)items : 0;
  hipLaunchKernelGGL((hbsa_fwd_kernel<D, E, OUT32, NW, EXTRAS, FUSED, PACK>), dim3(grid), dim3(NW * 64), lds_bytes, stream, launch);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail((int)e, "hbsa_fwd_kernel launch: %s", hipGetErrorString(e));
  return 0;
}
template <int D, typename E, bool OUT32>
int launch_fwd(const FwdParams &fp, long long items, hipStream_t stream) {
  const bool extras = fp.walk != 0 || fp.nparts > 1 || fp.lse != nullptr;
  if constexpr (D >= 64 && D <= 128) {
    if (fp.nw == 8)
      return extras ? launch_fwd_nw<D, E, OUT32, 8, true>(fp, items, stream) : launch_fwd_nw<D, E, OUT32, 8, false>(fp, items, stream);
  }
  return extras ? launch_fwd_nw<D, E, OUT32, 4, true>(fp, items, stream) : launch_fwd_nw<D, E, OUT32, 4, false>(fp, items, stream);
}
// the one-launch form (16-bit tensors, none of the extras)
template <int D, typename E>
int launch_fwd_fused(const FwdParams &fp, long long items, hipStream_t stream) {
  if constexpr (D >= 64 && D <= 128) {
    if (fp.nw == 8)
      return fp.pack ? launch_fwd_nw<D, E, false, 8, false, true, true>(fp, items, stream)
                     : launch_fwd_nw<D, E, false, 8, false, true, false>(fp, items, stream);
  }
  return fp.pack ? launch_fwd_nw<D, E, false, 4, false, true, true>(fp, items, stream)
                 : launch_fwd_nw<D, E, false, 4, false, true, false>(fp, items, stream);
}


// --------------------------------------------------------------------------------------
// fp32 kernel: fp32 operands, fp32 MFMA (v_mfma_f32_32x32x2_f32), fp32 softmax and output, for
// callers that need the arithmetic of the reference's fp32 path (dot products without operand
// rounding, reference hbsattn/fwd_triton_auto_tile_size.py:205,225).  One workgroup per work item
// (kv head, q block, group of four wave slots), no persistence or prefetching: the fp32 matrix
// rate (a sixteenth of the bf16 one) bounds it, not the loads.
//
// Same operand roles as the 16-bit kernel: S^T = K.Q^T with K rows from LDS and Q^T in registers,
// O^T += V^T.P^T with P^T taken from the S^T accumulator in place.  A 32x32x2 MFMA contracts over
// two indices, one per half of the wavefront; which two is free as long as both operands agree:
//   S: step (j, e), half g contracts over d = 8*j + 4*g + e, so a lane reads 4 consecutive floats of
//      its K row per j (one ds_read_b128) and holds Q the same way;
//   PV: step i, half g contracts over key 8*(i/4) + 4*g + (i%4), which is exactly the key whose
//      score the lane holds in accumulator element i.
// LDS: K[64][D+4] and V[64][D+4] floats (the 4-float pad spreads the rows over the banks).
// --------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(kThreads, D > 128 ? 1 : 2) void hbsa_fwd_f32_kernel(FwdParams p, float c_signed) {
  constexpr int LD = D + 4;       // LDS row stride in floats
  constexpr int DJ = D / 8;       // ds_read_b128 steps of S
  constexpr int DT = D / 32;      // 32-row tiles of O^T
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  float *lds_k = (float *)lds_raw;
  float *lds_v = lds_k + kTileKeys * LD;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g32 = lane >> 5, l32 = lane & 31;

  // item: heaviest q blocks first, like the queues of the 16-bit kernel
  const uint32_t t = fast_div(blockIdx.x, p.div_nsub);
  const int sub = (int)(blockIdx.x - t * (uint32_t)p.nsub);
  const uint32_t hk_u = fast_div(t, p.div_nqb);
  const int hk = (int)hk_u;
  const int qb = p.nqb - 1 - (int)(t - hk_u * (uint32_t)p.nqb);
  const QBlockInfo inf = p.info[qb];

  const int slot = sub * 4 + wave;
  const int head_in_group = slot / p.wps;
  const int row0 = (slot % p.wps) * kWaveRows;
  const int nrows = min(kWaveRows, inf.rows - row0);
  const bool active = head_in_group < p.ratio && nrows > 0;
  const int hq = hk * p.ratio + head_in_group;

  // Q^T fragments, pre-multiplied by softmax_scale * log2(e): scores come out in log2 units
  f32x4 qf[DJ];
  {
    const int r = min(row0 + l32, inf.rows - 1);
    const char *qrow = p.q + (int64_t)(inf.row_begin + r) * p.q_s + (int64_t)hq * p.q_h;
#pragma unroll
    for (int j = 0; j < DJ; ++j) {
      f32x4 x = {0.f, 0.f, 0.f, 0.f};
      if (active) x = *(const f32x4 *)(qrow + (8 * j + 4 * g32) * 4);
      qf[j] = x * c_signed;
    }
  }
  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const int lane_kvis = inf.q_pos + min(row0 + l32, inf.rows - 1) + inf.shift;   // last key position this query sees
  const int wave_kvis_max = inf.q_pos + row0 + nrows - 1 + inf.shift;
  const char *kg = p.k + (int64_t)hk * p.k_h + (int64_t)inf.key_begin * p.k_s;
  const char *vg = p.v + (int64_t)hk * p.v_h + (int64_t)inf.key_begin * p.v_s;
  const uint32_t *bits = p.bits + ((size_t)hk * p.nqb + qb) * p.wpr;
  const int nwords = inf.kmax > 0 ? (inf.nkblk + 31) >> 5 : 0;

  for (int w = 0; w < nwords; ++w) {
    uint32_t word = (uint32_t)__builtin_amdgcn_readfirstlane((int)bits[w]);
    while (word != 0) {
      const int j = w * 32 + __builtin_ctz(word);
      word &= word - 1;
      const int end = min(min((j + 1) * p.kbs, inf.klen), inf.kmax);
      for (int pos = j * p.kbs; pos < end; pos += kTileKeys) {   // ---- one tile of up to 64 keys
        const int valid = min(kTileKeys, end - pos);
        __syncthreads();   // the previous tile has been consumed
        for (int idx = threadIdx.x; idx < kTileKeys * (D / 4); idx += kThreads) {
          const int r = idx / (D / 4), c4 = idx % (D / 4);
          const int64_t tok = pos + min(r, valid - 1);   // rows past the end repeat the last one (masked below)
          *(f32x4 *)(lds_k + r * LD + c4 * 4) = *(const f32x4 *)(kg + tok * p.k_s + c4 * 16);
          *(f32x4 *)(lds_v + r * LD + c4 * 4) = *(const f32x4 *)(vg + tok * p.v_s + c4 * 16);
        }
        __syncthreads();
        if (!active || (p.causal && pos > wave_kvis_max)) continue;
#pragma unroll
        for (int h = 0; h < 2; ++h) {   // ---- 32 keys at a time
          if (32 * h >= valid || (p.causal && pos + 32 * h > wave_kvis_max)) continue;
          f32x16 sc;
#pragma unroll
          for (int i = 0; i < 16; ++i) sc[i] = 0.f;
          const float *krow = lds_k + (32 * h + l32) * LD + 4 * g32;
#pragma unroll
          for (int jj = 0; jj < DJ; ++jj) {
            const f32x4 kv = *(const f32x4 *)(krow + 8 * jj);
#pragma unroll
            for (int e = 0; e < 4; ++e) sc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[e], qf[jj][e], sc, 0, 0, 0);
          }
          int lim = valid - 32 * h;                                  // keys of this half below lim are visible
          if (p.causal) lim = min(lim, lane_kvis - pos - 32 * h + 1);
          float mx = -INFINITY;
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            if (8 * (i >> 2) + 4 * g32 + (i & 3) >= lim) sc[i] = -INFINITY;
            mx = fmaxf(mx, sc[i]);
          }
          mx = half_max(mx);
          // no branch on per-query values here: the MFMAs below need every lane
          const float m_new = fmaxf(m_run, mx);
          const float m_ref = m_new == -INFINITY ? 0.f : m_new;       // a query that has seen no key yet
          const float alpha = m_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run - m_ref);
          l_run *= alpha;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
          m_run = m_new;
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            sc[i] = __builtin_amdgcn_exp2f(sc[i] - m_ref);
            l_run += sc[i];
          }
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const float *vrow = lds_v + (32 * h + 8 * (i >> 2) + 4 * g32 + (i & 3)) * LD + l32;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) o[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[32 * dt], sc[i], o[dt], 0, 0, 0);
          }
        }
      }
    }
  }

  if (!active) return;
  const float l_tot = half_sum(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (l32 >= nrows) return;
  const int64_t row = inf.row_begin + row0 + l32;
  if (p.lse != nullptr && g32 == 0)
    p.lse[row * p.lse_s + (int64_t)hq * p.lse_h] =
        l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * 0.69314718055994531f : -INFINITY;
  char *orow = p.out + row * p.o_s + (int64_t)hq * p.o_h;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      f32x4 wv = {o[dt][4 * i4 + 0] * inv, o[dt][4 * i4 + 1] * inv, o[dt][4 * i4 + 2] * inv, o[dt][4 * i4 + 3] * inv};
      *(f32x4 *)(orow + (dt * 32 + 8 * i4 + 4 * g32) * 4) = wv;
    }
}

template <int D, typename E, bool OUT32>
int launch_fwd_split(FwdParams &fp, long long items, hipStream_t stream, char *area, int num_k_block, int total_q,
                     int nhead_q) {
  const int parts = fp.nparts;
  uint32_t *bit_copies = (uint32_t *)area;
  char *after_bits = area + split_bits_bytes(parts, fp.nhead_k, fp.nqb, num_k_block);
  fp.part_out = (float *)after_bits;
  fp.part_lse = (float *)(after_bits + split_out_bytes(parts, total_q, nhead_q, D));
  {
    const int64_t n = (int64_t)fp.nhead_k * fp.nqb * fp.wpr * parts;
    hipLaunchKernelGGL(hbsa_split_bits_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, fp.bits,
                       bit_copies, fp.info, fp.nhead_k, fp.nqb, fp.wpr, parts);
  }
  char *final_out = fp.out;
  float *final_lse = fp.lse;
  const int64_t o_s = fp.o_s, o_h = fp.o_h, lse_s = fp.lse_s, lse_h = fp.lse_h;
  const size_t rows = (size_t)total_q * nhead_q;
  fp.bits = bit_copies;
  int rc = launch_fwd<D, E, OUT32>(fp, items * parts, stream);
  if (rc != 0) return rc;
  constexpr int dshift = D == 32 ? 3 : D == 64 ? 4 : D == 128 ? 5 : 6;
  const int64_t n = (int64_t)rows << dshift;
  hipLaunchKernelGGL((hbsa_merge_kernel<E, OUT32>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, fp.part_out,
                     fp.part_lse, final_out, final_lse, fp.sched, parts, total_q, nhead_q, dshift, o_s, o_h, lse_s, lse_h);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail((int)e, "hbsa_merge_kernel launch: %s", hipGetErrorString(e));
  return 0;
}

template <int D, typename E, bool OUT32>
int run_fwd(FwdParams &fp, long long items, hipStream_t stream, char *split_area, int num_k_block) {
  if (fp.nparts > 1) return launch_fwd_split<D, E, OUT32>(fp, items, stream, split_area, num_k_block, fp.total_q, fp.nhead_q);
  return launch_fwd<D, E, OUT32>(fp, items, stream);
}

template <int D>
int launch_fwd_f32(const FwdParams &fp, float c_signed, long long items, hipStream_t stream) {
  constexpr int lds_bytes = 2 * kTileKeys * (D + 4) * 4;
  const void *kernel = reinterpret_cast<const void *>(&hbsa_fwd_f32_kernel<D>);
  static thread_local bool configured[kMaxDevices] = {};   // the attribute is per device
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(HBSA_ERR_UNSUPPORTED, "no current device, or device index above %d", kMaxDevices - 1);
  if (!configured[dev]) {
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    configured[dev] = true;
  }
  hipLaunchKernelGGL((hbsa_fwd_f32_kernel<D>), dim3((unsigned)items), dim3(kThreads), lds_bytes, stream, fp, c_signed);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail((int)e, "hbsa_fwd_f32_kernel launch: %s", hipGetErrorString(e));
  return 0;
}

}  // namespace

#include "hbsa_bwd.h"

// ---- Device memory inside the library.  In host code the name of a __device__ array is only a handle; its
// device address comes from hipGetSymbolAddress, once per device, and is what the kernels receive.  Every
// GPU the library runs on holds its own copy of each array at its own address until the process ends.
//
// scratch: the work description of hbsa_fwd_static (hbsa_fwd without a workspace argument).
// stream_sched: launch records (work-queue counters) of the one-launch form of hbsa_fwd, one per stream.  They
// are zero when the library is loaded and every attention launch leaves its record at zero, so a call needs
// no launch of its own to prepare one; calls on different streams use different records and may overlap.
static __device__ __align__(256) unsigned char scratch[HBSA_STATIC_SCRATCH_BYTES];
constexpr int kStreamSlots = 64;
static __device__ __align__(256) unsigned char stream_sched[kStreamSlots * sizeof(Sched)];
namespace {
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void **ptr) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail((int)e, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(HBSA_ERR_UNSUPPORTED, "device index above %d", kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) return fail(e != hipSuccess ? (int)e : HBSA_ERR_UNSUPPORTED, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}

// The launch record of `stream` on the current device, nullptr when there is none to give (no device, the
// lookup failed, or kStreamSlots other streams of this device have taken the records).
struct StreamSlots {
  char *base;
  int used;
  hipStream_t stream[kStreamSlots];
};
StreamSlots g_stream_slots[kMaxDevices] = {};
Sched *stream_sched_of(hipStream_t stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  StreamSlots &t = g_stream_slots[dev];
  if (t.base == nullptr) {
    void *p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(stream_sched)) != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      return nullptr;
    }
    t.base = (char *)p;
  }
  int i = 0;
  while (i < t.used && t.stream[i] != stream) ++i;
  if (i == t.used) {
    if (t.used == kStreamSlots) return nullptr;
    t.stream[t.used++] = stream;
  }
  return (Sched *)(t.base + (size_t)i * sizeof(Sched));
}

// The one-launch form of the forward is used when it applies (see hbsa_set_onepass in the header).
int g_onepass = [] {
  const char *e = std::getenv("HBSATTN_AMD_ONEPASS");
  return e != nullptr && e[0] == '0' && e[1] == 0 ? 0 : 1;
}();

// The launch record a call would use in the one-launch form, nullptr when the form does not apply to it.
Sched *onepass_record(int32_t dtype, int32_t batch, int32_t total_k, int32_t headdim, int32_t num_k_block, int32_t k_block_size,
                      int64_t mask_kblk_stride, long long items, hipStream_t st) {
  if (!g_onepass || (dtype != HBSA_DTYPE_BF16 && dtype != HBSA_DTYPE_F16)) return nullptr;
  if (mask_kblk_stride != 1 || batch < 1 || batch >= kSeqCap) return nullptr;
  if (items <= 0 || items > 0x7fffffffLL) return nullptr;
  if (split_parts(items, num_k_block) > 1) return nullptr;
  if (!g_deterministic && k_block_size % kTileKeys == 0 && 2ll * total_k * headdim * 2 >= g_walk_min_bytes) return nullptr;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &capturing) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  if (capturing != hipStreamCaptureStatusNone) return nullptr;
  return stream_sched_of(st);
}

constexpr int kNotOnePass = 0x7fffffff;   // try_onepass: the call has to take the two-launch path

// hbsa_fwd as ONE launch: the attention kernel's scheduler reads the sequence boundaries and the mask bytes
// itself.  Arguments are those of hbsa_fwd, already validated.  Returns kNotOnePass when the form does not
// apply: fp32 tensors, a mask whose k block stride is not 1, more than kSeqCap - 1 sequences, work that
// would be split over key blocks or walk by the clock, a stream that is being captured into a graph (the
// graph could be replayed on any stream, while the launch record belongs to this one), no launch record left.
int try_onepass(const void *q, const void *k, const void *v, void *out, const int32_t *cu_q_seqlens,
                const int32_t *cu_k_seqlens, const uint8_t *block_mask, const int32_t *cu_num_q_block,
                const int32_t *cu_num_k_block, int32_t dtype, int32_t batch, int32_t total_q, int32_t total_k, int32_t nhead_q,
                int32_t nhead_k, int32_t headdim, int32_t num_q_block, int32_t num_k_block, int32_t q_block_size,
                int32_t k_block_size, int32_t causal, float softmax_scale, const int64_t *strides, hipStream_t st) {
  FwdParams fp;
  std::memset(&fp, 0, sizeof(fp));
  fill_shape(fp, nhead_q, nhead_k, headdim, num_q_block, num_k_block, q_block_size, k_block_size, causal, softmax_scale, false,
             true);
  const long long items = (long long)nhead_k * num_q_block * fp.nsub;
  Sched *sched = onepass_record(dtype, batch, total_k, headdim, num_k_block, k_block_size, strides[10], items, st);
  if (sched == nullptr) return kNotOnePass;

  fp.q = (const char *)q; fp.k = (const char *)k; fp.v = (const char *)v; fp.out = (char *)out;
  fp.sched = sched;
  fp.q_s = strides[0] * 2; fp.q_h = strides[1] * 2; fp.k_s = strides[2] * 2; fp.k_h = strides[3] * 2;
  fp.v_s = strides[4] * 2; fp.v_h = strides[5] * 2; fp.o_s = strides[6] * 2; fp.o_h = strides[7] * 2;
  fp.nparts = 1;
  fp.div_nparts = make_fast_div(1u);
  fp.total_q = total_q; fp.nhead_q = nhead_q;
  fp.cu_q = cu_q_seqlens; fp.cu_k = cu_k_seqlens; fp.cu_nqb = cu_num_q_block; fp.cu_nkb = cu_num_k_block;
  fp.mask = block_mask; fp.ms_h = strides[8]; fp.ms_q = strides[9];
  fp.batch = batch; fp.nkb_total = num_k_block; fp.total_k = total_k; fp.qbs = q_block_size;
  const bool bf = dtype == HBSA_DTYPE_BF16;
  switch (headdim) {
    case 32: return bf ? launch_fwd_fused<32, ElemBF16>(fp, items, st) : launch_fwd_fused<32, ElemF16>(fp, items, st);
    case 64: return bf ? launch_fwd_fused<64, ElemBF16>(fp, items, st) : launch_fwd_fused<64, ElemF16>(fp, items, st);
    case 128: return bf ? launch_fwd_fused<128, ElemBF16>(fp, items, st) : launch_fwd_fused<128, ElemF16>(fp, items, st);
    default: return bf ? launch_fwd_fused<256, ElemBF16>(fp, items, st) : launch_fwd_fused<256, ElemF16>(fp, items, st);
  }
}
}  // namespace

extern "C" {

int hbsa_abi_version(void) { return HBSA_ABI_VERSION; }

int hbsa_set_deterministic(int on) {
  const int previous = g_deterministic;
  g_deterministic = on ? 1 : 0;
  return previous;
}

int hbsa_fwd_launches(int32_t dtype, int32_t batch, int32_t total_k, int32_t nhead_q, int32_t nhead_k, int32_t headdim,
                      int32_t num_q_block, int32_t num_k_block, int32_t q_block_size, int32_t k_block_size,
                      int64_t mask_kblk_stride, void *stream) {
  if (nhead_k <= 0 || nhead_q <= 0 || nhead_q % nhead_k != 0 || num_q_block <= 0 || num_k_block <= 0 || q_block_size <= 0 ||
      k_block_size <= 0 || (headdim != 32 && headdim != 64 && headdim != 128 && headdim != 256))
    return 2;
  const int slots = fwd_slots(nhead_q / nhead_k, q_block_size, fwd_packs(nhead_q / nhead_k, q_block_size));   // as try_onepass
  const int nw = fwd_wavefronts(slots, headdim, false);
  const long long items = (long long)nhead_k * num_q_block * ((slots + nw - 1) / nw);
  return onepass_record(dtype, batch, total_k, headdim, num_k_block, k_block_size, mask_kblk_stride, items,
                        (hipStream_t)stream) != nullptr ? 1 : 2;
}

int hbsa_set_onepass(int on) {
  const int previous = g_onepass;
  g_onepass = on ? 1 : 0;
  return previous;
}

long long hbsa_set_walk_min_bytes(long long bytes) {
  const long long previous = g_walk_min_bytes;
  if (bytes >= 0) g_walk_min_bytes = bytes;
  return previous;
}

const char *hbsa_last_error(void) { return g_err; }

int hbsa_calculate_blocks(const int32_t *cu_seqlen, int32_t batch, int32_t block_size, int32_t *num_block,
                          int32_t *cu_num_block, int32_t *cu_block, int32_t *block_to_batch, int32_t capacity) {
  g_err[0] = 0;
  if (!cu_seqlen || !num_block || batch < 0) return fail(HBSA_ERR_INVALID_ARGUMENT, "null pointer or negative batch");
  if (block_size <= 0) return fail(HBSA_ERR_INVALID_ARGUMENT, "block_size must be positive");
  int64_t total = 0;
  if (cu_num_block) cu_num_block[0] = 0;
  for (int b = 0; b < batch; ++b) {
    const int64_t len = (int64_t)cu_seqlen[b + 1] - cu_seqlen[b];
    if (len < 0) return fail(HBSA_ERR_INVALID_ARGUMENT, "cu_seqlen decreases at sequence %d", b);
    total += (len + block_size - 1) / block_size;
    if (total > 0x7fffffff) return fail(HBSA_ERR_UNSUPPORTED, "more than 2^31 - 1 blocks");
    if (cu_num_block) cu_num_block[b + 1] = (int32_t)total;
  }
  *num_block = (int32_t)total;
  if (!cu_block && !block_to_batch) return 0;
  if (capacity < total) return fail(HBSA_ERR_WORKSPACE_TOO_SMALL, "capacity %d < %lld blocks", capacity, (long long)total);
  int32_t j = 0;
  if (cu_block) cu_block[0] = 0;
  for (int b = 0; b < batch; ++b)
    for (int64_t start = cu_seqlen[b]; start < cu_seqlen[b + 1]; start += block_size, ++j) {
      if (block_to_batch) block_to_batch[j] = b;
      if (cu_block) cu_block[j + 1] = (int32_t)std::min<int64_t>(start + block_size, cu_seqlen[b + 1]);
    }
  return 0;
}

size_t hbsa_fwd_workspace_bytes(int32_t nhead_k, int32_t num_q_block, int32_t num_k_block) {
  if (nhead_k <= 0 || num_q_block <= 0 || num_k_block <= 0) return 256;
  const size_t bits = align_up((size_t)nhead_k * num_q_block * words_per_row(num_k_block) * sizeof(uint32_t), 256);
  return bits_offset(nhead_k, num_q_block) + bits;
}

size_t hbsa_fwd_workspace_bytes_dtype(int32_t dtype, int32_t total_q, int32_t total_k, int32_t nhead_q,
                                      int32_t nhead_k, int32_t headdim, int32_t num_q_block, int32_t num_k_block) {
  size_t n = hbsa_fwd_workspace_bytes(nhead_k, num_q_block, num_k_block);
  if (dtype == HBSA_DTYPE_F32_STAGED16 && total_q > 0 && total_k > 0 && nhead_q > 0 && nhead_k > 0 && headdim > 0)
    n += f32_stage_bytes(total_q, nhead_q, headdim) + 2 * f32_stage_bytes(total_k, nhead_k, headdim);
  return n;
}

size_t hbsa_fwd_split_workspace_bytes(int32_t total_q, int32_t nhead_q, int32_t nhead_k, int32_t headdim,
                                      int32_t num_q_block, int32_t num_k_block, int32_t q_block_size) {
  if (total_q <= 0 || nhead_q <= 0 || nhead_k <= 0 || headdim <= 0 || num_q_block <= 0 || num_k_block <= 0 || q_block_size <= 0)
    return 0;
  const int slots = fwd_slots(nhead_q / nhead_k, q_block_size, false);
  const int nw = fwd_wavefronts(slots, headdim, false);
  const long long items = (long long)nhead_k * num_q_block * ((slots + nw - 1) / nw);
  return split_bytes(split_parts(items, num_k_block), total_q, nhead_q, nhead_k, headdim, num_q_block, num_k_block);
}

int hbsa_fwd_prepare(const int32_t *cu_q_seqlens, const int32_t *cu_k_seqlens, const uint8_t *block_mask,
                     const int32_t *q_block_to_batch, const int32_t *cu_num_q_block, const int32_t *cu_num_k_block,
                     void *workspace, size_t workspace_bytes, int32_t batch, int32_t nhead_k, int32_t num_q_block,
                     int32_t num_k_block, int32_t q_block_size, int32_t k_block_size, int32_t causal,
                     int32_t total_q, int32_t total_k, const int64_t *mask_strides, void *stream) {
  g_err[0] = 0;
  if (batch < 0 || num_q_block < 0 || num_k_block < 0 || total_q < 0 || total_k < 0)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "negative size");
  if (num_q_block == 0) return 0;
  if (!cu_q_seqlens || !cu_k_seqlens || !block_mask || !q_block_to_batch || !cu_num_q_block || !cu_num_k_block ||
      !workspace || !mask_strides)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "null pointer argument");
  if (nhead_k <= 0) return fail(HBSA_ERR_INVALID_ARGUMENT, "nhead_k must be positive");
  if (q_block_size <= 0 || k_block_size <= 0 || q_block_size % 16 || k_block_size % 16)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "q_block_size (%d) and k_block_size (%d) must be positive multiples of 16",
                q_block_size, k_block_size);
  if (num_k_block <= 0) return fail(HBSA_ERR_INVALID_ARGUMENT, "no keys");
  if (nhead_k > 65535) return fail(HBSA_ERR_UNSUPPORTED, "nhead_k %d > 65535", nhead_k);
  if ((uintptr_t)workspace & 255) return fail(HBSA_ERR_INVALID_ARGUMENT, "workspace must be 256-byte aligned");
  const size_t need = hbsa_fwd_workspace_bytes(nhead_k, num_q_block, num_k_block);
  if (workspace_bytes < need)
    return fail(HBSA_ERR_WORKSPACE_TOO_SMALL, "workspace %zu bytes < required %zu", workspace_bytes, need);

  PrepParams pp;
  pp.cu_q = cu_q_seqlens; pp.cu_k = cu_k_seqlens; pp.q_block_to_batch = q_block_to_batch;
  pp.cu_num_q_block = cu_num_q_block; pp.cu_num_k_block = cu_num_k_block;
  pp.mask = block_mask; pp.ms_h = mask_strides[0]; pp.ms_q = mask_strides[1]; pp.ms_k = mask_strides[2];
  pp.info = (QBlockInfo *)workspace;
  pp.bits = (uint32_t *)((char *)workspace + bits_offset(nhead_k, num_q_block));
  pp.sched = (Sched *)((char *)workspace + sched_offset(num_q_block));
  pp.clock = (unsigned long long *)((char *)workspace + clock_offset(num_q_block));
  pp.nqb = num_q_block; pp.qbs = q_block_size; pp.kbs = k_block_size; pp.wpr = words_per_row(num_k_block);
  pp.causal = causal ? 1 : 0;
  pp.batch = batch; pp.nkb = num_k_block; pp.total_q = total_q; pp.total_k = total_k;
  hipLaunchKernelGGL(hbsa_prep_kernel, dim3((num_q_block + 3) / 4, nhead_k), dim3(kThreads), 0, (hipStream_t)stream, pp);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail((int)e, "hbsa_prep_kernel launch: %s", hipGetErrorString(e));
  return 0;
}

int hbsa_fwd_run(const void *q, const void *k, const void *v, void *out, void *workspace, size_t workspace_bytes,
                 int32_t dtype, int32_t total_q, int32_t total_k, int32_t nhead_q, int32_t nhead_k, int32_t headdim,
                 int32_t num_q_block, int32_t num_k_block, int32_t q_block_size, int32_t k_block_size, int32_t causal,
                 float softmax_scale, const int64_t *strides, void *stream) {
  return hbsa_fwd_run_lse(q, k, v, out, nullptr, nullptr, workspace, workspace_bytes, dtype, total_q, total_k, nhead_q,
                          nhead_k, headdim, num_q_block, num_k_block, q_block_size, k_block_size, causal, softmax_scale,
                          strides, stream);
}

int hbsa_fwd_run_lse(const void *q, const void *k, const void *v, void *out, float *lse, const int64_t *lse_strides,
                     void *workspace, size_t workspace_bytes, int32_t dtype, int32_t total_q, int32_t total_k,
                     int32_t nhead_q, int32_t nhead_k, int32_t headdim, int32_t num_q_block, int32_t num_k_block,
                     int32_t q_block_size, int32_t k_block_size, int32_t causal, float softmax_scale,
                     const int64_t *strides, void *stream) {
  g_err[0] = 0;
  if (lse != nullptr && lse_strides == nullptr) return fail(HBSA_ERR_INVALID_ARGUMENT, "lse without lse_strides");
  if (total_q < 0 || total_k < 0) return fail(HBSA_ERR_INVALID_ARGUMENT, "negative size");
  if (total_q == 0 || num_q_block == 0 || nhead_q == 0) return 0;  // nothing to write
  if (!q || !k || !v || !out || !workspace || !strides) return fail(HBSA_ERR_INVALID_ARGUMENT, "null pointer argument");
  if (nhead_k <= 0 || nhead_q % nhead_k != 0)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "nhead_q (%d) must be divisible by nhead_k (%d)", nhead_q, nhead_k);
  if (q_block_size <= 0 || k_block_size <= 0 || q_block_size % 16 || k_block_size % 16)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "q_block_size (%d) and k_block_size (%d) must be positive multiples of 16",
                q_block_size, k_block_size);
  if (headdim != 32 && headdim != 64 && headdim != 128 && headdim != 256)
    return fail(HBSA_ERR_UNSUPPORTED, "headdim %d not in {32, 64, 128, 256}", headdim);
  if (dtype < HBSA_DTYPE_BF16 || dtype > HBSA_DTYPE_F32_STAGED16)
    return fail(HBSA_ERR_UNSUPPORTED, "dtype code %d not supported", dtype);
  if (num_k_block <= 0 || total_k <= 0) return fail(HBSA_ERR_INVALID_ARGUMENT, "no keys");
  if (!std::isfinite(softmax_scale)) return fail(HBSA_ERR_INVALID_ARGUMENT, "softmax_scale is not finite");
  const bool f32 = dtype == HBSA_DTYPE_F32_STAGED16;    // fp32 tensors staged as scaled fp16
  const bool f32_exact = dtype == HBSA_DTYPE_F32;       // fp32 tensors, fp32 MFMA
  if (int rc = check_strides(strides, f32 || f32_exact)) return rc;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "q/k/v/out must be 16-byte aligned");
  if ((uintptr_t)workspace & 255) return fail(HBSA_ERR_INVALID_ARGUMENT, "workspace must be 256-byte aligned");
  const size_t base = hbsa_fwd_workspace_bytes(nhead_k, num_q_block, num_k_block);
  const size_t need = hbsa_fwd_workspace_bytes_dtype(dtype, total_q, total_k, nhead_q, nhead_k, headdim, num_q_block,
                                                     num_k_block);
  if (workspace_bytes < need)
    return fail(HBSA_ERR_WORKSPACE_TOO_SMALL, "workspace %zu bytes < required %zu", workspace_bytes, need);

  hipStream_t st = (hipStream_t)stream;
  FwdParams fp;
  fp.q = (const char *)q; fp.k = (const char *)k; fp.v = (const char *)v; fp.out = (char *)out;
  fp.info = (const QBlockInfo *)workspace;
  fp.bits = (const uint32_t *)((const char *)workspace + bits_offset(nhead_k, num_q_block));
  fp.sched = (Sched *)((char *)workspace + sched_offset(num_q_block));
  fp.clock = (unsigned long long *)((char *)workspace + clock_offset(num_q_block));
  fp.nhead_k = nhead_k;
  fp.f32 = f32 ? 1 : 0;
  fp.lse = lse;
  fp.lse_s = lse ? lse_strides[0] : 0;
  fp.lse_h = lse ? lse_strides[1] : 0;
  if (f32) {
    // fp16 staging copies (contiguous) behind the bit words; the attention kernel reads those
    char *sq = (char *)workspace + base;
    char *sk = sq + f32_stage_bytes(total_q, nhead_q, headdim);
    char *sv = sk + f32_stage_bytes(total_k, nhead_k, headdim);
    hipLaunchKernelGGL(hbsa_f32_begin_kernel, dim3(1), dim3(64), 0, st, fp.sched);
    for (int i = 0; i < 3; ++i) {
      const F32Tensor t = f32_tensor(i, q, k, v, strides, total_q, total_k, nhead_q, nhead_k, headdim);
      const unsigned nb = (unsigned)std::min<int64_t>((t.quads + 255) / 256, 4096);
      hipLaunchKernelGGL(hbsa_f32_absmax_kernel, dim3(nb), dim3(256), 0, st, t, &fp.sched->amax[i]);
    }
    fp.q = sq; fp.k = sk; fp.v = sv;
    fp.q_s = (int64_t)nhead_q * headdim * 2; fp.q_h = headdim * 2;
    fp.k_s = (int64_t)nhead_k * headdim * 2; fp.k_h = headdim * 2;
    fp.v_s = fp.k_s; fp.v_h = fp.k_h;
    fp.o_s = strides[6] * 4; fp.o_h = strides[7] * 4;
  } else {
    const int64_t es = f32_exact ? 4 : 2;
    fp.q_s = strides[0] * es; fp.q_h = strides[1] * es; fp.k_s = strides[2] * es; fp.k_h = strides[3] * es;
    fp.v_s = strides[4] * es; fp.v_h = strides[5] * es; fp.o_s = strides[6] * es; fp.o_h = strides[7] * es;
  }
  fill_shape(fp, nhead_q, nhead_k, headdim, num_q_block, num_k_block, q_block_size, k_block_size, causal, softmax_scale,
             f32_exact);
  const long long items = (long long)nhead_k * num_q_block * fp.nsub;
  if (items > 0x7fffffffLL) return fail(HBSA_ERR_UNSUPPORTED, "too many work items (%lld)", items);
  // split over key blocks when the items cannot fill the device and the caller's workspace has the room
  fp.nparts = 1;
  fp.part_out = nullptr; fp.part_lse = nullptr;
  fp.total_q = total_q; fp.nhead_q = nhead_q;
  char *split_area = (char *)workspace + need;
  if (!f32_exact) {
    const int parts = split_parts(items, num_k_block);
    if (parts > 1 && workspace_bytes >= need + split_bytes(parts, total_q, nhead_q, nhead_k, headdim, num_q_block, num_k_block))
      fp.nparts = parts;
  }
  fp.div_nparts = make_fast_div((uint32_t)fp.nparts);
  // the clocked walk: block sizes that are whole tiles, work that is not split, K/V of a head beyond what an L2 holds
  fp.walk = (!g_deterministic && fp.nparts == 1 && k_block_size % kTileKeys == 0 &&
             2ll * total_k * headdim * 2 >= g_walk_min_bytes) ? 1 : 0;

  if (f32_exact) {
    const float c_signed = softmax_scale * kLog2e;
    switch (headdim) {
      case 32: return launch_fwd_f32<32>(fp, c_signed, items, st);
      case 64: return launch_fwd_f32<64>(fp, c_signed, items, st);
      case 128: return launch_fwd_f32<128>(fp, c_signed, items, st);
      default: return launch_fwd_f32<256>(fp, c_signed, items, st);
    }
  }
  if (f32) {
    // setup (multipliers from the maxima), staging, attention: the launch order on the stream is the
    // dependency order
    hipLaunchKernelGGL(hbsa_setup_kernel, dim3(1), dim3(64), 0, st, fp.sched, fp.c, 1);
    const char *dst[3] = {fp.q, fp.k, fp.v};
    for (int i = 0; i < 3; ++i) {
      const F32Tensor t = f32_tensor(i, q, k, v, strides, total_q, total_k, nhead_q, nhead_k, headdim);
      const unsigned nb = (unsigned)std::min<int64_t>((t.quads + 255) / 256, 8192);
      hipLaunchKernelGGL(hbsa_f32_stage_kernel, dim3(nb), dim3(256), 0, st, t, &fp.sched->in_mul[i], (uint32_t *)dst[i]);
    }
    switch (headdim) {
      case 32: return run_fwd<32, ElemF16, true>(fp, items, st, split_area, num_k_block);
      case 64: return run_fwd<64, ElemF16, true>(fp, items, st, split_area, num_k_block);
      case 128: return run_fwd<128, ElemF16, true>(fp, items, st, split_area, num_k_block);
      default: return run_fwd<256, ElemF16, true>(fp, items, st, split_area, num_k_block);
    }
  }
  const bool bf = dtype == HBSA_DTYPE_BF16;
  switch (headdim) {
    case 32: return bf ? run_fwd<32, ElemBF16, false>(fp, items, st, split_area, num_k_block)
                       : run_fwd<32, ElemF16, false>(fp, items, st, split_area, num_k_block);
    case 64: return bf ? run_fwd<64, ElemBF16, false>(fp, items, st, split_area, num_k_block)
                       : run_fwd<64, ElemF16, false>(fp, items, st, split_area, num_k_block);
    case 128: return bf ? run_fwd<128, ElemBF16, false>(fp, items, st, split_area, num_k_block)
                        : run_fwd<128, ElemF16, false>(fp, items, st, split_area, num_k_block);
    default: return bf ? run_fwd<256, ElemBF16, false>(fp, items, st, split_area, num_k_block)
                       : run_fwd<256, ElemF16, false>(fp, items, st, split_area, num_k_block);
  }
}

}  // extern "C"
namespace {
// hbsa_fwd, with the one-launch form allowed or not
int fwd_call(const void *q, const void *k, const void *v, void *out, const int32_t *cu_q_seqlens,
             const int32_t *cu_k_seqlens, const uint8_t *block_mask, const int32_t *q_block_to_batch,
             const int32_t *cu_num_q_block, const int32_t *cu_num_k_block, void *workspace,
             size_t workspace_bytes, int32_t dtype, int32_t batch, int32_t total_q, int32_t total_k,
             int32_t nhead_q, int32_t nhead_k, int32_t headdim, int32_t num_q_block, int32_t num_k_block,
             int32_t q_block_size, int32_t k_block_size, int32_t causal, float softmax_scale,
             const int64_t *strides, void *stream, bool allow_onepass) {
  g_err[0] = 0;
  if (total_q == 0 || num_q_block == 0 || nhead_q == 0) return 0;
  if (!strides) return fail(HBSA_ERR_INVALID_ARGUMENT, "null pointer argument");
  // Validate the main launch before queueing anything, so a refused call leaves no work behind.
  if (!q || !k || !v || !out) return fail(HBSA_ERR_INVALID_ARGUMENT, "null pointer argument");
  if (nhead_k <= 0 || nhead_q % nhead_k != 0)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "nhead_q (%d) must be divisible by nhead_k (%d)", nhead_q, nhead_k);
  if (headdim != 32 && headdim != 64 && headdim != 128 && headdim != 256)
    return fail(HBSA_ERR_UNSUPPORTED, "headdim %d not in {32, 64, 128, 256}", headdim);
  if (dtype < HBSA_DTYPE_BF16 || dtype > HBSA_DTYPE_F32_STAGED16)
    return fail(HBSA_ERR_UNSUPPORTED, "dtype code %d not supported", dtype);
  if (!std::isfinite(softmax_scale)) return fail(HBSA_ERR_INVALID_ARGUMENT, "softmax_scale is not finite");
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "q/k/v/out must be 16-byte aligned");
  if (int rc = check_strides(strides, dtype == HBSA_DTYPE_F32 || dtype == HBSA_DTYPE_F32_STAGED16)) return rc;
  if (batch < 0 || num_q_block < 0 || num_k_block < 0 || total_q < 0 || total_k < 0)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "negative size");
  if (!cu_q_seqlens || !cu_k_seqlens || !block_mask || !q_block_to_batch || !cu_num_q_block || !cu_num_k_block)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "null pointer argument");
  if (q_block_size <= 0 || k_block_size <= 0 || q_block_size % 16 || k_block_size % 16)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "q_block_size (%d) and k_block_size (%d) must be positive multiples of 16",
                q_block_size, k_block_size);
  if (num_k_block <= 0 || total_k <= 0) return fail(HBSA_ERR_INVALID_ARGUMENT, "no keys");
  if (nhead_k > 65535) return fail(HBSA_ERR_UNSUPPORTED, "nhead_k %d > 65535", nhead_k);
  if (allow_onepass) {
    const int one = try_onepass(q, k, v, out, cu_q_seqlens, cu_k_seqlens, block_mask, cu_num_q_block, cu_num_k_block, dtype,
                                batch, total_q, total_k, nhead_q, nhead_k, headdim, num_q_block, num_k_block, q_block_size,
                                k_block_size, causal, softmax_scale, strides, (hipStream_t)stream);
    if (one != kNotOnePass) return one;
  }
  {
    const size_t need = hbsa_fwd_workspace_bytes_dtype(dtype, total_q, total_k, nhead_q, nhead_k, headdim, num_q_block,
                                                       num_k_block);
    if (!workspace || workspace_bytes < need)
      return fail(HBSA_ERR_WORKSPACE_TOO_SMALL, "workspace %zu bytes < required %zu", workspace ? workspace_bytes : (size_t)0, need);
  }
  int rc = hbsa_fwd_prepare(cu_q_seqlens, cu_k_seqlens, block_mask, q_block_to_batch, cu_num_q_block, cu_num_k_block,
                            workspace, workspace_bytes, batch, nhead_k, num_q_block, num_k_block, q_block_size,
                            k_block_size, causal, total_q, total_k, strides + 8, stream);
  if (rc != 0) return rc;
  return hbsa_fwd_run(q, k, v, out, workspace, workspace_bytes, dtype, total_q, total_k, nhead_q, nhead_k, headdim,
                      num_q_block, num_k_block, q_block_size, k_block_size, causal, softmax_scale, strides, stream);
}
}  // namespace
extern "C" {

int hbsa_fwd(const void *q, const void *k, const void *v, void *out, const int32_t *cu_q_seqlens,
             const int32_t *cu_k_seqlens, const uint8_t *block_mask, const int32_t *q_block_to_batch,
             const int32_t *cu_num_q_block, const int32_t *cu_num_k_block, void *workspace,
             size_t workspace_bytes, int32_t dtype, int32_t batch, int32_t total_q, int32_t total_k,
             int32_t nhead_q, int32_t nhead_k, int32_t headdim, int32_t num_q_block, int32_t num_k_block,
             int32_t q_block_size, int32_t k_block_size, int32_t causal, float softmax_scale,
             const int64_t *strides, void *stream) {
  return fwd_call(q, k, v, out, cu_q_seqlens, cu_k_seqlens, block_mask, q_block_to_batch, cu_num_q_block, cu_num_k_block,
                  workspace, workspace_bytes, dtype, batch, total_q, total_k, nhead_q, nhead_k, headdim, num_q_block,
                  num_k_block, q_block_size, k_block_size, causal, softmax_scale, strides, stream, true);
}

int hbsa_fwd_v(const void *const *ptrs, size_t workspace_bytes, const int32_t *sizes, float softmax_scale,
               const int64_t *strides, void *stream) {
  if (!ptrs || !sizes) {
    g_err[0] = 0;
    return fail(HBSA_ERR_INVALID_ARGUMENT, "null pointer argument");
  }
  return fwd_call(ptrs[0], ptrs[1], ptrs[2], (void *)ptrs[3], (const int32_t *)ptrs[4], (const int32_t *)ptrs[5],
                  (const uint8_t *)ptrs[6], (const int32_t *)ptrs[7], (const int32_t *)ptrs[8], (const int32_t *)ptrs[9],
                  (void *)ptrs[10], workspace_bytes, sizes[0], sizes[1], sizes[2], sizes[3], sizes[4], sizes[5], sizes[6], sizes[7],
                  sizes[8], sizes[9], sizes[10], sizes[11], softmax_scale, strides, stream, true);
}

int hbsa_fwd_static(const void *q, const void *k, const void *v, void *out, const int32_t *cu_q_seqlens,
                    const int32_t *cu_k_seqlens, const uint8_t *block_mask, const int32_t *q_block_to_batch,
                    const int32_t *cu_num_q_block, const int32_t *cu_num_k_block, int32_t dtype, int32_t batch,
                    int32_t total_q, int32_t total_k, int32_t nhead_q, int32_t nhead_k, int32_t headdim,
                    int32_t num_q_block, int32_t num_k_block, int32_t q_block_size, int32_t k_block_size, int32_t causal,
                    float softmax_scale, const int64_t *strides, void *stream) {
  g_err[0] = 0;
  if (total_q == 0 || num_q_block == 0 || nhead_q == 0) return 0;
  const size_t need = hbsa_fwd_workspace_bytes_dtype(dtype, total_q, total_k, nhead_q, nhead_k, headdim, num_q_block,
                                                     num_k_block);
  if (need > (size_t)HBSA_STATIC_SCRATCH_BYTES)
    return fail(HBSA_ERR_WORKSPACE_TOO_SMALL,
                "this problem needs %zu bytes of scratch, hbsa_fwd_static holds %zu: use hbsa_fwd with a workspace", need,
                (size_t)HBSA_STATIC_SCRATCH_BYTES);
  void *ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // (always the pre-pass and the attention kernel on the static array: this form may be captured into a graph)
  return fwd_call(q, k, v, out, cu_q_seqlens, cu_k_seqlens, block_mask, q_block_to_batch, cu_num_q_block, cu_num_k_block, ws,
                  (size_t)HBSA_STATIC_SCRATCH_BYTES, dtype, batch, total_q, total_k, nhead_q, nhead_k, headdim, num_q_block,
                  num_k_block, q_block_size, k_block_size, causal, softmax_scale, strides, stream, false);
}

size_t hbsa_bwd_workspace_bytes(int32_t total_q, int32_t nhead_q) {
  if (total_q < 0 || nhead_q < 0) return 0;
  return 2 * align_up((size_t)total_q * nhead_q * sizeof(float), 256);   // delta and the scaled log-sum-exp of every (row, q head)
}

int hbsa_bwd(const void *q, const void *k, const void *v, const void *out, const void *dout, const float *lse, void *dq,
             void *dk, void *dv, const int32_t *cu_k_seqlens, const int32_t *cu_num_q_block, const int32_t *cu_num_k_block,
             const void *workspace, size_t workspace_bytes, void *bwd_workspace, size_t bwd_workspace_bytes, int32_t dtype,
             int32_t batch, int32_t total_q, int32_t total_k, int32_t nhead_q, int32_t nhead_k, int32_t headdim,
             int32_t num_q_block, int32_t num_k_block, int32_t q_block_size, int32_t k_block_size, int32_t causal,
             float softmax_scale, const int64_t *strides, void *stream) {
  g_err[0] = 0;
  if (!q || !k || !v || !out || !dout || !lse || !dq || !dk || !dv || !cu_k_seqlens || !cu_num_q_block || !cu_num_k_block ||
      !workspace || !bwd_workspace || !strides)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "null pointer argument");
  if (dtype != HBSA_DTYPE_BF16 && dtype != HBSA_DTYPE_F16)
    return fail(HBSA_ERR_UNSUPPORTED, "the backward takes bf16 or fp16 tensors (dtype code %d given)", dtype);
  if (headdim != 32 && headdim != 64 && headdim != 128) return fail(HBSA_ERR_UNSUPPORTED, "headdim %d not in {32, 64, 128}", headdim);
  if (batch <= 0 || total_q < 0 || total_k < 0 || nhead_q <= 0 || nhead_k <= 0 || nhead_q % nhead_k != 0 || num_q_block < 0 ||
      num_k_block < 0)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "bad sizes");
  if (q_block_size <= 0 || k_block_size <= 0 || q_block_size % 16 || k_block_size % 16)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "q_block_size and k_block_size must be positive multiples of 16");
  for (int i = 0; i < 16; ++i)
    if (strides[i] % 8 != 0)
      return fail(HBSA_ERR_INVALID_ARGUMENT, "stride %d (%lld elements) is not a multiple of 8 (16-byte rows)", i,
                  (long long)strides[i]);
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)dout | (uintptr_t)dq | (uintptr_t)dk |
       (uintptr_t)dv) & 15)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "q/k/v/out/dout/dq/dk/dv must be 16-byte aligned");
  if ((uintptr_t)workspace & 255) return fail(HBSA_ERR_INVALID_ARGUMENT, "workspace must be 256-byte aligned");
  if (workspace_bytes < hbsa_fwd_workspace_bytes(nhead_k, num_q_block, num_k_block))
    return fail(HBSA_ERR_WORKSPACE_TOO_SMALL, "workspace smaller than hbsa_fwd_workspace_bytes");
  if (((uintptr_t)bwd_workspace & 15) || bwd_workspace_bytes < hbsa_bwd_workspace_bytes(total_q, nhead_q))
    return fail(HBSA_ERR_WORKSPACE_TOO_SMALL, "bwd_workspace smaller than hbsa_bwd_workspace_bytes, or not 16-byte aligned");
  if (total_q == 0 || total_k == 0 || num_q_block == 0 || num_k_block == 0) return 0;
  // (the kernels address a tile's rows with 32-bit offsets from the tile's first row: K and V tiles in the dQ
  // kernel, Q and dO tiles in the dK/dV kernels)
  if (strides[2] < 0 || strides[4] < 0 || strides[2] > (1 << 24) || strides[4] > (1 << 24))
    return fail(HBSA_ERR_UNSUPPORTED, "k/v token stride (%lld, %lld elements) outside [0, 2^24]", (long long)strides[2],
                (long long)strides[4]);
  if (strides[0] < 0 || strides[8] < 0 || strides[0] > (1 << 24) || strides[8] > (1 << 24))
    return fail(HBSA_ERR_UNSUPPORTED, "q/dout token stride (%lld, %lld elements) outside [0, 2^24]", (long long)strides[0],
                (long long)strides[8]);

  const int es = 2;
  BwdParams bp;
  std::memset(&bp, 0, sizeof(bp));
  bp.q = (const char *)q; bp.k = (const char *)k; bp.v = (const char *)v; bp.out = (const char *)out; bp.dout = (const char *)dout;
  bp.dq = (char *)dq; bp.dk = (char *)dk; bp.dv = (char *)dv;
  bp.lse = lse; bp.delta = (float *)bwd_workspace;
  bp.lse2 = bp.delta + align_up((size_t)total_q * nhead_q * sizeof(float), 256) / sizeof(float);
  bp.info = (const QBlockInfo *)workspace;
  bp.bits = (const uint32_t *)((const char *)workspace + bits_offset(nhead_k, num_q_block));
  bp.cu_k = cu_k_seqlens; bp.cu_num_q_block = cu_num_q_block; bp.cu_num_k_block = cu_num_k_block;
  bp.q_s = strides[0] * es; bp.q_h = strides[1] * es; bp.k_s = strides[2] * es; bp.k_h = strides[3] * es;
  bp.v_s = strides[4] * es; bp.v_h = strides[5] * es; bp.o_s = strides[6] * es; bp.o_h = strides[7] * es;
  bp.do_s = strides[8] * es; bp.do_h = strides[9] * es;
  bp.dq_s = strides[10] * es; bp.dq_h = strides[11] * es; bp.dk_s = strides[12] * es; bp.dk_h = strides[13] * es;
  bp.dv_s = strides[14] * es; bp.dv_h = strides[15] * es;
  bp.nqb = num_q_block; bp.nkb = num_k_block; bp.batch = batch; bp.total_k = total_k;
  bp.ratio = nhead_q / nhead_k; bp.nhead_q = nhead_q; bp.qbs = q_block_size;
  bp.kbs = k_block_size;
  bp.wpr = words_per_row(num_k_block); bp.causal = causal ? 1 : 0;
  bp.wps = (q_block_size + kWaveRows - 1) / kWaveRows;
  bp.nsub = (bp.ratio * bp.wps + 3) / 4;
  bp.nsub_k = (k_block_size + 4 * kWaveRows - 1) / (4 * kWaveRows);
  bp.xcd_heads = (nhead_k % 8 == 0 && (long long)num_k_block * bp.nsub_k * nhead_k < (1LL << 31) &&
                  (long long)num_q_block * bp.nsub * nhead_k < (1LL << 31)) ? 1 : 0;
  bp.c = softmax_scale * kLog2e;
  bp.scale = softmax_scale;
  hipStream_t st = (hipStream_t)stream;
  const bool bf = dtype == HBSA_DTYPE_BF16;
  switch (headdim) {
    case 32: return bf ? launch_bwd<32, ElemBF16>(bp, nhead_k, num_k_block, st) : launch_bwd<32, ElemF16>(bp, nhead_k, num_k_block, st);
    case 64: return bf ? launch_bwd<64, ElemBF16>(bp, nhead_k, num_k_block, st) : launch_bwd<64, ElemF16>(bp, nhead_k, num_k_block, st);
    default: return bf ? launch_bwd<128, ElemBF16>(bp, nhead_k, num_k_block, st) : launch_bwd<128, ElemF16>(bp, nhead_k, num_k_block, st);
  }
}
}  // extern "C"
