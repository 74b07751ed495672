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
#include <cstring>

#include "hbsattn_amd.h"

namespace {

typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define HBSA_AS1(p) ((const __attribute__((address_space(1))) void *)(p))
#define HBSA_AS3(p) ((__attribute__((address_space(3))) void *)(p))

constexpr int kThreads = 256;   // 4 wavefronts
constexpr int kWaveRows = 32;   // query rows per wavefront (the MFMA N dimension)
constexpr int kTileKeys = 64;   // keys per main-loop step
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLazyRescaleLog2 = 8.0f;  // running max may lag the true max by 2^8

// Geometry of one q block, written by the pre-pass (32 bytes).
struct QBlockInfo {
  int32_t row_begin;   // token row of the block's first query
  int32_t rows;        // queries in the block (ragged last block of a sequence)
  int32_t key_begin;   // token row of the sequence's first key
  int32_t klen;        // keys in the sequence
  int32_t q_pos;       // in-sequence position of the block's first query
  int32_t shift;       // k_len - q_len: bottom-right causal alignment
  int32_t nkblk;       // k blocks in the sequence
  int32_t kmax;        // exclusive in-sequence bound of keys any row of the block may see
};

struct PrepParams {
  const int32_t *cu_q, *cu_k, *q_block_to_batch, *cu_num_q_block, *cu_num_k_block;
  const uint8_t *mask;
  int64_t ms_h, ms_q, ms_k;
  QBlockInfo *info;
  uint32_t *bits;
  int32_t nqb, qbs, kbs, wpr, causal;
};

struct FwdParams {
  const char *q, *k, *v;
  char *out;
  const QBlockInfo *info;
  const uint32_t *bits;
  int64_t q_s, q_h, k_s, k_h, v_s, v_h, o_s, o_h;  // bytes
  int32_t nqb, ratio, kbs, wpr, causal;
  int32_t wps;    // wave slots per q head = ceil(q_block_size / 32)
  int32_t nsub;   // workgroups per (kv head, q block) = ceil(ratio * wps / 4)
  uint32_t q_sign;  // 0x80008000 when softmax_scale < 0 (Q is negated, |scale| used)
  float c;        // |softmax_scale| * log2(e)
  float lag;      // kLazyRescaleLog2 / c, in raw score units
};

// --------------------------------------------------------------------------------------
// Pre-pass: one wavefront per (kv head, q block).
// --------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void hbsa_prep_kernel(PrepParams p) {
  const int lane = threadIdx.x & 63;
  const int g = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (g >= p.nqb) return;
  const int hk = blockIdx.y;
  const int b = p.q_block_to_batch[g];
  const int q0 = p.cu_q[b], qlen = p.cu_q[b + 1] - q0;
  const int k0 = p.cu_k[b], klen = p.cu_k[b + 1] - k0;
  const int q_pos = (g - p.cu_num_q_block[b]) * p.qbs;
  const int rows = min(p.qbs, qlen - q_pos);
  const int shift = klen - qlen;
  const int kb0 = p.cu_num_k_block[b];
  const int nkb = p.cu_num_k_block[b + 1] - kb0;
  int kmax = p.causal ? min(klen, q_pos + rows + shift) : klen;
  if (kmax < 0) kmax = 0;
  const int nvis = min(nkb, (kmax + p.kbs - 1) / p.kbs);
  if (hk == 0 && lane == 0) {
    QBlockInfo r;
    r.row_begin = q0 + q_pos; r.rows = rows; r.key_begin = k0; r.klen = klen;
    r.q_pos = q_pos; r.shift = shift; r.nkblk = nkb; r.kmax = kmax;
    p.info[g] = r;
  }
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
};
struct ElemF16 {
  static __device__ __forceinline__ f32x16 mfma(short8v a, short8v b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
};

// Walks the kept k blocks of one (kv head, q block): adjacent kept blocks form a run of
// keys; runs are handed out in tiles of kTileKeys.  All state is wavefront-uniform.  The
// row's bit words live in a VGPR (lane i holds word i of the current 64-word window) and
// are fetched with v_readlane, so stepping costs no memory latency.
struct TileWalker {
  const uint32_t *bits;
  int nwords, kbs, kmax, lane;
  int window;     // index of the 64-word window held in `held`
  uint32_t held;  // lane i: word window*64 + i (0 past the end of the row)
  int blk;        // next k block (in-sequence) to examine
  int pos, end;   // remaining keys of the current run, in-sequence positions

  __device__ __forceinline__ void init(const uint32_t *row, int nwords_, int kbs_, int kmax_, int lane_) {
    bits = row; nwords = nwords_; kbs = kbs_; kmax = kmax_; lane = lane_;
    window = 0;
    held = lane < nwords ? row[lane] : 0u;
    blk = 0; pos = 0; end = 0;
  }
  __device__ __forceinline__ uint32_t word(int w) {
    if ((w >> 6) != window) {
      window = w >> 6;
      const int i = window * 64 + lane;
      held = i < nwords ? bits[i] : 0u;
    }
    return (uint32_t)__builtin_amdgcn_readlane((int)held, w & 63);
  }
  __device__ __forceinline__ bool next(int &kpos, int &valid) {
    if (pos >= end) {
      int w = blk >> 5;
      if (w >= nwords) return false;
      uint32_t cur = word(w) & (~0u << (blk & 31));
      while (cur == 0) {
        if (++w >= nwords) return false;
        cur = word(w);
      }
      const int first = w * 32 + __builtin_ctz(cur);
      uint32_t inv = ~word(w) & (~0u << (first & 31));
      while (inv == 0) {
        if (++w >= nwords) break;
        inv = ~word(w);
      }
      const int stop = (w >= nwords) ? nwords * 32 : w * 32 + __builtin_ctz(inv);
      blk = stop;
      pos = first * kbs;
      end = min(stop * kbs, kmax);
      if (pos >= end) return false;
    }
    kpos = pos;
    valid = min(kTileKeys, end - pos);
    pos += kTileKeys;
    return true;
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
// Main kernel.  D = head dim (32, 64 or 128); rows of K/V tiles are D*2 bytes in LDS.
// LDS: K[2][64][D] then V[2][64][D] (double-buffered 64-key tiles), 16-byte chunks of
// every row XOR-swizzled so that both the K reads (16 rows x one chunk per 16 lanes) and
// the transposing V reads (4 rows x 64 bytes per 32 lanes) spread over all banks.
// --------------------------------------------------------------------------------------
template <int D, typename E>
__global__ __launch_bounds__(kThreads, 2) void hbsa_fwd_kernel(FwdParams p) {
  constexpr int RB = D * 2;            // row bytes
  constexpr int CPR = RB / 16;         // 16-byte chunks per row
  constexpr int RPG = 16 / CPR > 0 ? 16 / CPR : 1;  // rows per 256-byte bank sweep
  constexpr int TILE_BYTES = kTileKeys * RB;
  constexpr int LOADS = CPR / 4;       // 16-byte loads per thread per tile per operand
  constexpr int KSTEPS = D / 16;       // MFMA k-steps of Q.K^T
  constexpr int DT = D / 32;           // 32-row tiles of O^T

  extern __shared__ __attribute__((aligned(1024))) char lds[];
  char *lds_k = lds;
  char *lds_v = lds + 2 * TILE_BYTES;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g32 = lane >> 5;   // which half of the wavefront
  const int l32 = lane & 31;   // query within the wave slot / key row within a sub-tile

  // ---- work item: head-major, q blocks from the end of the packed batch backwards so
  // that under a causal mask the heaviest blocks of every sequence are issued first.
  const int bid = blockIdx.x;
  const int sub = bid % p.nsub;
  const int t = bid / p.nsub;
  const int qb = p.nqb - 1 - (t % p.nqb);
  const int hk = t / p.nqb;

  const QBlockInfo info = p.info[qb];
  const int slot = sub * 4 + wave;
  const int head_in_group = slot / p.wps;
  const int row0 = (slot % p.wps) * kWaveRows;          // first row of this wave inside the q block
  const int nrows = min(kWaveRows, info.rows - row0);
  const bool active = head_in_group < p.ratio && nrows > 0;
  const int hq = hk * p.ratio + head_in_group;

  // ---- per-thread source/destination pattern of the tile loads (same for every tile)
  int ld_row[LOADS];
  int ld_koff[LOADS], ld_voff[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int c = (i * 4 + wave) * 64 + lane;
    const int r = c / CPR, pc = c % CPR;
    ld_row[i] = r;
    ld_koff[i] = (pc ^ ((r / RPG) % CPR)) * 16;
    ld_voff[i] = (pc ^ ((CPR >= 8) ? (((r / RPG) % (CPR / 4)) << 2) : 0)) * 16;
  }
  const char *kg = p.k + (int64_t)hk * p.k_h;
  const char *vg = p.v + (int64_t)hk * p.v_h;

  auto issue_loads = [&](int buf, int kpos, int valid) {
    const int tok0 = info.key_begin + kpos;
    const int tok_last = tok0 + valid - 1;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int tok = min(tok0 + ld_row[i], tok_last);
      const int lds_off = buf * TILE_BYTES + (i * 4 + wave) * 1024;
      __builtin_amdgcn_global_load_lds(HBSA_AS1(kg + (int64_t)tok * p.k_s + ld_koff[i]), HBSA_AS3(lds_k + lds_off), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(HBSA_AS1(vg + (int64_t)tok * p.v_s + ld_voff[i]), HBSA_AS3(lds_v + lds_off), 16, 0, 0);
    }
  };

  TileWalker walk;
  walk.init(p.bits + ((size_t)hk * p.nqb + qb) * p.wpr, 2 * ((info.nkblk + 63) >> 6), p.kbs, info.kmax, lane);

  int kpos = 0, valid = 0;
  bool have = walk.next(kpos, valid);
  if (have) issue_loads(0, kpos, valid);

  // ---- Q^T fragments (B operand): lane holds query l32, d = 16*ks + 8*g32 .. +7
  short8v qf[KSTEPS];
  if (active) {
    const int r = min(row0 + l32, info.rows - 1);
    const char *qrow = p.q + (int64_t)(info.row_begin + r) * p.q_s + (int64_t)hq * p.q_h + g32 * 16;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      u32x4 raw = *(const u32x4 *)(qrow + ks * 32);
      raw ^= p.q_sign;
      qf[ks] = __builtin_bit_cast(short8v, raw);
    }
  } else {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[ks] = (short8v)0;
  }

  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
  float m_run = -INFINITY;  // running reference max, raw (unscaled) score units
  float l_run = 0.f;        // this lane's share of the row sum

  // causal visibility of this lane's / this wave's rows: key position <= qpos + shift
  const int lane_kvis = info.q_pos + min(row0 + l32, info.rows - 1) + info.shift;
  const int wave_kvis_min = info.q_pos + row0 + info.shift;
  const int wave_kvis_max = info.q_pos + row0 + nrows - 1 + info.shift;

  // ---- per-lane LDS read addresses
  // K (A operand of S^T): row l32 (+32), chunk (2*ks + g32) ^ swz(row)
  const int k_rd = l32 * RB + ((g32 ^ ((l32 / RPG) % CPR)) << 4);
  // V^T (A operand of O^T) through ds_read_b64_tr_b16: within a group of 16 lanes, lane r
  // supplies the address of key (r / 4), dims 4*(r % 4) .. +3 and receives dim r of 4 keys.
  const int v_key = 4 * g32 + ((lane & 15) >> 2);
  const int v_lc = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
  const int v_swz = (CPR >= 8) ? (((v_key / RPG) % (CPR / 4)) << 2) : 0;
  const int v_rd = v_key * RB + ((v_lc | v_swz) << 4) + 8 * (lane & 1);

  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): first tile has landed in LDS
  __syncthreads();

  int buf = 0;
  while (have) {
    int nkpos = 0, nvalid = 0;
    const bool have_next = walk.next(nkpos, nvalid);
    if (have_next) issue_loads(buf ^ 1, nkpos, nvalid);

    if (active && (!p.causal || kpos <= wave_kvis_max)) {
      const uint32_t kt_base = (uint32_t)(uintptr_t)HBSA_AS3(lds_k + buf * TILE_BYTES);
      const uint32_t vt_base = (uint32_t)(uintptr_t)HBSA_AS3(lds_v + buf * TILE_BYTES);
      // ---- S^T = K . Q^T  (two 32-key sub-tiles)
      f32x16 s[2];
#pragma unroll
      for (int i = 0; i < 16; ++i) { s[0][i] = 0.f; s[1][i] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const uint32_t a = kt_base + (uint32_t)(k_rd ^ (ks * 32));
        const short8v a0 = *(const __attribute__((address_space(3))) short8v *)(uintptr_t)a;
        const short8v a1 = *(const __attribute__((address_space(3))) short8v *)(uintptr_t)(a + 32 * RB);
        s[0] = E::mfma(a0, qf[ks], s[0]);
        s[1] = E::mfma(a1, qf[ks], s[1]);
      }
      // ---- edge tiles: ragged run tail and the causal diagonal
      const bool edge = valid < kTileKeys || (p.causal && kpos + valid - 1 > wave_kvis_min);
      if (edge) {
        int lim = valid;
        if (p.causal) lim = min(lim, lane_kvis - kpos + 1);
        lim -= 4 * g32;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if (kt * 32 + 8 * (i >> 2) + (i & 3) >= lim) s[kt][i] = -INFINITY;
      }
      // ---- online softmax, one query per lane (keys split with lane ^ 32)
      float mx = fmaxf(s[0][0], s[1][0]);
#pragma unroll
      for (int i = 1; i < 16; ++i) mx = fmaxf(mx, fmaxf(s[0][i], s[1][i]));
      mx = half_max(mx);
      const bool grow = mx > m_run + p.lag;
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
        const float m_new = grow ? mx : m_run;
        const float alpha = grow ? __builtin_amdgcn_exp2f((m_run - m_new) * p.c) : 1.f;
        l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
        m_run = m_new;
      }
      const float mc = (m_run == -INFINITY) ? 0.f : m_run * p.c;
      float rs = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][i], p.c, -mc));
          s[kt][i] = e;
          rs += e;
        }
      l_run += rs;
      // ---- O^T += V^T . P^T
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          u32x4 pw;
#pragma unroll
          for (int e = 0; e < 4; ++e) pw[e] = E::pack2(s[kt][8 * j + 2 * e], s[kt][8 * j + 2 * e + 1]);
          const short8v pb = __builtin_bit_cast(short8v, pw);
          const uint32_t vrow = vt_base + (kt * 32 + 16 * j) * RB;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const uint32_t a = vrow + (uint32_t)(v_rd ^ (dt * 64));
            const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(uintptr_t)a);
            const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(uintptr_t)(a + 8 * RB));
            const short8v va = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            o[dt] = E::mfma(va, pb, o[dt]);
          }
        }
    }

    if (!have_next) break;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): next tile has landed
    __syncthreads();                     // and every wave is done with the current buffers
    buf ^= 1;
    kpos = nkpos;
    valid = nvalid;
  }

  // ---- epilogue: normalise, convert, store (rows with no visible key store exact zeros)
  if (active) {
    const float l_tot = half_sum(l_run);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (l32 < nrows) {
      char *orow = p.out + (int64_t)(info.row_begin + row0 + l32) * p.o_s + (int64_t)hq * p.o_h;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          uint2 w;
          w.x = E::pack2(o[dt][4 * i4 + 0] * inv, o[dt][4 * i4 + 1] * inv);
          w.y = E::pack2(o[dt][4 * i4 + 2] * inv, o[dt][4 * i4 + 3] * inv);
          *(uint2 *)(orow + (dt * 32 + 8 * i4 + 4 * g32) * 2) = w;
        }
    }
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

template <int D, typename E>
int launch_fwd(const FwdParams &fp, int grid, hipStream_t stream) {
  constexpr int lds_bytes = 4 * kTileKeys * D * 2;
  static thread_local bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&hbsa_fwd_kernel<D, E>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    attr_set = true;
  }
  hipLaunchKernelGGL((hbsa_fwd_kernel<D, E>), dim3(grid), dim3(kThreads), lds_bytes, stream, fp);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail((int)e, "hbsa_fwd_kernel launch: %s", hipGetErrorString(e));
  return 0;
}

}  // namespace

extern "C" {

int hbsa_abi_version(void) { return HBSA_ABI_VERSION; }

const char *hbsa_last_error(void) { return g_err; }

size_t hbsa_fwd_workspace_bytes(int32_t nhead_k, int32_t num_q_block, int32_t num_k_block) {
  if (nhead_k <= 0 || num_q_block <= 0 || num_k_block <= 0) return 256;
  const size_t info = align_up((size_t)num_q_block * sizeof(QBlockInfo), 256);
  const size_t bits = align_up((size_t)nhead_k * num_q_block * words_per_row(num_k_block) * sizeof(uint32_t), 256);
  return info + bits;
}

int hbsa_fwd_prepare(const int32_t *cu_q_seqlens, const int32_t *cu_k_seqlens, const uint8_t *block_mask,
                     const int32_t *q_block_to_batch, const int32_t *cu_num_q_block, const int32_t *cu_num_k_block,
                     void *workspace, size_t workspace_bytes, int32_t batch, int32_t nhead_k, int32_t num_q_block,
                     int32_t num_k_block, int32_t q_block_size, int32_t k_block_size, int32_t causal,
                     const int64_t *mask_strides, void *stream) {
  g_err[0] = 0;
  if (batch < 0 || num_q_block < 0 || num_k_block < 0) return fail(HBSA_ERR_INVALID_ARGUMENT, "negative size");
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
  pp.bits = (uint32_t *)((char *)workspace + align_up((size_t)num_q_block * sizeof(QBlockInfo), 256));
  pp.nqb = num_q_block; pp.qbs = q_block_size; pp.kbs = k_block_size; pp.wpr = words_per_row(num_k_block);
  pp.causal = causal ? 1 : 0;
  hipLaunchKernelGGL(hbsa_prep_kernel, dim3((num_q_block + 3) / 4, nhead_k), dim3(kThreads), 0, (hipStream_t)stream, pp);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail((int)e, "hbsa_prep_kernel launch: %s", hipGetErrorString(e));
  return 0;
}

int hbsa_fwd_run(const void *q, const void *k, const void *v, void *out, const void *workspace, size_t workspace_bytes,
                 int32_t dtype, int32_t total_q, int32_t total_k, int32_t nhead_q, int32_t nhead_k, int32_t headdim,
                 int32_t num_q_block, int32_t num_k_block, int32_t q_block_size, int32_t k_block_size, int32_t causal,
                 float softmax_scale, const int64_t *strides, void *stream) {
  g_err[0] = 0;
  if (total_q < 0 || total_k < 0) return fail(HBSA_ERR_INVALID_ARGUMENT, "negative size");
  if (total_q == 0 || num_q_block == 0 || nhead_q == 0) return 0;  // nothing to write
  if (!q || !k || !v || !out || !workspace || !strides) return fail(HBSA_ERR_INVALID_ARGUMENT, "null pointer argument");
  if (nhead_k <= 0 || nhead_q % nhead_k != 0)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "nhead_q (%d) must be divisible by nhead_k (%d)", nhead_q, nhead_k);
  if (q_block_size <= 0 || k_block_size <= 0 || q_block_size % 16 || k_block_size % 16)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "q_block_size (%d) and k_block_size (%d) must be positive multiples of 16",
                q_block_size, k_block_size);
  if (headdim != 32 && headdim != 64 && headdim != 128)
    return fail(HBSA_ERR_UNSUPPORTED, "headdim %d not in {32, 64, 128}", headdim);
  if (dtype != HBSA_DTYPE_BF16 && dtype != HBSA_DTYPE_F16)
    return fail(HBSA_ERR_UNSUPPORTED, "dtype code %d not supported", dtype);
  if (num_k_block <= 0 || total_k <= 0) return fail(HBSA_ERR_INVALID_ARGUMENT, "no keys");
  if (!std::isfinite(softmax_scale)) return fail(HBSA_ERR_INVALID_ARGUMENT, "softmax_scale is not finite");
  for (int i = 0; i < 8; ++i)
    if (strides[i] % 8 != 0)
      return fail(HBSA_ERR_INVALID_ARGUMENT, "stride %d (%lld elements) is not a multiple of 8 (16-byte rows)", i,
                  (long long)strides[i]);
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "q/k/v/out must be 16-byte aligned");
  if ((uintptr_t)workspace & 255) return fail(HBSA_ERR_INVALID_ARGUMENT, "workspace must be 256-byte aligned");
  const size_t need = hbsa_fwd_workspace_bytes(nhead_k, num_q_block, num_k_block);
  if (workspace_bytes < need)
    return fail(HBSA_ERR_WORKSPACE_TOO_SMALL, "workspace %zu bytes < required %zu", workspace_bytes, need);

  FwdParams fp;
  fp.q = (const char *)q; fp.k = (const char *)k; fp.v = (const char *)v; fp.out = (char *)out;
  fp.info = (const QBlockInfo *)workspace;
  fp.bits = (const uint32_t *)((const char *)workspace + align_up((size_t)num_q_block * sizeof(QBlockInfo), 256));
  fp.q_s = strides[0] * 2; fp.q_h = strides[1] * 2; fp.k_s = strides[2] * 2; fp.k_h = strides[3] * 2;
  fp.v_s = strides[4] * 2; fp.v_h = strides[5] * 2; fp.o_s = strides[6] * 2; fp.o_h = strides[7] * 2;
  fp.nqb = num_q_block; fp.ratio = nhead_q / nhead_k; fp.kbs = k_block_size; fp.wpr = words_per_row(num_k_block);
  fp.causal = causal ? 1 : 0;
  fp.wps = (q_block_size + kWaveRows - 1) / kWaveRows;
  fp.nsub = (fp.ratio * fp.wps + 3) / 4;
  fp.q_sign = softmax_scale < 0.f ? 0x80008000u : 0u;
  float c = std::fabs(softmax_scale) * kLog2e;
  if (c < 1e-30f) c = 1e-30f;  // scale 0: uniform weights over the visible keys, and -inf * c stays -inf
  fp.c = c;
  fp.lag = kLazyRescaleLog2 / c;
  const long long grid = (long long)nhead_k * num_q_block * fp.nsub;
  if (grid > 0x7fffffffLL) return fail(HBSA_ERR_UNSUPPORTED, "too many work items (%lld)", grid);

  hipStream_t st = (hipStream_t)stream;
  const bool bf = dtype == HBSA_DTYPE_BF16;
  switch (headdim) {
    case 32: return bf ? launch_fwd<32, ElemBF16>(fp, (int)grid, st) : launch_fwd<32, ElemF16>(fp, (int)grid, st);
    case 64: return bf ? launch_fwd<64, ElemBF16>(fp, (int)grid, st) : launch_fwd<64, ElemF16>(fp, (int)grid, st);
    default: return bf ? launch_fwd<128, ElemBF16>(fp, (int)grid, st) : launch_fwd<128, ElemF16>(fp, (int)grid, st);
  }
}

int hbsa_fwd(const void *q, const void *k, const void *v, void *out, const int32_t *cu_q_seqlens,
             const int32_t *cu_k_seqlens, const uint8_t *block_mask, const int32_t *q_block_to_batch,
             const int32_t *cu_num_q_block, const int32_t *cu_num_k_block, void *workspace,
             size_t workspace_bytes, int32_t dtype, int32_t batch, int32_t total_q, int32_t total_k,
             int32_t nhead_q, int32_t nhead_k, int32_t headdim, int32_t num_q_block, int32_t num_k_block,
             int32_t q_block_size, int32_t k_block_size, int32_t causal, float softmax_scale,
             const int64_t *strides, void *stream) {
  g_err[0] = 0;
  if (total_q == 0 || num_q_block == 0 || nhead_q == 0) return 0;
  if (!strides) return fail(HBSA_ERR_INVALID_ARGUMENT, "null pointer argument");
  // Validate the main launch before queueing anything, so a refused call leaves no work behind.
  if (!q || !k || !v || !out) return fail(HBSA_ERR_INVALID_ARGUMENT, "null pointer argument");
  if (nhead_k <= 0 || nhead_q % nhead_k != 0)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "nhead_q (%d) must be divisible by nhead_k (%d)", nhead_q, nhead_k);
  if (headdim != 32 && headdim != 64 && headdim != 128)
    return fail(HBSA_ERR_UNSUPPORTED, "headdim %d not in {32, 64, 128}", headdim);
  if (dtype != HBSA_DTYPE_BF16 && dtype != HBSA_DTYPE_F16)
    return fail(HBSA_ERR_UNSUPPORTED, "dtype code %d not supported", dtype);
  if (!std::isfinite(softmax_scale)) return fail(HBSA_ERR_INVALID_ARGUMENT, "softmax_scale is not finite");
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15)
    return fail(HBSA_ERR_INVALID_ARGUMENT, "q/k/v/out must be 16-byte aligned");
  for (int i = 0; i < 8; ++i)
    if (strides[i] % 8 != 0)
      return fail(HBSA_ERR_INVALID_ARGUMENT, "stride %d (%lld elements) is not a multiple of 8 (16-byte rows)", i,
                  (long long)strides[i]);
  int rc = hbsa_fwd_prepare(cu_q_seqlens, cu_k_seqlens, block_mask, q_block_to_batch, cu_num_q_block, cu_num_k_block,
                            workspace, workspace_bytes, batch, nhead_k, num_q_block, num_k_block, q_block_size,
                            k_block_size, causal, strides + 8, stream);
  if (rc != 0) return rc;
  return hbsa_fwd_run(q, k, v, out, workspace, workspace_bytes, dtype, total_q, total_k, nhead_q, nhead_k, headdim,
                      num_q_block, num_k_block, q_block_size, k_block_size, causal, softmax_scale, strides, stream);
}

}  // extern "C"
