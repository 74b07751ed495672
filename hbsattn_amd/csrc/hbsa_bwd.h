// Block-sparse attention backward for gfx950: dQ, dK, dV from dO, the forward's output and its
// log-sum-exp.  Part of the translation unit hbsa_fwd.hip (included after the forward's helpers).
//
// The reference stops at the forward (reference hbsattn/hbsa_interface.py:31-32 raises
// NotImplementedError in backward), so this follows the mathematics of that forward
// (reference hbsattn/reference.py:23-107): with S = scale * Q K^T masked like the forward,
// P = exp(S - lse), delta = rowsum(dO * O):
//     dV = P^T dO      dP = dO V^T      dS = P * (dP - delta)
//     dQ = scale * dS K                 dK = scale * dS^T Q
//
// Two launches per call, no atomics, every output element written by exactly one workgroup:
//   hbsa_bwd_dq_kernel    : one workgroup per (kv head, q block, group of four 32-row wave slots), the
//                           forward's decomposition; walks the kept k blocks of the q block's bit row.
//                           Per 64-key tile  S^T = K Q^T,  dP^T = V dO^T  (A = tile rows from LDS,
//                           B = Q^T / dO^T in registers),  dS^T in the accumulator layout is the B
//                           operand of  dQ^T += K^T dS^T  (A = K^T through transposing LDS reads).  It also forms
//                           delta of its rows (it holds their dO; their O is one more row load) and leaves
//                           it for the second launch.
//   hbsa_bwd_dkv_kernel   : (head dims up to 64; hbsa_bwd_dkv8_kernel is the form for D = 128) the same
//                           with the roles of queries and keys exchanged: one workgroup per
//                           (kv head, k block, group of four 32-key slots); K^T and V^T stay in
//                           registers, the Q and dO rows of every q block that keeps the k block (and of
//                           every q head of the group) stream through LDS in 64-row tiles:
//                           S = Q K^T,  dP = dO V^T,  dV^T += dO^T P,  dK^T += Q^T dS.
// Both recompute S.  The kept blocks of a mask row or column are found with one load per 32 or 64
// blocks, not one per block.  Tiles go from global memory straight into LDS (global_load_lds_dwordx4),
// two buffers: tile t + 1 travels while tile t is computed on, one barrier per tile (the D = 128 dK/dV kernel
// has four Q and three dO buffers and fetches two tiles ahead).  A tile that is
// read both by rows and transposed is stored once, in a layout without bank conflicts for either
// (BwdTile::swz_both).  In the dQ kernel and the D = 128 dK/dV kernel the operand reads from LDS are issued by
// hand, a fixed number ahead of the products that use them (BwdOperandOffsets).  The forward's persistent
// scheduling is not applied here: the grids already start their heaviest workgroups first, and what bounds
// both kernels at long sequences is the stream of tiles from memory next to the matrix work, not the tail.

namespace {

struct BwdParams {
  const char *q, *k, *v, *out, *dout;
  char *dq, *dk, *dv;
  const float *lse;           // [total_q, nhead_q], contiguous
  float *delta;               // [total_q, nhead_q], contiguous: rowsum(dO * O), written by the dQ kernel, read by the dK/dV kernels
  float *lse2;                // [total_q, nhead_q]: lse * log2(e), +inf where lse is -inf; written by the dQ kernel for the D = 128 dK/dV kernel
  const QBlockInfo *info;
  const uint32_t *bits;
  const int32_t *cu_k, *cu_num_q_block, *cu_num_k_block;
  int64_t q_s, q_h, k_s, k_h, v_s, v_h, o_s, o_h, do_s, do_h, dq_s, dq_h, dk_s, dk_h, dv_s, dv_h;   // bytes
  int32_t nqb, nkb, xcd_heads, batch, ratio, nhead_q, qbs, kbs, wpr, causal;   // xcd_heads: see the dK/dV kernels
  int32_t total_k;
  int32_t wps, nsub;     // q side: wave slots per q head and workgroups per (kv head, q block), as in the forward
  int32_t nsub_k;        // k side: workgroups per (kv head, k block) = ceil(k_block_size / 128)
  float c;               // softmax_scale * log2(e), signed
  float scale;
};

// ---- shared pieces of the two main kernels ---------------------------------------------------------
template <int D>
struct BwdTile {
  static constexpr int RB = D * 2;            // row bytes
  static constexpr int CPR = RB / 16;         // 16-byte chunks per row
  static constexpr int RPG = 16 / CPR > 0 ? 16 / CPR : 1;
  static constexpr int TILE_BYTES = 64 * RB;
  static constexpr int KSTEPS = D / 16;
  static constexpr int DT = D / 32;
  // One chunk swizzle for a tile that is read both ways, so that it is stored once: chunk c of row r sits
  // at chunk position c ^ swz_both(r).  With a = (r / RPG) % CPR, the bits of a rotated so that its lowest
  // bits select the 64-byte column group.  Over any 16 consecutive rows the 16-byte slots of a chunk
  // column are all different (reads by rows), and rows 0-7 of a group spread evenly over the column
  // groups (transposing reads).
  static __host__ __device__ constexpr int swz_both(int r) {
    const int a = (r / RPG) % CPR;
    if constexpr (CPR == 16) return ((a & 3) << 2) | (a >> 2);
    else if constexpr (CPR == 8) return ((a & 1) << 2) | (a >> 1);
    else return a;
  }
};

// 16 bytes per lane from global memory (scalar base + 32-bit lane offset) straight into LDS at lds_addr + 16 * lane
__device__ __forceinline__ void bwd_dma16(uint32_t lds_addr, const char *sbase, uint32_t voff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(sbase) : "memory", "m0");
}

// 4 bytes per lane likewise, to lds_addr + 4 * lane
__device__ __forceinline__ void bwd_dma4(uint32_t lds_addr, const void *sbase, uint32_t voff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" : : "s"(lds_addr), "v"(voff), "s"(sbase) : "memory", "m0");
}

// ---- Operand reads issued by hand (lds_read_b128 / lds_read_tr16_b64 of the forward, which explain the rules):
// the compiler puts a read next to the product that uses it, and a chain of products on one accumulator then
// waits out the LDS latency at every step.  Here a fixed number of reads is under way ahead of the products.
//
// Per-lane byte offsets of the operands inside a tile stored with BwdTile::swz_both, computed once per kernel:
//   rows[ks]   : row lane % 32 (+ 32 * h as an immediate), the 16 bytes of step ks for this lane's half of the step
//   tr[dt]     : the first of the two transposing reads of head dim slice dt for keys 16 * g .. (+ g * 16 rows as an
//                immediate); the second one, eight rows further down, sits at (tr[dt] ^ 32) + 8 rows: for every
//                head dim swz_both(key + 8) = swz_both(key) ^ 2 when key < 8
template <int D>
struct BwdOperandOffsets {
  using T = BwdTile<D>;
  uint32_t rows[T::KSTEPS], tr[T::DT];
  static constexpr bool second_read_is_xor_32() {
    for (int key = 0; key < 8; ++key)
      if (T::swz_both(key + 8) != (T::swz_both(key) ^ 2)) return false;
    return true;
  }
  static_assert(second_read_is_xor_32(), "the second transposing read's address is derived from the first one's");
  __device__ __forceinline__ void init(int lane) {
    const int l32 = lane & 31, g32 = lane >> 5;
    const int rd = l32 * T::RB + ((g32 ^ T::swz_both(l32)) << 4);
#pragma unroll
    for (int ks = 0; ks < T::KSTEPS; ++ks) rows[ks] = (uint32_t)(rd ^ (ks * 32));
    const int key = 4 * g32 + ((lane & 15) >> 2);
    const int lc = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
    const int t0 = key * T::RB + ((lc ^ T::swz_both(key)) << 4) + 8 * (lane & 1);
#pragma unroll
    for (int dt = 0; dt < T::DT; ++dt) tr[dt] = (uint32_t)(t0 ^ (dt * 64));
  }
};

// the 2 * DT transposing reads of key group G of the tile at LDS address tile (all head dim slices)
template <int D, int G>
__device__ __forceinline__ void bwd_issue_transposed(const BwdOperandOffsets<D> &off, uint32_t tile, short4v *dst) {
  using T = BwdTile<D>;
  static_for<0, T::DT>([&](auto dt_) {
    constexpr int dt = decltype(dt_)::value;
    dst[2 * dt] = lds_read_tr16_b64<G * 16 * T::RB>(off.tr[dt] + tile);
    dst[2 * dt + 1] = lds_read_tr16_b64<G * 16 * T::RB + 8 * T::RB>((off.tr[dt] ^ 32u) + tile);
  });
}
// returns once at most N LDS operations issued after those 2 * DT reads are outstanding
template <int D, int N>
__device__ __forceinline__ void bwd_wait_transposed(short4v *v) {
  constexpr int DT = BwdTile<D>::DT;
  static_assert(N <= 15, "the counter has four bits");
  if constexpr (DT == 4) lds_wait<N>(v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7]);
  else if constexpr (DT == 2) asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]) : "n"(N));
  else asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(v[0]), "+v"(v[1]) : "n"(N));
}
// acc[dt] += (those operands)^T . packed
template <int D, typename E>
__device__ __forceinline__ void bwd_transposed_products(const short4v *v, short8v packed, f32x16 *acc) {
#pragma unroll
  for (int dt = 0; dt < BwdTile<D>::DT; ++dt) {
    const short8v va = __builtin_shufflevector(v[2 * dt], v[2 * dt + 1], 0, 1, 2, 3, 4, 5, 6, 7);
    acc[dt] = E::mfma(va, packed, acc[dt]);
  }
}

// rows 32*h .. 32*h+31 of the tile . frag^T, the forward's S^T = K Q^T for one half of a tile
template <int D, typename E>
__device__ __forceinline__ f32x16 bwd_rows_times_frag(const char *tile, int h, const short8v *frag, int lane) {
  using T = BwdTile<D>;
  const int l32 = lane & 31, g32 = lane >> 5;
  const int rd = l32 * T::RB + ((g32 ^ T::swz_both(l32)) << 4) + h * 32 * T::RB;
  f32x16 a;
#pragma unroll
  for (int i = 0; i < 16; ++i) a[i] = 0.f;
#pragma unroll
  for (int ks = 0; ks < T::KSTEPS; ++ks) a = E::mfma(*(const short8v *)(tile + (rd ^ (ks * 32))), frag[ks], a);
  return a;
}

// acc[dt] += tile^T (rows 16*g .. 16*g+15 of the tile as the contraction index) . packed, the forward's
// O^T += V^T P^T for one group of 16 keys
template <int D, typename E>
__device__ __forceinline__ void bwd_transposed_times_packed(const char *tile, int g, short8v packed, int lane, f32x16 *acc) {
  using T = BwdTile<D>;
  const int g32 = lane >> 5;
  const int key = 4 * g32 + ((lane & 15) >> 2);
  const int lc = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
  const int rd = key * T::RB + ((lc ^ T::swz_both(key)) << 4) + 8 * (lane & 1);
  const int rd8 = (key + 8) * T::RB + ((lc ^ T::swz_both(key + 8)) << 4) + 8 * (lane & 1);   // the row 8 further down
#pragma unroll
  for (int dt = 0; dt < T::DT; ++dt) {
    const char *a = tile + (rd ^ (dt * 64)) + g * 16 * T::RB;
    const char *a8 = tile + (rd8 ^ (dt * 64)) + g * 16 * T::RB;
    const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)HBSA_AS3(a));
    const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)HBSA_AS3(a8));
    const short8v va = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    acc[dt] = E::mfma(va, packed, acc[dt]);
  }
}

// 16 accumulator values of one lane -> two B operands (rows 0-15 and 16-31 of the half tile)
template <typename E>
__device__ __forceinline__ void bwd_pack(const float *e, short8v &lo, short8v &hi) {
  u32x4 w[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) w[j][q4] = E::pack2(e[8 * j + 2 * q4], e[8 * j + 2 * q4 + 1]);
  lo = __builtin_bit_cast(short8v, w[0]);
  hi = __builtin_bit_cast(short8v, w[1]);
}

// accumulators [d, row = lane % 32] * f -> out row (16-bit), the forward's plain epilogue
template <int D, typename E>
__device__ __forceinline__ void bwd_store_rows(char *row_ptr, const f32x16 *acc, float f, int g32) {
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      u32x2 w;
      w.x = E::pack2(acc[dt][4 * i4 + 0] * f, acc[dt][4 * i4 + 1] * f);
      w.y = E::pack2(acc[dt][4 * i4 + 2] * f, acc[dt][4 * i4 + 3] * f);
      *(u32x2 *)(row_ptr + (dt * 32 + 8 * i4 + 4 * g32) * 2) = w;
    }
}

// The dK/dV kernels' check of the sequence b their k block belongs to.  A sequence the pre-pass found not to
// fit the tensors (flagged q block records, no bit rows) takes no part: its keys get zero gradients where they
// lie inside dk and dv, and the workgroup is done.
template <int D>
__device__ __forceinline__ bool bwd_sequence_skipped(const BwdParams &p, int b, int kb, int sub, int hk) {
  const int first_qb = p.cu_num_q_block[b];
  if (first_qb < 0 || first_qb >= p.nqb) return true;
  if (first_qb >= p.cu_num_q_block[b + 1] || p.info[first_qb].flags == 0) return false;
  const int64_t k0 = p.cu_k[b], k1 = p.cu_k[b + 1];
  const int kbl = kb - p.cu_num_k_block[b];
  if (k0 < 0 || k1 <= k0 || kbl < 0) return true;
  const int64_t first = k0 + (int64_t)kbl * p.kbs + (int64_t)sub * 4 * kWaveRows;
  int64_t stop = k0 + (int64_t)(kbl + 1) * p.kbs;
  stop = stop < k1 ? stop : k1;
  stop = stop < first + 4 * kWaveRows ? stop : first + 4 * kWaveRows;
  stop = stop < p.total_k ? stop : (int64_t)p.total_k;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  for (int64_t i = threadIdx.x; i < (stop - first) * (D / 8); i += blockDim.x) {
    const int64_t row = first + i / (D / 8);
    const int c = (int)(i % (D / 8));
    *(u32x4 *)(p.dk + row * p.dk_s + (int64_t)hk * p.dk_h + c * 16) = zero;
    *(u32x4 *)(p.dv + row * p.dv_s + (int64_t)hk * p.dv_h + c * 16) = zero;
  }
  return true;
}

// ---- dQ ----------------------------------------------------------------------------------------------
template <int D, typename E>
__global__ __launch_bounds__(kThreads, 2) void hbsa_bwd_dq_kernel(BwdParams p) {
  using T = BwdTile<D>;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  // three K tiles and two V tiles, filled straight from global memory, in the layout that serves the reads by
  // rows and the transposing reads (BwdTile::swz_both)

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g32 = lane >> 5, l32 = lane & 31;
  // (grid decoding by XCD: see hbsa_bwd_dkv_kernel)
  int hk = blockIdx.y, bx = blockIdx.x;
  if (p.xcd_heads) {
    const unsigned t = blockIdx.x >> 3, per_head = (unsigned)(p.nqb * p.nsub);
    hk = (int)(blockIdx.x & 7u) + 8 * (int)(t / per_head);
    bx = (int)(t % per_head);
  }
  // last q blocks first: under a causal mask they are the long ones, and the grid should not end on them
  const int qb_rev = bx / p.nsub, sub = bx - qb_rev * p.nsub;
  const int qb = p.nqb - 1 - qb_rev;
  const QBlockInfo inf = p.info[qb];
  if (inf.rows <= 0) return;   // a q block with no row inside the tensors (its sequence did not fit them)

  const int slot = sub * 4 + wave;
  const int head_in_group = slot / p.wps;
  const int row0 = (slot % p.wps) * kWaveRows;
  const int nrows = min(kWaveRows, inf.rows - row0);
  const bool active = head_in_group < p.ratio && nrows > 0;
  const int hq = hk * p.ratio + head_in_group;

  short8v qf[T::KSTEPS], dof[T::KSTEPS];   // Q^T and dO^T fragments: lane holds row l32, d = 16*ks + 8*g32 .. +7
  float lse2 = INFINITY, dlt = 0.f;         // a row that takes no part gets P = exp2(-inf) = 0
  const int my_row = inf.row_begin + min(row0 + l32, inf.rows - 1);
  if (active) {
    const char *qrow = p.q + (int64_t)my_row * p.q_s + (int64_t)hq * p.q_h + g32 * 16;
    const char *grow = p.dout + (int64_t)my_row * p.do_s + (int64_t)hq * p.do_h + g32 * 16;
#pragma unroll
    for (int ks = 0; ks < T::KSTEPS; ++ks) {
      qf[ks] = *(const short8v *)(qrow + ks * 32);
      dof[ks] = *(const short8v *)(grow + ks * 32);
    }
    const float l = p.lse[(int64_t)my_row * p.nhead_q + hq];
    lse2 = l == -INFINITY ? INFINITY : l * kLog2e;
    // delta = sum over d of dO * O of the row: this lane's half of the head dim, then the other half's from lane + 32.
    // Every (row, q head) belongs to exactly one wavefront of this grid, which also leaves it for the dK/dV kernel.
    const char *orow = p.out + (int64_t)my_row * p.o_s + (int64_t)hq * p.o_h + g32 * 16;
#pragma unroll
    for (int ks = 0; ks < T::KSTEPS; ++ks) {
      const u32x4 a = __builtin_bit_cast(u32x4, dof[ks]), b = *(const u32x4 *)(orow + ks * 32);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        dlt += E::lo(a[j]) * E::lo(b[j]);
        dlt += E::hi(a[j]) * E::hi(b[j]);
      }
    }
    dlt = half_sum(dlt);
    if (g32 == 0 && l32 < nrows) {
      p.delta[(int64_t)my_row * p.nhead_q + hq] = dlt;
      p.lse2[(int64_t)my_row * p.nhead_q + hq] = lse2;
    }
  } else {
#pragma unroll
    for (int ks = 0; ks < T::KSTEPS; ++ks) { qf[ks] = short8v{0, 0, 0, 0, 0, 0, 0, 0}; dof[ks] = qf[ks]; }
  }
  f32x16 acc[T::DT];
#pragma unroll
  for (int dt = 0; dt < T::DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;

  const int lane_kvis = inf.q_pos + min(row0 + l32, inf.rows - 1) + inf.shift;   // last key position the row sees (causal)
  const int wave_kvis_min = inf.q_pos + min(row0, inf.rows - 1) + inf.shift;      // ... the wavefront's first row sees
  const uint32_t *bits = p.bits + ((size_t)hk * p.nqb + qb) * p.wpr;
  const char *kg = p.k + (int64_t)hk * p.k_h + (int64_t)inf.key_begin * p.k_s;
  const char *vg = p.v + (int64_t)hk * p.v_h + (int64_t)inf.key_begin * p.v_s;

  // the tile sequence: 64-key tiles of the kept k blocks, cut at the last key any row of the block sees
  int j = -1, kpos = 0;
  int word_base = -32;      // k block of bit 0 of the word being walked
  uint32_t word_left = 0;   // its kept blocks not visited yet
  // The bit row is read once, a word per lane (64 words = 2048 k blocks at a time), so that no load and its wait
  // stand between two tiles.
  const int last_word = (inf.nkblk - 1) >> 5;
  uint32_t row_words = lane <= last_word ? bits[lane] : 0u;
  auto next_tile = [&]() -> bool {
    if (j >= 0) {
      kpos += kTileKeys;
      if (kpos < min((j + 1) * p.kbs, inf.kmax)) return true;
    }
    while (word_left == 0) {   // next word of the bit row: 32 k blocks, kept or not
      word_base += 32;
      if (word_base >= inf.nkblk) return false;
      const int w = word_base >> 5;
      if (w >= 64 && (w & 63) == 0) {   // beyond 2048 k blocks: the next 64 words, waited for here so that no other path waits
        row_words = w + lane <= last_word ? bits[w + lane] : 0u;
        __builtin_amdgcn_s_waitcnt(0x0F70);
      }
      word_left = (uint32_t)__builtin_amdgcn_readlane((int)row_words, w & 63);
    }
    j = word_base + __builtin_ctz(word_left);
    word_left &= word_left - 1;
    kpos = j * p.kbs;   // below kmax: the pre-pass cleared the bits of blocks no row can see
    return true;
  };
  auto tile_valid = [&]() { return min(kTileKeys, min((j + 1) * p.kbs, inf.kmax) - kpos); };
  // A tile's chunks over four wavefronts: one load of a wavefront fills 1024 bytes (RPL rows); load i of
  // wavefront w the rows RPL * (4 * i + w) .. + RPL - 1; lane l the chunk position l % CPR of row l / CPR
  // of those, which holds the row's chunk (l % CPR) ^ swz_both(row).
  constexpr int RPL = 1024 / T::RB, LOADS = 64 / (4 * RPL);
  const int ld_row = RPL * wave + lane / T::CPR;                                  // + 4 * RPL * i
  const uint32_t ld_chunk = (uint32_t)(((lane % T::CPR) ^ T::swz_both(ld_row)) * 16);
  const uint32_t k_s32 = (uint32_t)p.k_s, v_s32 = (uint32_t)p.v_s;              // the host checks that they fit
  const uint32_t k_voff = (uint32_t)ld_row * k_s32 + ld_chunk, v_voff = (uint32_t)ld_row * v_s32 + ld_chunk;   // of a full tile's first load
  const uint32_t tiles_addr = (uint32_t)(uintptr_t)HBSA_AS3(lds) + (uint32_t)wave * 1024u;
  // LDS: three K tiles, then two V tiles.  K tiles are requested two tiles ahead, V tiles one (with two workgroups
  // of 5 tiles of D = 128 a CU's LDS is full).
  auto fetch_one = [&](uint32_t dst, const char *src, int64_t stride, uint32_t s32, uint32_t full_voff, int valid) {
    if (valid == kTileKeys) {   // a full tile: the loads differ in their scalar base only
#pragma unroll
      for (int i = 0; i < LOADS; ++i) bwd_dma16(dst + (uint32_t)(i * 4 * 1024), src + (int64_t)(4 * RPL * i) * stride, full_voff);
    } else {
#pragma unroll
      for (int i = 0; i < LOADS; ++i) {
        const uint32_t rr = (uint32_t)min(ld_row + 4 * RPL * i, valid - 1);   // rows past the end repeat the last one (masked later)
        bwd_dma16(dst + (uint32_t)(i * 4 * 1024), src, rr * s32 + ld_chunk);
      }
    }
  };
  auto fetch_k = [&](int kb, int at, int valid) {
    fetch_one(tiles_addr + (uint32_t)(kb * T::TILE_BYTES), kg + (int64_t)at * p.k_s, p.k_s, k_s32, k_voff, valid);
  };
  auto fetch_v = [&](int vb, int at, int valid) {
    fetch_one(tiles_addr + (uint32_t)((3 + vb) * T::TILE_BYTES), vg + (int64_t)at * p.v_s, p.v_s, v_s32, v_voff, valid);
  };
  // Operand addresses of the K tile in use: they move to the next buffer with one addition per tile instead of
  // one per read (the V tile's reads add the distance between the two buffers in use).
  BwdOperandOffsets<D> off;
  off.init(lane);
  {
    const uint32_t lds_base = (uint32_t)(uintptr_t)HBSA_AS3(lds);
#pragma unroll
    for (int ks = 0; ks < T::KSTEPS; ++ks) off.rows[ks] += lds_base;
#pragma unroll
    for (int dt = 0; dt < T::DT; ++dt) off.tr[dt] += lds_base;   // a multiple of 64: the second read's "^ 32" still holds
  }
  int off_buf = 0;   // the buffer they point to
  // Reads of one half tile's two chains S^T = K Q^T and dP^T = V dO^T: K and V rows in turn, PF under way
  constexpr int PF = 4, NC = 2 * T::KSTEPS;
  static_assert(NC >= PF, "the first reads of a half are issued as one group");
  static_assert(LOADS <= 15, "vmcnt immediate");
  // What was loaded so far (the rows' Q above all, first used in the loop) has arrived before the first tile is
  // requested: the compiler counts only the loads it knows, and a wait of its own for them inside the loop would
  // also wait for every tile under way.
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
  bool have_c = next_tile(), have_n = false;   // the current tile exists; the one after it exists (its K is requested)
  int kpos_c = 0, valid_c = 0, kpos_n = 0, valid_n = 0;
  int kb = 0, vb = 0;   // K and V buffer of the current tile
  if (have_c) {
    kpos_c = kpos;
    valid_c = tile_valid();
    fetch_k(0, kpos_c, valid_c);
    fetch_v(0, kpos_c, valid_c);
    have_n = next_tile();
    if (have_n) {
      kpos_n = kpos;
      valid_n = tile_valid();
      fetch_k(1, kpos_n, valid_n);
    }
  }
  while (have_c) {
    const int cur_kpos = kpos_c, valid = valid_c, cur_kb = kb, cur_vb = vb;
    // This wavefront's part of the tile has landed; the K loads of the tile after it (requested last; a
    // wavefront's loads return in order) may still be under way.
    if (have_n) __builtin_amdgcn_s_waitcnt(0x0F70 | LOADS);   // vmcnt(LOADS)
    else __builtin_amdgcn_s_waitcnt(0x0F70);                  // vmcnt(0)
    __syncthreads();   // ... every wavefront's, and the buffers of the tile before have been read by all
    if (have_n) fetch_v(vb ^ 1, kpos_n, valid_n);
    const bool have_nn = have_n && next_tile();
    kpos_c = kpos_n;
    valid_c = valid_n;
    have_c = have_n;
    if (have_nn) {
      kpos_n = kpos;
      valid_n = tile_valid();
      fetch_k(kb == 0 ? 2 : kb - 1, kpos_n, valid_n);   // two tiles ahead
    }
    have_n = have_nn;
    kb = kb == 2 ? 0 : kb + 1;
    vb ^= 1;
    if (!active) continue;
    if (off_buf != cur_kb) {
      const uint32_t step = (uint32_t)((cur_kb - off_buf) * T::TILE_BYTES);
#pragma unroll
      for (int ks = 0; ks < T::KSTEPS; ++ks) off.rows[ks] += step;
#pragma unroll
      for (int dt = 0; dt < T::DT; ++dt) off.tr[dt] += step;
      off_buf = cur_kb;
    }
    const uint32_t v_from_k = (uint32_t)((3 + cur_vb - cur_kb) * T::TILE_BYTES);   // from a K tile address to the V tile's
    int lim = valid;   // keys of the tile below lim are visible to this lane's row
    if (p.causal) lim = min(lim, lane_kvis - cur_kpos + 1);
    lim -= 4 * g32;
    short8v rb[PF];
    auto chain_read = [&](auto h_, auto i_) {
      constexpr int h = decltype(h_)::value, i = decltype(i_)::value;
      if constexpr (i & 1) rb[i % PF] = lds_read_b128<h * 32 * T::RB>(off.rows[i >> 1] + v_from_k);
      else rb[i % PF] = lds_read_b128<h * 32 * T::RB>(off.rows[i >> 1]);
    };
    // edge: some key of the tile is hidden from some row of the wavefront (the tile's end, or the causal
    // diagonal); elsewhere the per-element comparison and select are left out.  Rows past the block's end
    // have lse2 = +inf and so P = 0 either way.
    const bool edge = valid < kTileKeys || (p.causal && cur_kpos + valid - 1 > wave_kvis_min);
    auto half = [&](auto h_) {
      constexpr int h = decltype(h_)::value;
      f32x16 s, dp;
#pragma unroll
      for (int i = 0; i < 16; ++i) { s[i] = 0.f; dp[i] = 0.f; }
      static_for<0, NC>([&](auto i_) {
        constexpr int i = decltype(i_)::value;
        constexpr int ahead = (NC - 1 - i) < (PF - 1) ? (NC - 1 - i) : (PF - 1);
        lds_wait1<ahead>(rb[i % PF]);
        if constexpr (i & 1) dp = E::mfma(rb[i % PF], dof[i >> 1], dp);
        else s = E::mfma(rb[i % PF], qf[i >> 1], s);
        if constexpr (i + PF < NC) chain_read(h_, std::integral_constant<int, i + PF>{});
      });
      // The K^T operands of this half's first dQ products are on their way while the vector ALU forms dS, and
      // behind them (first half) the first reads of the second half's chains.
      short4v tb[2][2 * T::DT];
      bwd_issue_transposed<D, 2 * h>(off, 0u, tb[0]);
      if constexpr (h == 0)
        static_for<0, PF>([&](auto i_) { chain_read(std::integral_constant<int, 1>{}, i_); });
      short8v lo, hi;
      auto form_ds = [&](auto edge_) {
        float e[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], p.c, -lse2));
          if constexpr (decltype(edge_)::value) pv = 32 * h + 8 * (i >> 2) + (i & 3) < lim ? pv : 0.f;
          e[i] = pv * (dp[i] - dlt);
        }
        bwd_pack<E>(e, lo, hi);
      };
      if (edge) form_ds(std::true_type{});
      else form_ds(std::false_type{});
      // the second key group's operands travel during the first group's products (the registers for both
      // at once, next to dS in the making, are not there)
      bwd_issue_transposed<D, 2 * h + 1>(off, 0u, tb[1]);
      bwd_wait_transposed<D, 2 * T::DT + (h == 0 ? PF : 0)>(tb[0]);
      bwd_transposed_products<D, E>(tb[0], lo, acc);
      bwd_wait_transposed<D, 0>(tb[1]);
      bwd_transposed_products<D, E>(tb[1], hi, acc);
    };
    static_for<0, PF>([&](auto i_) { chain_read(std::integral_constant<int, 0>{}, i_); });
    half(std::integral_constant<int, 0>{});
    half(std::integral_constant<int, 1>{});
  }
  if (active && l32 < nrows)
    bwd_store_rows<D, E>(p.dq + (int64_t)(inf.row_begin + row0 + l32) * p.dq_s + (int64_t)hq * p.dq_h, acc, p.scale, g32);
}

// ---- dK, dV (head dims up to 64) ---------------------------------------------------------------------
// Four wavefronts; K^T and V^T of a wavefront's 32 keys stay in registers.  The Q and dO tiles go straight
// into LDS like the dQ kernel's (two buffers, one layout, one barrier per tile).  When the workgroup's keys
// fill at most two 32-key slots (k blocks of up to 64 keys, or the narrow rest of a wider block), two
// wavefronts share a slot and take the upper and lower 32 rows of every tile; their partial sums are added
// through LDS at the end, as in the D = 128 kernel below.
template <int D, typename E>
__global__ __launch_bounds__(kThreads, 2) void hbsa_bwd_dkv_kernel(BwdParams p) {
  static_assert(D <= 64, "head dim 128 has its own kernel");
  using T = BwdTile<D>;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  // buffer s of the tiles: Q rows at s * 2 * TILE_BYTES, dO rows one tile further
  float *rowv = (float *)(lds + 4 * T::TILE_BYTES);    // buffer s: [64] log2-domain log-sum-exp of the tile's rows, [64] their delta

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g32 = lane >> 5, l32 = lane & 31;
  // With a multiple of eight kv heads the grid is one-dimensional and workgroup ids, which go round the
  // eight XCDs (each with its own L2), are decoded so that XCD x works on the heads x, x + 8, ...: the
  // workgroups that share an L2 then walk the k blocks of one head in order and read the Q and dO rows of
  // one sequence at a time, and every XCD has the same amount of work whatever the sequence lengths.
  int hk = blockIdx.y, bx = blockIdx.x;
  if (p.xcd_heads) {
    const unsigned t = blockIdx.x >> 3, per_head = (unsigned)(p.nkb * p.nsub_k);
    hk = (int)(blockIdx.x & 7u) + 8 * (int)(t / per_head);
    bx = (int)(t % per_head);
  }
  const int kb = bx / p.nsub_k, sub = bx - kb * p.nsub_k;

  int b = 0;   // the sequence the k block belongs to
  while (b + 1 < p.batch && p.cu_num_k_block[b + 1] <= kb) ++b;
  if (bwd_sequence_skipped<D>(p, b, kb, sub, hk)) return;
  const int kbl = kb - p.cu_num_k_block[b];          // in-sequence index of the k block
  const int k0 = p.cu_k[b], klen = p.cu_k[b + 1] - k0;
  const int krows = min(p.kbs, klen - kbl * p.kbs);  // keys in the block
  const int wg_keys = min(4 * kWaveRows, p.kbs - sub * 4 * kWaveRows);   // by the block size: the same for every k block
  const bool shared_slots = wg_keys <= 2 * kWaveRows;                    // two wavefronts per 32-key slot
  const int slot = shared_slots ? (wave & 1) : wave;
  const int part = shared_slots ? (wave >> 1) : 0;                       // which 32 rows of a tile (shared slots)
  const int row0 = (sub * 4 + slot) * kWaveRows;
  const int nrows = min(kWaveRows, krows - row0);
  const bool active = nrows > 0;
  const int key_pos = kbl * p.kbs + min(row0 + l32, krows - 1);   // in-sequence position of this lane's key
  const int wg_first_key = kbl * p.kbs + sub * 4 * kWaveRows;     // of the workgroup's first key

  short8v kf[T::KSTEPS], vf[T::KSTEPS];   // K^T and V^T fragments: lane holds key l32, d = 16*ks + 8*g32 .. +7
  if (active) {
    const char *krow = p.k + (int64_t)(k0 + key_pos) * p.k_s + (int64_t)hk * p.k_h + g32 * 16;
    const char *vrow = p.v + (int64_t)(k0 + key_pos) * p.v_s + (int64_t)hk * p.v_h + g32 * 16;
#pragma unroll
    for (int ks = 0; ks < T::KSTEPS; ++ks) {
      kf[ks] = *(const short8v *)(krow + ks * 32);
      vf[ks] = *(const short8v *)(vrow + ks * 32);
    }
  } else {
#pragma unroll
    for (int ks = 0; ks < T::KSTEPS; ++ks) { kf[ks] = short8v{0, 0, 0, 0, 0, 0, 0, 0}; vf[ks] = kf[ks]; }
  }
  f32x16 acc_k[T::DT], acc_v[T::DT];
#pragma unroll
  for (int dt = 0; dt < T::DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) { acc_k[dt][i] = 0.f; acc_v[dt][i] = 0.f; }

  // the tile sequence: for every q block of the sequence that keeps this k block, for every q head of
  // the group, the block's rows in 64-row tiles (under a causal mask only those with a row that sees a
  // key of this workgroup)
  int qb = p.cu_num_q_block[b] - 1, r = 0, qoff = 0;
  const int qb_end = p.cu_num_q_block[b + 1];
  const int qb_begin = p.cu_num_q_block[b];
  int kept_base = qb_begin - 64;   // q blocks kept_base .. +63: those that keep this k block, not visited yet
  uint64_t kept = 0;
  QBlockInfo inf = {};
  int seq_row0 = 0, seq_qlen = 0;   // first query row and query count of the sequence
  if (qb_begin < qb_end) {
    const QBlockInfo first = p.info[qb_begin];
    seq_row0 = first.row_begin;
    seq_qlen = klen - first.shift;
    inf.shift = first.shift;
  }
  auto tile_reaches = [&]() {
    return !p.causal || inf.q_pos + qoff + min(64, inf.rows - qoff) - 1 + inf.shift >= wg_first_key;
  };
  auto next_tile = [&]() -> bool {
    for (;;) {
      if (qb >= qb_begin) {   // inside a kept q block: next tile, then next head
        qoff += 64;
        if (qoff >= inf.rows) { qoff = 0; ++r; }
        if (r < p.ratio) {
          if (tile_reaches()) return true;
          continue;
        }
      }
      while (kept == 0) {   // one load per 64 q blocks: lane i looks at q block kept_base + i
        kept_base += 64;
        if (kept_base >= qb_end) return false;
        uint32_t word = 0;
        if (kept_base + lane < qb_end) word = p.bits[((size_t)hk * p.nqb + kept_base + lane) * p.wpr + (kbl >> 5)];
        kept = __ballot((word >> (kbl & 31)) & 1u);
      }
      qb = kept_base + __builtin_ctzll(kept);
      kept &= kept - 1;
      // the q block's geometry follows from the sequence's (no load on this path)
      inf.q_pos = (qb - qb_begin) * p.qbs;
      inf.row_begin = seq_row0 + inf.q_pos;
      inf.rows = min(p.qbs, seq_qlen - inf.q_pos);
      r = 0;
      qoff = -64;   // the step above moves to the block's first tile
    }
  };
  // (placement of a tile's chunks over the four wavefronts: see hbsa_bwd_dq_kernel)
  constexpr int RPL = 1024 / T::RB, LOADS = 64 / (4 * RPL);
  const int ld_row = RPL * wave + lane / T::CPR;
  const uint32_t ld_chunk = (uint32_t)(((lane % T::CPR) ^ T::swz_both(ld_row)) * 16);
  const uint32_t q_s32 = (uint32_t)p.q_s, do_s32 = (uint32_t)p.do_s;   // the host checks that they fit
  const uint32_t tiles_addr = (uint32_t)(uintptr_t)HBSA_AS3(lds) + (uint32_t)wave * 1024u;
  float l2_next = INFINITY, dl_next = 0.f;   // threads 0-63: log2-domain log-sum-exp and delta of the tile's row
  auto fetch = [&](int buf) {
    const int valid = min(64, inf.rows - qoff);
    const int64_t row_first = inf.row_begin + qoff;
    const int hq = hk * p.ratio + r;
    const char *qsrc = p.q + row_first * p.q_s + (int64_t)hq * p.q_h;
    const char *gsrc = p.dout + row_first * p.do_s + (int64_t)hq * p.do_h;
    const uint32_t dst = tiles_addr + (uint32_t)(buf * 2 * T::TILE_BYTES);
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const uint32_t rr = (uint32_t)min(ld_row + 4 * RPL * i, valid - 1);   // rows past the block's end repeat its last row
      bwd_dma16(dst + (uint32_t)(i * 4 * 1024), qsrc, rr * q_s32 + ld_chunk);
      bwd_dma16(dst + (uint32_t)(T::TILE_BYTES + i * 4 * 1024), gsrc, rr * do_s32 + ld_chunk);
    }
    l2_next = INFINITY;   // rows past the block's end take no part: P = exp2(-inf) = 0
    dl_next = 0.f;
    if (threadIdx.x < valid) {
      const float l = p.lse[(row_first + threadIdx.x) * p.nhead_q + hq];
      l2_next = l == -INFINITY ? INFINITY : l * kLog2e;
      dl_next = p.delta[(row_first + threadIdx.x) * p.nhead_q + hq];
    }
  };
  bool have = next_tile();
  int buf = 0;
  if (have) fetch(0);
  while (have) {
    const int first_q_pos = inf.q_pos + qoff, shift = inf.shift;
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wavefront's part of the tile has landed (and its lse, delta)
    if (threadIdx.x < 64) {
      rowv[buf * 128 + threadIdx.x] = l2_next;
      rowv[buf * 128 + 64 + threadIdx.x] = dl_next;
    }
    __syncthreads();   // ... every wavefront's, and the other buffer has been read by all
    const char *q_t = lds + buf * 2 * T::TILE_BYTES, *g_t = q_t + T::TILE_BYTES;
    const float *lse_s = rowv + buf * 128, *dlt_s = lse_s + 64;
    have = next_tile();
    if (have) fetch(buf ^ 1);   // on its way while this tile is computed on
    buf ^= 1;
    if (!active) continue;
    // rows of the tile from first_vis on see this lane's key (causal); lanes past the block's keys see nothing
    int first_vis = 0;
    if (p.causal) first_vis = max(0, key_pos - shift - first_q_pos);
    if (l32 >= nrows) first_vis = 64;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      if (shared_slots && h != part) continue;   // the slot's other wavefront takes these rows
      const f32x16 s = bwd_rows_times_frag<D, E>(q_t, h, kf, lane);
      const f32x16 dp = bwd_rows_times_frag<D, E>(g_t, h, vf, lane);
      float ep[16], ed[16];
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const int rr0 = 32 * h + 8 * a + 4 * g32;
        const f32x4 l4 = *(const f32x4 *)(lse_s + rr0), d4 = *(const f32x4 *)(dlt_s + rr0);
#pragma unroll
        for (int bq = 0; bq < 4; ++bq) {
          const int i = 4 * a + bq;
          const bool vis = rr0 + bq >= first_vis;   // rows past the block's end carry lse = +inf, hence P = 0
          const float pv = vis ? __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], p.c, -l4[bq])) : 0.f;
          ep[i] = pv;
          ed[i] = pv * (dp[i] - d4[bq]);
        }
      }
      short8v plo, phi, dlo, dhi;
      bwd_pack<E>(ep, plo, phi);
      bwd_pack<E>(ed, dlo, dhi);
      bwd_transposed_times_packed<D, E>(g_t, 2 * h, plo, lane, acc_v);
      bwd_transposed_times_packed<D, E>(g_t, 2 * h + 1, phi, lane, acc_v);
      bwd_transposed_times_packed<D, E>(q_t, 2 * h, dlo, lane, acc_k);
      bwd_transposed_times_packed<D, E>(q_t, 2 * h + 1, dhi, lane, acc_k);
    }
  }
  if (shared_slots) {   // the wavefronts of the lower rows hand their sums to those of the upper rows: [slot][register][lane] floats
    __syncthreads();
    float *xch = (float *)lds + (size_t)slot * (2 * T::DT * 16) * 64 + lane;
    if (part == 1) {
#pragma unroll
      for (int dt = 0; dt < T::DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          xch[(dt * 16 + i) * 64] = acc_k[dt][i];
          xch[((T::DT + dt) * 16 + i) * 64] = acc_v[dt][i];
        }
    }
    __syncthreads();
    if (part == 0) {
#pragma unroll
      for (int dt = 0; dt < T::DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          acc_k[dt][i] += xch[(dt * 16 + i) * 64];
          acc_v[dt][i] += xch[((T::DT + dt) * 16 + i) * 64];
        }
    }
  }
  if (part == 0 && active && l32 < nrows) {
    const int64_t row = k0 + kbl * p.kbs + row0 + l32;
    bwd_store_rows<D, E>(p.dk + row * p.dk_s + (int64_t)hk * p.dk_h, acc_k, p.scale, g32);
    bwd_store_rows<D, E>(p.dv + row * p.dv_s + (int64_t)hk * p.dv_h, acc_v, 1.f, g32);
  }
}

// ---- dK, dV at D = 128: eight wavefronts in two roles -------------------------------------------------
// The kernel above would hold K^T, V^T and both accumulators of a wavefront in registers: 256 + 238 at
// D = 128, one wavefront per SIMD.  Here two wavefronts share a 32-key slot (and a SIMD) and split the four
// products between them, each with one operand and one accumulator in registers:
//   the P wavefront  keeps K^T:  S = Q K^T,  P = exp(S - lse) (masked),   dV^T += dO^T P,   hands P over;
//   the dS wavefront keeps V^T:  dP = dO V^T,  dS = P * (dP - delta),      dK^T += Q^T dS.
// P travels through LDS in the element type, as the P wavefront packs it for its own product (4 KB per slot and
// tile), and one tile late: in the iteration in which the P wavefront works on tile t, the dS wavefront
// finishes tile t - 1 (whose dP it kept in registers) and forms dP of tile t, so one barrier per tile orders
// everything.  Tiles go from global memory straight into LDS, stored once in the layout of BwdTile::swz_both,
// and two tiles ahead (one workgroup per CU has nobody else to cover its waits for memory): four Q buffers
// (tile t - 1 is still read while tile t + 2 arrives), three for dO, and with them three and four sets of the
// rows' log-sum-exp and delta, which wavefront 0 loads into LDS the same way.
template <typename E>
__global__ __launch_bounds__(512, 1) void hbsa_bwd_dkv8_kernel(BwdParams p) {
  constexpr int D = 128;
  using T = BwdTile<D>;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  char *q_buf = lds;                                   // [4] Q tiles
  char *g_buf = lds + 4 * T::TILE_BYTES;               // [3] dO tiles
  char *p_buf = lds + 7 * T::TILE_BYTES;               // [2 tile parities][4 slots][2 halves][2][64 lanes] eight 16-bit values
  float *lse_s = (float *)(lds + 9 * T::TILE_BYTES);   // [3][64] log2-domain log-sum-exp of the tile's rows (index: the dO buffer's)
  float *dlt_s = lse_s + 192;                          // [4][64] their delta (index: the Q buffer's)

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slot = wave & 3, role = wave >> 2;   // 32-key slot of the workgroup; 0: the P wavefront, 1: the dS wavefront
  const int g32 = lane >> 5, l32 = lane & 31;
  // With a multiple of eight kv heads the grid is one-dimensional and workgroup ids, which go round the
  // eight XCDs (each with its own L2), are decoded so that XCD x works on the heads x, x + 8, ...: the
  // workgroups that share an L2 then walk the k blocks of one head in order and read the Q and dO rows of
  // one sequence at a time, and every XCD has the same amount of work whatever the sequence lengths.
  int hk = blockIdx.y, bx = blockIdx.x;
  if (p.xcd_heads) {
    const unsigned t = blockIdx.x >> 3, per_head = (unsigned)(p.nkb * p.nsub_k);
    hk = (int)(blockIdx.x & 7u) + 8 * (int)(t / per_head);
    bx = (int)(t % per_head);
  }
  const int kb = bx / p.nsub_k, sub = bx - kb * p.nsub_k;

  int b = 0;   // the sequence the k block belongs to
  while (b + 1 < p.batch && p.cu_num_k_block[b + 1] <= kb) ++b;
  if (bwd_sequence_skipped<D>(p, b, kb, sub, hk)) return;
  const int kbl = kb - p.cu_num_k_block[b];
  const int k0 = p.cu_k[b], klen = p.cu_k[b + 1] - k0;
  const int krows = min(p.kbs, klen - kbl * p.kbs);
  const int wg_row0 = sub * 4 * kWaveRows;                 // first key of the workgroup inside the block
  const int row0 = wg_row0 + slot * kWaveRows;
  const int nrows = min(kWaveRows, krows - row0);
  const bool active = nrows > 0;
  const int key_pos = kbl * p.kbs + min(row0 + l32, krows - 1);
  const int wg_first_key = kbl * p.kbs + wg_row0;
  const int wave_key_max = kbl * p.kbs + min(row0 + kWaveRows - 1, krows - 1);   // position of the wavefront's last key

  // this wavefront's resident operand: K^T (P wavefront) or V^T (dS wavefront) of its 32 keys; lane holds
  // key l32, d = 16 * ks + 8 * g32 .. + 7
  short8v frag[T::KSTEPS];
  if (active) {
    const char *src = role == 0 ? p.k + (int64_t)(k0 + key_pos) * p.k_s + (int64_t)hk * p.k_h
                                : p.v + (int64_t)(k0 + key_pos) * p.v_s + (int64_t)hk * p.v_h;
#pragma unroll
    for (int ks = 0; ks < T::KSTEPS; ++ks) frag[ks] = *(const short8v *)(src + g32 * 16 + ks * 32);
  } else {
#pragma unroll
    for (int ks = 0; ks < T::KSTEPS; ++ks) frag[ks] = short8v{0, 0, 0, 0, 0, 0, 0, 0};
  }
  f32x16 acc[T::DT];   // dV^T (P wavefront) or dK^T (dS wavefront) of the 32 keys
#pragma unroll
  for (int dt = 0; dt < T::DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;

  int qb = p.cu_num_q_block[b] - 1, r = 0, qoff = 0;
  const int qb_end = p.cu_num_q_block[b + 1];
  const int qb_begin = p.cu_num_q_block[b];
  int kept_base = qb_begin - 64;   // q blocks kept_base .. +63: those that keep this k block, not visited yet
  uint64_t kept = 0;
  QBlockInfo inf = {};
  int seq_row0 = 0, seq_qlen = 0;   // first query row and query count of the sequence
  if (qb_begin < qb_end) {
    const QBlockInfo first = p.info[qb_begin];
    seq_row0 = first.row_begin;
    seq_qlen = klen - first.shift;
    inf.shift = first.shift;
  }
  auto tile_reaches = [&]() {
    return !p.causal || inf.q_pos + qoff + min(64, inf.rows - qoff) - 1 + inf.shift >= wg_first_key;
  };
  auto next_tile = [&]() -> bool {
    for (;;) {
      if (qb >= qb_begin) {
        qoff += 64;
        if (qoff >= inf.rows) { qoff = 0; ++r; }
        if (r < p.ratio) {
          if (tile_reaches()) return true;
          continue;
        }
      }
      while (kept == 0) {   // one load per 64 q blocks: lane i looks at q block kept_base + i; waited for here so that no other path waits
        kept_base += 64;
        if (kept_base >= qb_end) return false;
        uint32_t word = 0;
        if (kept_base + lane < qb_end) word = p.bits[((size_t)hk * p.nqb + kept_base + lane) * p.wpr + (kbl >> 5)];
        __builtin_amdgcn_s_waitcnt(0x0F70);
        kept = __ballot((word >> (kbl & 31)) & 1u);
      }
      qb = kept_base + __builtin_ctzll(kept);
      kept &= kept - 1;
      // the q block's geometry follows from the sequence's (no load on this path)
      inf.q_pos = (qb - qb_begin) * p.qbs;
      inf.row_begin = seq_row0 + inf.q_pos;
      inf.rows = min(p.qbs, seq_qlen - inf.q_pos);
      r = 0;
      qoff = -64;
    }
  };
  // A tile's 1024 chunks over eight wavefronts: wavefront w fills rows 4 * (8 * i + w) .. + 3 with load i
  // (i = 0, 1), lane l the 16 bytes at chunk position l % 16 of row l / 16 of those, which hold the
  // row's chunk (l % 16) ^ swz_both(row).
  const int ld_row = 4 * wave + (lane >> 4);                              // + 32 * i
  const uint32_t ld_chunk = (uint32_t)(((lane & 15) ^ T::swz_both(ld_row & 15)) * 16);
  const uint32_t q_s32 = (uint32_t)p.q_s, do_s32 = (uint32_t)p.do_s;      // the host checks that they fit
  const uint32_t q_addr = (uint32_t)(uintptr_t)HBSA_AS3(q_buf) + (uint32_t)wave * 1024u;
  const uint32_t g_addr = (uint32_t)(uintptr_t)HBSA_AS3(g_buf) + (uint32_t)wave * 1024u;
  const uint32_t q_voff = (uint32_t)ld_row * q_s32 + ld_chunk, g_voff = (uint32_t)ld_row * do_s32 + ld_chunk;   // of a full tile's first load
  const uint32_t row_addr = (uint32_t)(uintptr_t)HBSA_AS3(lse_s);
  // Loads of one tile per wavefront: two Q and two dO loads, and in wavefront 0 the two loads of the rows' values
  auto fetch = [&](int qi, int gi) {   // the tile next_tile() has moved to, into Q buffer qi and dO buffer gi
    const int valid = min(64, inf.rows - qoff);
    const int64_t row_first = inf.row_begin + qoff;
    const int hq = hk * p.ratio + r;
    const char *qsrc = p.q + row_first * p.q_s + (int64_t)hq * p.q_h;
    const char *gsrc = p.dout + row_first * p.do_s + (int64_t)hq * p.do_h;
    if (valid == 64) {   // a full tile: the loads differ in their scalar base only
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        bwd_dma16(q_addr + (uint32_t)(qi * T::TILE_BYTES + i * 8 * 1024), qsrc + (int64_t)(32 * i) * p.q_s, q_voff);
        bwd_dma16(g_addr + (uint32_t)(gi * T::TILE_BYTES + i * 8 * 1024), gsrc + (int64_t)(32 * i) * p.do_s, g_voff);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint32_t rr = (uint32_t)min(ld_row + 32 * i, valid - 1);   // rows past the block's end repeat its last row
        bwd_dma16(q_addr + (uint32_t)(qi * T::TILE_BYTES + i * 8 * 1024), qsrc, rr * q_s32 + ld_chunk);
        bwd_dma16(g_addr + (uint32_t)(gi * T::TILE_BYTES + i * 8 * 1024), gsrc, rr * do_s32 + ld_chunk);
      }
    }
    if (wave == 0) {   // the rows' log-sum-exp and delta, one row per lane (rows past the block's end repeat its last row)
      const uint32_t rvoff = (uint32_t)min(lane, valid - 1) * (uint32_t)(p.nhead_q * 4);
      bwd_dma4(row_addr + (uint32_t)(gi * 256), p.lse2 + row_first * p.nhead_q + hq, rvoff);
      bwd_dma4(row_addr + (uint32_t)(768 + qi * 256), p.delta + row_first * p.nhead_q + hq, rvoff);
    }
  };
  // this lane's 2 x 16 bytes of a (tile parity, slot, half) record of P
  char *p_mine = p_buf + (size_t)slot * 4096 + lane * 16;

  BwdOperandOffsets<D> off;
  off.init(lane);
  const uint32_t lds_base = (uint32_t)(uintptr_t)HBSA_AS3(lds);   // Q tiles at 0 .. 3 tile sizes, dO tiles at 4 .. 6
  // The loop exists once per role (the same barriers in both): with the roles as branches of one loop body the
  // register allocator keeps both roles' temporaries apart and spills.
  auto run = [&](auto role_) {
  constexpr int ROLE = decltype(role_)::value;
  // Tiles are fetched two ahead: tile t lives in Q buffer t % 4 and dO buffer t % 3 (the dS wavefront still reads
  // Q of tile t - 1 in the iteration in which tile t + 2 arrives).
  int n_ahead = 0;                               // tiles fetched and not computed on yet
  int qi_f = 0, gi_f = 0;                        // buffers of the next fetch
  int fq_a = 0, fq_b = 0, va_a = 64, va_b = 64;  // first query position and row count of those tiles (a: the older)
  // Everything loaded so far (the resident operand above all) has arrived before the first tile is requested: the
  // compiler counts only the loads it knows, and a wait of its own for them inside the loop would also wait for
  // every tile under way.
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
  bool more = next_tile();
  auto issue = [&]() {   // fetches the tile next_tile() stands on and moves on
    const int fq = inf.q_pos + qoff, va = min(64, inf.rows - qoff);
    if (n_ahead == 0) { fq_a = fq; va_a = va; } else { fq_b = fq; va_b = va; }
    fetch(qi_f, gi_f);
    qi_f = (qi_f + 1) & 3;
    gi_f = gi_f == 2 ? 0 : gi_f + 1;
    ++n_ahead;
    more = next_tile();
  };
  if (more) issue();
  if (more) issue();
  bool prev = false;        // the tile before the current one exists: its dK part is still due
  int qi = 0, gi = 0, par = 0;   // Q buffer, dO buffer and parity of the current tile
  f32x16 dp_prev[2];        // dS wavefront: dP of the previous tile, both halves
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int i = 0; i < 16; ++i) dp_prev[h][i] = 0.f;
  const int shift = inf.shift;
  while (n_ahead > 0 || prev) {
    const bool had = n_ahead > 0;
    const int first_q_pos = fq_a, valid = va_a;   // of the current tile (if any)
    // This wavefront's part of the current tile has landed; the loads of the tile after it (a wavefront's loads
    // return in order) may still be under way.
    if (n_ahead >= 2) {
      if (wave == 0) __builtin_amdgcn_s_waitcnt(0x0F76);   // vmcnt(6)
      else __builtin_amdgcn_s_waitcnt(0x0F74);             // vmcnt(4)
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);                  // vmcnt(0)
    }
    __syncthreads();   // ... every wavefront's; what the iteration before read and wrote is settled
    const int q_now = qi, q_before = (qi + 3) & 3;
    if (had) {
      fq_a = fq_b;
      va_a = va_b;
      --n_ahead;
      if (more) issue();   // two tiles ahead: the buffers it fills were last read an iteration ago
    }
    if (active) {
      // Operand reads are issued by hand (BwdOperandOffsets): PF reads of a pair of chains under way ahead of
      // their products, the transposing reads of a key group before the vector ALU work that precedes their
      // products.  The counts in the waits name only reads that every path issues.
      constexpr int PF = 4, NC = 2 * T::KSTEPS;
      short8v rb[PF];
      short4v tb[2][2 * T::DT];
      if constexpr (ROLE == 0) {
        if (had) {   // ---- P wavefront, current tile
          const uint32_t q_t = lds_base + (uint32_t)(q_now * T::TILE_BYTES), g_t = lds_base + (uint32_t)((4 + gi) * T::TILE_BYTES);
          int first_vis = 0;   // rows of the tile from first_vis on see this lane's key (causal)
          if (p.causal) first_vis = max(0, key_pos - shift - first_q_pos);
          if (l32 >= nrows) first_vis = 64;
          // S = Q K^T of both halves of the tile, their steps in turn (read i: half i % 2, step i / 2)
          auto chain_read = [&](auto i_) {
            constexpr int i = decltype(i_)::value;
            rb[i % PF] = lds_read_b128<(i & 1) * 32 * T::RB>(off.rows[i >> 1] + q_t);
          };
          static_for<0, PF>(chain_read);
          f32x16 sv[2];
#pragma unroll
          for (int i = 0; i < 16; ++i) { sv[0][i] = 0.f; sv[1][i] = 0.f; }
          static_for<0, NC>([&](auto i_) {
            constexpr int i = decltype(i_)::value;
            constexpr int ahead = (NC - 1 - i) < (PF - 1) ? (NC - 1 - i) : (PF - 1);
            lds_wait1<ahead>(rb[i % PF]);
            sv[i & 1] = E::mfma(rb[i % PF], frag[i >> 1], sv[i & 1]);
            if constexpr (i + PF < NC) chain_read(std::integral_constant<int, i + PF>{});
          });
          bwd_issue_transposed<D, 0>(off, g_t, tb[0]);
          bwd_issue_transposed<D, 1>(off, g_t, tb[1]);
          // edge: some row of the tile does not see some key of the wavefront (the causal diagonal, a slot with
          // fewer than 32 keys, a tile with fewer than 64 rows); elsewhere the per-element comparison and select
          // are left out.
          const bool edge = nrows < kWaveRows || valid < 64 || (p.causal && wave_key_max - shift - first_q_pos > 0);
          auto half = [&](auto h_) {
            constexpr int h = decltype(h_)::value;
            float ep[16];
            auto form_p = [&](auto edge_) {
#pragma unroll
              for (int a = 0; a < 4; ++a) {
                const int rr0 = 32 * h + 8 * a + 4 * g32;
                const f32x4 l4 = *(const f32x4 *)(lse_s + gi * 64 + rr0);
#pragma unroll
                for (int bq = 0; bq < 4; ++bq) {
                  float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[h][4 * a + bq], p.c, -l4[bq]));
                  if constexpr (decltype(edge_)::value) pv = (rr0 + bq >= first_vis && rr0 + bq < valid) ? pv : 0.f;   // rows past the block's end repeat its last row
                  ep[4 * a + bq] = pv;
                }
              }
            };
            if (edge) form_p(std::true_type{});
            else form_p(std::false_type{});
            short8v plo, phi;
            bwd_pack<E>(ep, plo, phi);
            *(short8v *)(p_mine + par * 16384 + h * 2048) = plo;
            *(short8v *)(p_mine + par * 16384 + h * 2048 + 1024) = phi;
            bwd_wait_transposed<D, 2 * T::DT>(tb[0]);
            bwd_transposed_products<D, E>(tb[0], plo, acc);
            if constexpr (h == 0) bwd_issue_transposed<D, 2>(off, g_t, tb[0]);
            bwd_wait_transposed<D, (h == 0 ? 2 * T::DT : 0)>(tb[1]);
            bwd_transposed_products<D, E>(tb[1], phi, acc);
            if constexpr (h == 0) bwd_issue_transposed<D, 3>(off, g_t, tb[1]);
          };
          half(std::integral_constant<int, 0>{});
          half(std::integral_constant<int, 1>{});
        }
      } else {
        const uint32_t q_t = lds_base + (uint32_t)(q_before * T::TILE_BYTES), g_t = lds_base + (uint32_t)((4 + gi) * T::TILE_BYTES);
        auto chain_read = [&](auto i_) {   // dP = dO V^T of both halves of the current tile, as above
          constexpr int i = decltype(i_)::value;
          rb[i % PF] = lds_read_b128<(i & 1) * 32 * T::RB>(off.rows[i >> 1] + g_t);
        };
        if (prev) {   // ---- dS wavefront, the tile before: dS = P * (dP - delta), dK^T += Q^T dS
          bwd_issue_transposed<D, 0>(off, q_t, tb[0]);
          bwd_issue_transposed<D, 1>(off, q_t, tb[1]);
          auto half = [&](auto h_) {
            constexpr int h = decltype(h_)::value;
            float ed[16];
            const u32x4 pw[2] = {*(const u32x4 *)(p_mine + (par ^ 1) * 16384 + h * 2048),
                                 *(const u32x4 *)(p_mine + (par ^ 1) * 16384 + h * 2048 + 1024)};
#pragma unroll
            for (int a = 0; a < 4; ++a) {
              const int rr0 = 32 * h + 8 * a + 4 * g32;
              const f32x4 d4 = *(const f32x4 *)(dlt_s + q_before * 64 + rr0);
#pragma unroll
              for (int bq = 0; bq < 4; ++bq) {
                const uint32_t w = pw[a >> 1][2 * (a & 1) + (bq >> 1)];
                const float pv = (bq & 1) ? E::hi(w) : E::lo(w);
                ed[4 * a + bq] = pv * (dp_prev[h][4 * a + bq] - d4[bq]);
              }
            }
            short8v dlo, dhi;
            bwd_pack<E>(ed, dlo, dhi);
            bwd_wait_transposed<D, 2 * T::DT>(tb[0]);
            bwd_transposed_products<D, E>(tb[0], dlo, acc);
            if constexpr (h == 0) bwd_issue_transposed<D, 2>(off, q_t, tb[0]);
            bwd_wait_transposed<D, (h == 0 ? 2 * T::DT : 0)>(tb[1]);
            bwd_transposed_products<D, E>(tb[1], dhi, acc);
            if constexpr (h == 0) bwd_issue_transposed<D, 3>(off, q_t, tb[1]);
          };
          half(std::integral_constant<int, 0>{});
          half(std::integral_constant<int, 1>{});
        }
        if (had) {   // ---- dS wavefront, current tile: dP = dO V^T, kept for the next iteration
          static_for<0, PF>(chain_read);
#pragma unroll
          for (int i = 0; i < 16; ++i) { dp_prev[0][i] = 0.f; dp_prev[1][i] = 0.f; }
          static_for<0, NC>([&](auto i_) {
            constexpr int i = decltype(i_)::value;
            constexpr int ahead = (NC - 1 - i) < (PF - 1) ? (NC - 1 - i) : (PF - 1);
            lds_wait1<ahead>(rb[i % PF]);
            dp_prev[i & 1] = E::mfma(rb[i % PF], frag[i >> 1], dp_prev[i & 1]);
            if constexpr (i + PF < NC) chain_read(std::integral_constant<int, i + PF>{});
          });
        }
      }
    }
    prev = had;
    qi = (qi + 1) & 3;
    gi = gi == 2 ? 0 : gi + 1;
    par ^= 1;
  }
  if (active && l32 < nrows) {
    const int64_t row = k0 + kbl * p.kbs + row0 + l32;
    if constexpr (ROLE == 0) bwd_store_rows<D, E>(p.dv + row * p.dv_s + (int64_t)hk * p.dv_h, acc, 1.f, g32);
    else bwd_store_rows<D, E>(p.dk + row * p.dk_s + (int64_t)hk * p.dk_h, acc, p.scale, g32);
  }
  };
  if (role == 0) run(std::integral_constant<int, 0>{});
  else run(std::integral_constant<int, 1>{});
}

template <int D, typename E>
int launch_bwd(const BwdParams &bp, int nhead_k, int num_k_block, hipStream_t stream) {
  using T = BwdTile<D>;
  // LDS: the dQ kernel's three K and two V tiles; the dK/dV kernels' tile buffers, P records and row values
  const int lds_dq = 5 * T::TILE_BYTES, lds_dkv = D == 128 ? 9 * T::TILE_BYTES + 2048 : 4 * T::TILE_BYTES + 1024;
  if (lds_dkv > 48 * 1024) {
    static thread_local bool raised[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
      return fail(HBSA_ERR_UNSUPPORTED, "no current device, or device index above %d", kMaxDevices - 1);
    if (!raised[dev]) {
      const void *dkv = nullptr;
      if constexpr (D == 128) dkv = reinterpret_cast<const void *>(&hbsa_bwd_dkv8_kernel<E>);
      else dkv = reinterpret_cast<const void *>(&hbsa_bwd_dkv_kernel<D, E>);
      hipError_t e = hipFuncSetAttribute(dkv, hipFuncAttributeMaxDynamicSharedMemorySize, lds_dkv);
      if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&hbsa_bwd_dq_kernel<D, E>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, lds_dq);
      if (e != hipSuccess) return (int)e;
      raised[dev] = true;
    }
  }
  const dim3 q_grid = bp.xcd_heads ? dim3((unsigned)(bp.nqb * bp.nsub * nhead_k)) : dim3((unsigned)(bp.nqb * bp.nsub), (unsigned)nhead_k);
  hipLaunchKernelGGL((hbsa_bwd_dq_kernel<D, E>), q_grid, dim3(kThreads), lds_dq, stream, bp);
  const dim3 kv_grid = bp.xcd_heads ? dim3((unsigned)(num_k_block * bp.nsub_k * nhead_k))
                                    : dim3((unsigned)(num_k_block * bp.nsub_k), (unsigned)nhead_k);
  if constexpr (D == 128) {
    hipLaunchKernelGGL((hbsa_bwd_dkv8_kernel<E>), kv_grid, dim3(512),
                       lds_dkv, stream, bp);
  } else {
    hipLaunchKernelGGL((hbsa_bwd_dkv_kernel<D, E>), kv_grid,
                       dim3(kThreads), lds_dkv, stream, bp);
  }
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

}  // namespace
