// Flash-attention forward, f16 in / f16 out, head dimension 64, no mask.
//
// Reference: test/Integration/Dialect/XeGPU/WG/flash_attention_fwd.mlir
//   kernel :25-307 -- per workgroup a 128 x 64 Q tile, K/V walked in 64-key
//   blocks, online softmax (running max m, running sum l, accumulator rescaled by
//   exp(m_old - m_new)), P truncated to f16 before P.V, O = acc / l at the end;
//   CPU check :332-421 -- softmax(scale * Q K^T) V per (batch, head), Q/K/V/O stored
//   as [(Z*H*N_CTX), 64] row-major.
//
// On MI355X the products are formed TRANSPOSED, so that a lane owns one query:
//   S^T[key, q] = K_tile . Q^T     A operand = K rows (k-contiguous in LDS),
//                                  B operand = Q rows, loaded once into registers;
//   O^T[d, q]  += V_tile^T . P^T   A operand = V^T via the LDS transpose read,
//                                  B operand = P^T straight from the S^T
//                                  accumulator registers (no shuffles: the MFMA's
//                                  k index is bound to the keys in the order the
//                                  accumulator holds them, and V^T is read in
//                                  the same order).
// With v_mfma_f32_32x32x16_f16 a lane holds query q = lane % 32 and, per 32-key
// block, keys (r/4)*8 + (lane/32)*4 + r%4: the softmax max and sum over keys are
// plain register loops plus ONE exchange between lane l and l+32 per block of
// keys.
//
// Workgroup = QB query blocks of 32 x KG key groups, one wavefront each: 64, 128 or 256
// queries of one (batch, head) as (QB, KG) = (2,4), (4,2), (8,1) with 512 threads, or 256
// queries as (8,2) with 1024 threads.  Wavefront w takes query block w % QB and every KG-th
// 64-key tile, group w / QB; partial (m, l, O) of the key groups are merged through LDS at the
// end.  Every workgroup walks all keys of its head, so K / V traffic from L2 falls with the
// queries per workgroup; key groups exist to keep all CUs busy on small problems (the
// reference's 2 x 2 x 4096 x 64 gives one 64-query workgroup per CU) and, in the 1024-thread
// form, to put four wavefronts on every SIMD (the tiled path needs 114 registers).  The launch
// says which: N_CTX / gridDim.x queries per workgroup, blockDim.x threads.  K and V blocks of
// 64 KG keys go from global memory straight into an LDS ring (buffer_load ... lds) of 2, 4 or
// 8 stages, up to seven blocks ahead.
//
// Arguments: (Q, K, V, Out, sm_scale: f32, ZH: i64, N_CTX: i64)   dims = {ZH, N_CTX}
//   ZH = batch * heads; all four tensors [(ZH*N_CTX), 64]; sm_scale > 0.  N_CTX need not divide the
//   tiles: queries past the end are not stored, keys past the end get a score of -inf.
// Launch: grid (ceil(N_CTX / q), ZH, 1) with q = 64, 128 or 256 and block (512,1,1), or q = 256
// and block (1024,1,1).  Other launches (and a scale <= 0, or misaligned tensors) take the
// one-query-per-lane reference loop of the same kernel (grid-stride, any grid and block).

#include "device_common.h"

using namespace imexhip;

namespace {

constexpr int kMaxThreads = 1024; // 8 or 16 wavefronts per workgroup
constexpr int D = 64;                 // head dimension
constexpr int BN = 64;                // keys per tile; a ring stage holds one K and one V tile per key group
constexpr int kTileBytes = BN * D * 2;          // 8 KiB
constexpr int kLdsBytes = 128 * 1024;           // the ring: 2 stages of 64 KiB, 4 of 32 KiB or 8 of 16 KiB

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4 LdsI16x4;
typedef __attribute__((address_space(3))) char LdsChar;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, int64_t bytes) {
  const int range = bytes > 0x7fffffff ? 0x7fffffff : int(bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, range, 0x00020000);
}
template <int N> __device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}
// the value lane l+32 (or l-32) holds
__device__ __forceinline__ float other_half(float v) { return __shfl_xor(v, 32, 64); }

// ---- any-shape path: one lane per query, the reference loop ----------------------------
__device__ __forceinline__ void attention_scalar(const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                                                 uint16_t *Out, float scale, int64_t ZH, int64_t N) {
  const int64_t block = int64_t(blockIdx.z) * gridDim.y * gridDim.x + int64_t(blockIdx.y) * gridDim.x + blockIdx.x;
  const int64_t stride = int64_t(gridDim.x) * gridDim.y * gridDim.z * blockDim.x;
  const float c = scale * 1.44269504088896341f;
  for (int64_t row = block * blockDim.x + threadIdx.x; row < ZH * N; row += stride) {
    const int64_t head0 = (row / N) * N;
    float o[D]; // the query row is re-read per key (it stays in cache): 64 registers, not 128
    for (int d = 0; d < D; ++d)
      o[d] = 0.0f;
    float m = -__builtin_inff(), l = 0.0f;
    for (int64_t j = 0; j < N; ++j) {
      float s = 0.0f;
      for (int d = 0; d < D; ++d)
        s += half_bits_to_float(Q[row * D + d]) * half_bits_to_float(K[(head0 + j) * D + d]);
      s *= c;
      const float mNew = fmaxf(m, s);
      const float alpha = exp2f(m - mNew);
      const float p = half_bits_to_float(float_to_half_bits(exp2f(s - mNew)));
      l = l * alpha + p;
      for (int d = 0; d < D; ++d)
        o[d] = o[d] * alpha + p * half_bits_to_float(V[(head0 + j) * D + d]);
      m = mNew;
    }
    for (int d = 0; d < D; ++d)
      Out[row * D + d] = static_cast<uint16_t>(float_to_half_bits(o[d] / l));
  }
}

// ---- MFMA path ---------------------------------------------------------------------------
// QB = 32-query blocks per workgroup, KG = key groups: QB x KG wavefronts (8 or 16).  More query
// blocks mean fewer workgroups but proportionally less K / V traffic from L2 (every workgroup walks
// all keys of its head); fewer key groups mean smaller ring stages and therefore a deeper ring.
// kRagged: N_CTX is not a multiple of the workgroup's 32 QB queries or of its 64 KG-key blocks; the
// padding logic below is compiled in only then.
template <int QB, int KG, bool kRagged>
__device__ __forceinline__ void attention_tiled(const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K,
                                                const uint16_t *__restrict__ V, uint16_t *__restrict__ Out,
                                                float scale, int64_t N, char *lds) {
  LdsChar *ldsBase = (LdsChar *)lds;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr int kWaves = QB * KG;
  constexpr int kStageBytes = 2 * KG * kTileBytes; // K tiles of all key groups, then their V tiles
  constexpr int kStages = kLdsBytes / kStageBytes; // 2, 4 or 8
  constexpr int kAhead = kStages - 1;              // blocks in flight ahead of the one being multiplied
  constexpr int kCopies = 64 * KG / (8 * kWaves);  // 1 KiB (8-row) copies per wavefront, stage and operand
  const int wq = wave % QB, wk = wave / QB;
  const int qi = lane & 31, half = lane >> 5;
  // Workgroups go to the 8 XCDs round-robin in launch order, and each XCD has its own L2.  Renumber
  // them so that one XCD gets consecutive query blocks -- whole heads, or a contiguous part of one --
  // and its L2 holds the K / V of a few heads instead of a slice of the traffic of all of them.
  uint32_t bx = blockIdx.x, by = blockIdx.y;
  {
    const uint32_t total = gridDim.x * gridDim.y, launched = by * gridDim.x + bx;
    if (total % 8 == 0) {
      const uint32_t logical = (launched & 7) * (total >> 3) + (launched >> 3);
      by = logical / gridDim.x;
      bx = logical - by * gridDim.x;
    }
  }
  const int64_t head0 = int64_t(by) * N;                 // first row of this (batch, head)
  const int64_t q0 = head0 + int64_t(bx) * (32 * QB) + wq * 32;
  // N_CTX need not divide the tiles.  Queries past the end of the head are computed on a copy of
  // its last row and not stored; keys past the end are copies of the last key whose scores are
  // set to -inf before the softmax (below), so no address ever leaves the head.
  const int64_t qRow = kRagged ? min(q0 + qi, head0 + N - 1) : q0 + qi;

  // Q^T operand: lane (q, half) keeps Q[q][ds*16 + half*8 .. +7] for the four 16-wide steps
  f16x8 qf[4];
#pragma unroll
  for (int ds = 0; ds < 4; ++ds)
    qf[ds] = *reinterpret_cast<const f16x8 *>(Q + qRow * D + ds * 16 + half * 8);

  // -- global -> LDS copies.  A stage is [K tile 0 .. KG-1][V tile 0 .. KG-1], each 64
  // rows of 128 bytes; one copy = 8 rows.  16-byte chunk c of row r is stored at
  //   K: c ^ ((r ^ (r>>3 & 3)) & 7)   (conflict-free 128-bit fragment reads; same for r and r+32)
  //   V: c ^ (((r>>1) & 1) << 2)     (conflict-free transpose reads)
  // applied on the global side, since a direct copy fixes the lane's LDS position.
  const __amdgpu_buffer_rsrc_t kRsrc = make_rsrc(K + head0 * D, N * D * 2);
  const __amdgpu_buffer_rsrc_t vRsrc = make_rsrc(V + head0 * D, N * D * 2);
  const int iters = int((N + KG * BN - 1) / (KG * BN));            // key blocks of 64 KG keys
  const int lastRows = int(N - int64_t(iters - 1) * (KG * BN));    // keys in the last block: 1 .. 64 KG
  const bool raggedKeys = kRagged && lastRows != KG * BN;
  int kVoff[kCopies], vVoff[kCopies];   // per-lane byte offsets inside a block
  int kVoffT[kCopies], vVoffT[kCopies]; // the same for the last block, rows clamped to its last key
#pragma unroll
  for (int c = 0; c < kCopies; ++c) {
    // wavefront w copies rows [8 kCopies w, 8 kCopies (w+1)) of the stage's 64 KG K rows and of its V rows
    const int row = wave * (8 * kCopies) + c * 8 + (lane >> 3); // key within the stage's block of 64 KG keys
    const int r = row & 63;                          // row within its tile
    const int kc = (lane & 7) ^ ((r ^ ((r >> 3) & 3)) & 7);
    const int vc = (lane & 7) ^ (((r >> 1) & 1) << 2);
    kVoff[c] = (row * D + kc * 8) * 2;
    vVoff[c] = (row * D + vc * 8) * 2;
    const int rowT = kRagged ? min(row, lastRows - 1) : row;
    kVoffT[c] = (rowT * D + kc * 8) * 2;
    vVoffT[c] = (rowT * D + vc * 8) * 2;
  }
  auto dma_stage = [&](int block, int stage) { // keys [64 KG block, 64 KG (block + 1)) into ring stage `stage`
    LdsChar *dst = ldsBase + stage * kStageBytes + wave * (kCopies * 1024);
    const int soff = block * (KG * BN * D * 2);
    const bool tail = raggedKeys && block == iters - 1; // uniform
#pragma unroll
    for (int c = 0; c < kCopies; ++c)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(kRsrc, dst + c * 1024, 16, tail ? kVoffT[c] : kVoff[c], soff, 0, 0);
#pragma unroll
    for (int c = 0; c < kCopies; ++c)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(vRsrc, dst + KG * kTileBytes + c * 1024, 16,
                                               tail ? vVoffT[c] : vVoff[c], soff, 0, 0);
  };

  // -- LDS read addresses (relative to this wavefront's K / V tile of a stage)
  // K fragment (key block kb, step ds): row kb*32 + qi, logical chunk ds*2 + half
  int kRd[4];
#pragma unroll
  for (int ds = 0; ds < 4; ++ds) {
    const int r = qi; // the swizzle term is the same for rows r and r + 32
    kRd[ds] = wk * kTileBytes + r * 128 + ((((ds * 2 + half) ^ r ^ ((r >> 3) & 3)) & 7) << 4);
  }
  // V^T fragment (d block db, key step kk): two transpose reads.  Lane t of a 16-lane group
  // supplies the address of 4 consecutive d at key row (base + t/4) and receives 4 consecutive
  // key rows of d = t.  Key rows of element e of the operand: kk*16 + (e/4)*8 + half*4 + e%4 --
  // the order in which the S^T accumulator holds the keys.
  int vRd[2];
  {
    const int t = lane & 15, blk = (lane >> 4) & 1;
    const int row = half * 4 + (t >> 2);
#pragma unroll
    for (int db = 0; db < 2; ++db) {
      const int chunk = ((db ^ ((t >> 3) & 1)) << 2) | (blk << 1) | ((t & 3) >> 1);
      vRd[db] = KG * kTileBytes + wk * kTileBytes + row * 128 + chunk * 16 + (t & 1) * 8;
    }
  }

  f32x16 o[2];
#pragma unroll
  for (int db = 0; db < 2; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      o[db][r] = 0.0f;
  float m = -__builtin_inff(); // running max of scale*log2(e)*s over this lane's query (both halves agree)
  float l = 0.0f;              // running sum of p over THIS lane's keys only
  const float c = scale * 1.44269504088896341f;

  // The ring always holds kAhead blocks in flight (past the end the last block is simply fetched
  // again, into stages nobody reads any more), so "block `it` has landed" is one fixed vmcnt.
#pragma unroll
  for (int b = 0; b < kAhead; ++b)
    dma_stage(min(b, iters - 1), b);
  int cur = 0; // ring stage of block `it`
  for (int it = 0; it < iters; ++it) {
    wait_vmcnt<(kAhead - 1) * 2 * kCopies>(); // block `it` has landed (this wavefront's copies)
    __builtin_amdgcn_s_barrier();             // ... everyone's; and everyone is done reading block it-1
    __builtin_amdgcn_sched_barrier(0);
    dma_stage(min(it + kAhead, iters - 1), cur == 0 ? kStages - 1 : cur - 1); // into the stage block it-1 occupied
    const char *st = lds + cur * kStageBytes;

    // S^T = K . Q^T for this wavefront's 64 keys (the first product of each chain takes a
    // literal zero accumulator, so no registers are cleared)
    f32x16 s[2];
    {
      const f32x16 zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
      f16x8 kf[2][4];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int ds = 0; ds < 4; ++ds)
          kf[kb][ds] = *reinterpret_cast<const f16x8 *>(st + kRd[ds] + kb * 32 * 128);
      // the two accumulator chains alternate, so no MFMA waits for the one just issued
#pragma unroll
      for (int ds = 0; ds < 4; ++ds)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
          s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[kb][ds], qf[ds], ds == 0 ? zero : s[kb], 0, 0, 0);
    }
    // keys of this wavefront's tile that exist: fewer than 64 only in the last block of a ragged N_CTX
    const int nValid = int(N) - (it * (KG * BN) + wk * BN);
    if (kRagged && nValid < BN) { // uniform over the wavefront
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          s[kb][r] = kb * 32 + (r >> 2) * 8 + half * 4 + (r & 3) < nValid ? s[kb][r] : -__builtin_inff();
    }
    // online softmax over the keys; this lane owns 32 of the query's 64 scores
    float mx = s[0][0];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        mx = fmaxf(mx, s[kb][r]);
    mx = fmaxf(mx, other_half(mx));
    const float mRun = fmaxf(m, mx * c);
    // a key group that has seen no key yet (ragged N_CTX shorter than its first tile) stays at -inf;
    // 0 stands in for it below so that -inf - -inf never forms: every p and alpha is then exp2(-inf) = 0
    const float mNew = kRagged && mRun == -__builtin_inff() ? 0.0f : mRun;
    const float alpha = __builtin_amdgcn_exp2f(m - mNew);
    m = mRun;
    float sum = 0.0f;
    f16x8 pf[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kk >> 1][(kk & 1) * 8 + e], c, -mNew)); // one fused op per score
        pf[kk][e] = static_cast<_Float16>(p); // the reference truncates P to f16 before P.V (:262-265)
        sum += p;                             // ... and sums the untruncated f32 values (:243-247)
      }
    }
    l = l * alpha + sum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) { // the running max moved for some query of this wavefront
#pragma unroll
      for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          o[db][r] *= alpha;
    }
    // O^T += V^T . P^T
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
      for (int db = 0; db < 2; ++db) {
        const char *p = st + vRd[db] + kk * 16 * 128;
        const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsI16x4 *)(p));
        const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsI16x4 *)(p + 8 * 128));
        const f16x8 vf = __builtin_bit_cast(f16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[kk], o[db], 0, 0, 0);
      }
    }
    cur = cur == kStages - 1 ? 0 : cur + 1;
  }
  wait_vmcnt<0>();
  l += other_half(l); // both key halves of the lane pair

  // -- merge the key groups through LDS: groups 1.. hand (m, l, O^T) to group 0
  __syncthreads(); // the ring is free
  constexpr int kSlot = 34 * 64; // floats per (query half, key group): 32 accumulator rows, m, l
  float *xchg = reinterpret_cast<float *>(lds) + wq * (KG - 1) * kSlot;
  if (wk != 0) {
    float *mine = xchg + (wk - 1) * kSlot;
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        mine[(db * 16 + r) * 64 + lane] = o[db][r];
    mine[32 * 64 + lane] = m;
    mine[33 * 64 + lane] = l;
  }
  __syncthreads();
  if (wk == 0) {
    float mAll = m;
#pragma unroll
    for (int g = 0; g < KG - 1; ++g)
      mAll = fmaxf(mAll, xchg[g * kSlot + 32 * 64 + lane]);
    float a[KG];
    a[0] = exp2f(m - mAll);
    float lAll = l * a[0];
#pragma unroll
    for (int g = 0; g < KG - 1; ++g) {
      a[g + 1] = exp2f(xchg[g * kSlot + 32 * 64 + lane] - mAll);
      lAll += xchg[g * kSlot + 33 * 64 + lane] * a[g + 1];
    }
    const float inv = 1.0f / lAll;
    // lane holds, for query q = qi, d = db*32 + (r/4)*8 + half*4 + r%4
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        f16x4 out4;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = g4 * 4 + e;
          float acc = o[db][r] * a[0];
#pragma unroll
          for (int g = 0; g < KG - 1; ++g)
            acc += xchg[g * kSlot + (db * 16 + r) * 64 + lane] * a[g + 1];
          out4[e] = static_cast<_Float16>(acc * inv);
        }
        if (!kRagged || q0 + qi < head0 + N)
          *reinterpret_cast<f16x4 *>(Out + (q0 + qi) * D + db * 32 + g4 * 8 + half * 4) = out4;
      }
  }
}

} // namespace

extern "C" __global__ __launch_bounds__(kMaxThreads) void imex_flash_attention_fwd_f16(const uint16_t *Q,
                                                                                   const uint16_t *K,
                                                                                   const uint16_t *V,
                                                                                   uint16_t *Out, float sm_scale,
                                                                                   int64_t ZH, int64_t N_CTX) {
  __shared__ __attribute__((aligned(16))) char lds[kLdsBytes];
  // The launch says how many queries a workgroup takes (ceil(N_CTX / gridDim.x) = 64, 128 or 256) and
  // with how many wavefronts.  The tiled path assumes a positive scale (it takes the row maximum
  // before scaling) and 32-bit byte offsets inside one head.
  const bool shaped = N_CTX > 0 && N_CTX < (int64_t(1) << 24) && sm_scale > 0.0f && gridDim.y == ZH && gridDim.z == 1 &&
                      ((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K) |
                        reinterpret_cast<uintptr_t>(V) | reinterpret_cast<uintptr_t>(Out)) & 15) == 0;
  const int64_t gx = gridDim.x;
  const bool even = N_CTX % 256 == 0; // every tiling divides it
  if (shaped && blockDim.x == 512 && gx == (N_CTX + 63) / 64) {
    if (even)
      attention_tiled<2, 4, false>(Q, K, V, Out, sm_scale, N_CTX, lds);
    else
      attention_tiled<2, 4, true>(Q, K, V, Out, sm_scale, N_CTX, lds);
  } else if (shaped && blockDim.x == 512 && gx == (N_CTX + 127) / 128) {
    if (even)
      attention_tiled<4, 2, false>(Q, K, V, Out, sm_scale, N_CTX, lds);
    else
      attention_tiled<4, 2, true>(Q, K, V, Out, sm_scale, N_CTX, lds);
  } else if (shaped && blockDim.x == 512 && gx == (N_CTX + 255) / 256) {
    if (even)
      attention_tiled<8, 1, false>(Q, K, V, Out, sm_scale, N_CTX, lds);
    else
      attention_tiled<8, 1, true>(Q, K, V, Out, sm_scale, N_CTX, lds);
  } else if (shaped && blockDim.x == 1024 && gx == (N_CTX + 255) / 256) {
    if (even)
      attention_tiled<8, 2, false>(Q, K, V, Out, sm_scale, N_CTX, lds);
    else
      attention_tiled<8, 2, true>(Q, K, V, Out, sm_scale, N_CTX, lds);
  } else {
    attention_scalar(Q, K, V, Out, sm_scale, ZH, N_CTX);
  }
}
