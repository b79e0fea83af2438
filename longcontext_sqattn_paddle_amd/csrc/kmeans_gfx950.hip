// KV k-means clustering and centroid-scored token selection for gfx950 (MI355X).
//
// Replaces the reference's Triton kernels in cache_hub/kmeans.py:
//   _triton_assign_kernel :7-79, _triton_update_kernel :82-124, _triton_k_means_train :127-196,
//   _triton_reverse_index_kernel :199-262, _triton_index_add_kernel :265-329.
// The reference scatters every token into its cluster sum with fp32 atomics (16.8 M atomics per head and
// iteration at 131072 x 128).  Here the assignment is a dense bf16 MFMA contraction with an arg-max
// epilogue in registers, tokens are then grouped by cluster tile by tile and every cluster is summed by one
// workgroup in fp64, which is exact for bf16 data and therefore independent of order -- and of how the sums were
// arrived at: a run of iterations may keep them in the workspace and apply only the tokens that changed cluster
// (sq_kmeans_train_stateful).  A counting sort in ascending token order yields the reverse index.
#include "common.hpp"

namespace sq {
namespace {

constexpr int kD = 128;
constexpr int kCB = 64;            // centroids per LDS stage
constexpr int kTileTok = 256;      // tokens per workgroup in assign / sort kernels
constexpr int kMaxC = 8192;

// ------------------------------------------------------------------------------------------ fill
__global__ void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = v;
}

// ---------------------------------------------------------------------------------------- assign
struct AssignArgs {
  const uint16_t* data;  // [G,N,128] bf16
  const uint16_t* cent;  // [G,C,128] bf16
  int32_t* idx;          // [G,N]
  int64_t d_sg, d_sn, c_sg, c_sc, i_sg;
  int32_t N, C;
  double* keep_sum;      // TRACK: [G,C,128] the clusters' exact sums, carried from the previous step
  int32_t* keep_cnt;     // TRACK: [G,C] and their sizes
};

constexpr int kAssignWaves = 4;   // x 64 tokens; two workgroups per CU put two waves on every SIMD

// Workgroup = 256 tokens of one group, 64 per wave (two 32-token operand sets in registers): every centroid fragment
// read from LDS feeds two MFMAs, which halves the LDS traffic per MFMA -- with 32 tokens per wave the fragment reads
// of the four SIMDs add up to the LDS's whole 128 bytes per cycle.  Centroids stream through LDS in blocks of 64
// (global_load_lds, unpadded rows, 16-byte chunks XOR-swizzled by row so that the MFMA operand reads are conflict
// free), double buffered with one barrier per block; the arg-max over one half block's scores runs underneath the
// MFMAs of the next half block (see `phase` below).
// TRACK: the sums that are carried across iterations.  After the first few Lloyd iterations hardly any token changes its
// cluster (configuration 4: 1 % in the fourth iteration, 0.1 % in the tenth), yet a full re-sum reads every row again.
// The sums are exact (fp64 of bf16 values), so they can be carried: `idx` holds the previous iteration's assignment on
// entry, and a token whose cluster changes is subtracted from its old cluster's sum and added to its new one's, in any
// order, by fp64 atomics that round nothing -- the result is the sum a full re-sum would give, bit for bit.  The
// workgroup lists its movers in LDS and applies them itself at the end (one channel per thread, the first 128 threads
// adding, the others subtracting); kmeans_update_kernel then turns sums and sizes into centroids.
template <bool TRACK>
__global__ __launch_bounds__(kAssignWaves * 64, 1) void kmeans_assign_kernel(AssignArgs a) {
  __shared__ __attribute__((aligned(16))) char smem[2 * kCB * 256];
  __shared__ int32_t s_chg_n;
  __shared__ uint2 s_chg[TRACK ? kTileTok : 1];   // (token, old cluster << 16 | new cluster)
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  const int g_id = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, g = lane >> 5;
  const int tok0 = blockIdx.x * kTileTok + wave * 64;

  // token fragments (B operand of S^T = Cent . Data^T): lane (column = token 32 tb + c32, k-group g)
  const uint16_t* db = a.data + (int64_t)g_id * a.d_sg;
  uint4 tf[2][8];
#pragma unroll
  for (int tb = 0; tb < 2; ++tb) {
    const int n = min(tok0 + 32 * tb + c32, a.N - 1);
    const uint16_t* rp = db + (int64_t)n * a.d_sn + 8 * g;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) tf[tb][kk] = *(const uint4*)(rp + 16 * kk);
  }
  int old_idx[2] = {-1, -1};
  if constexpr (TRACK) {   // requested now, needed at the very end
    if (tid == 0) s_chg_n = 0;   // (the block loop below passes at least one barrier before anyone adds to it)
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      const int n = tok0 + 32 * tb + c32;
      if (n < a.N) old_idx[tb] = a.idx[(int64_t)g_id * a.i_sg + n];
    }
  }
  const uint16_t* cb = a.cent + (int64_t)g_id * a.c_sg;
  // per-lane source of the wave's four 1 KB copies of a block (4 centroid rows each), as a byte offset from the block's
  // first row; rows past C are clamped to the last centroid, which only a block that runs past C has to do
  int64_t src_off[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int row = 4 * (wave * 4 + c) + (lane >> 4);
    src_off[c] = ((int64_t)row * a.c_sc + 8 * ((lane & 15) ^ (row & 15))) * 2;
  }
  auto stage = [&](int chunk, int st) {
    char* buf = smem + st * (kCB * 256);
    const char* blk = (const char*)cb + (int64_t)chunk * kCB * a.c_sc * 2;
    if ((chunk + 1) * kCB <= a.C) {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        __builtin_amdgcn_global_load_lds((const void*)(blk + src_off[c]), (lds_ptr_t)(buf + (wave * 4 + c) * 1024), 16, 0, 0);
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int q = wave * 4 + c;
        const int row = 4 * q + (lane >> 4);
        const int ch = (lane & 15) ^ (row & 15);
        const int crow = min(chunk * kCB + row, a.C - 1);
        __builtin_amdgcn_global_load_lds((const void*)(cb + (int64_t)crow * a.c_sc + 8 * ch), (lds_ptr_t)(buf + q * 1024), 16, 0, 0);
      }
    }
  };
  // Fragment number n = 8 half + kk of a block: centroid row 32 half + c32, 16-byte chunk (2 kk + g) ^ (row & 15).  The
  // reads go through lds_read128 / lds_wait (explicit lgkmcnt counts): left to the compiler, every wait was a full
  // lgkmcnt(0), i.e. also for the fragments requested a moment ago.
  const int ksw = c32 & 15;
  const uint32_t smem_addr = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
  uint32_t fa[8];
#pragma unroll
  for (int kk = 0; kk < 8; ++kk) fa[kk] = smem_addr + c32 * 256 + (((2 * kk + g) ^ ksw) << 4);
  auto frag = [&](uint32_t boff, auto NUM) {
    constexpr int n = decltype(NUM)::value;
    return lds_read128<(n >> 3) * 8192>(fa[n & 7] + boff);
  };
  // Running arg-max in ascending centroid order with strict '>' = lowest index on ties (kmeans.py:62-65), four scores
  // at a time: the group's maximum (v_max3 + v_max) is compared with the running best; a group that wins leaves its
  // id and its first three scores behind, from which the position inside the group follows at the end (the first score
  // equal to the best; if none of the three, the fourth).  Eight vector instructions per four scores instead of
  // twelve.  Rows past C (C % 64 == 32) are clamped copies of the last centroid; they come after it in this order and
  // can never beat it strictly.
  float best[2] = {-INFINITY, -INFINITY};
  float keep0[2] = {0.f, 0.f}, keep1[2] = {0.f, 0.f}, keep2[2] = {0.f, 0.f};
  int bgrp[2] = {0, 0}, bhalf[2] = {0, 0};
  // S[tb][h]: scores of token set tb against centroid half h (32 centroids) of the current block.  A block is
  // computed in two phases of 16 MFMAs, half 0 then half 1, each as two accumulator chains (tb = 0, 1) over the eight
  // 16-wide slices of the dimension.  Underneath the MFMAs of one phase runs the arg-max over the results of the
  // previous phase, as one hand-ordered instruction stream: an MFMA occupies the matrix pipe for 32 cycles, half a
  // group's arg-max (four vector instructions) issues behind it.  The accumulators are not double-buffered; with
  // the MFMAs in their VGPR form (build flag) the arg-max reads them without copies out of the accumulation registers.
  f32x16_t S[2][2];
#pragma unroll
  for (int tb = 0; tb < 2; ++tb)
#pragma unroll
    for (int i = 0; i < 16; ++i) S[tb][1][i] = -INFINITY;   // "previous phase" of the very first one
  // One group of four scores against the running best, as one instruction block in the short encodings with the
  // condition in VCC (the compiler's form of the same selects is a masked block of moves behind s_and_saveexec):
  // VCC = not (m > best); a group that wins leaves its id and its first three scores behind.
  auto group_step = [&](const f32x16_t& P, int tb, auto Q) {
    constexpr int q = decltype(Q)::value;
    float m;
    float &b = best[tb], &k0 = keep0[tb], &k1 = keep1[tb], &k2 = keep2[tb];
    int& grp = bgrp[tb];
    asm volatile(
        "v_max3_f32 %[m], %[p0], %[p1], %[p2]\n\t"
        "v_max_f32_e32 %[m], %[m], %[p3]\n\t"
        "v_cmp_le_f32_e32 vcc, %[m], %[best]\n\t"
        "v_cndmask_b32_e32 %[k0], %[p0], %[k0], vcc\n\t"
        "v_cndmask_b32_e32 %[k1], %[p1], %[k1], vcc\n\t"
        "v_cndmask_b32_e32 %[k2], %[p2], %[k2], vcc\n\t"
        "v_cndmask_b32_e32 %[grp], %[qq], %[grp], vcc\n\t"
        "v_max_f32_e32 %[best], %[best], %[m]"
        : [m] "=&v"(m), [best] "+v"(b), [k0] "+v"(k0), [k1] "+v"(k1), [k2] "+v"(k2), [grp] "+v"(grp)
        : [p0] "v"(P[4 * q]), [p1] "v"(P[4 * q + 1]), [p2] "v"(P[4 * q + 2]), [p3] "v"(P[4 * q + 3]), [qq] "n"(q)
        : "vcc");
  };
  // The 16 centroid fragments of a block (half h, slice kk -> number 8 h + kk) are requested kFragAhead steps before
  // the MFMA pair that uses them: an LDS read takes longer than one pair of MFMAs when eight waves read at once.
  constexpr int kFragAhead = 3;
  auto phase = [&](auto H, uint32_t boff, int half_id, u32x4_t (&fr)[16]) {
    constexpr int h = decltype(H)::value;   // centroid half computed now; the arg-max runs over half 1 - h
    const float before0 = best[0], before1 = best[1];
    static_for<0, 8>([&](auto KK) {
      constexpr int kk = decltype(KK)::value;
      constexpr int cur = 8 * h + kk, nxt = cur + kFragAhead;
      if constexpr (nxt < 16) fr[nxt] = frag(boff, std::integral_constant<int, nxt>{});
      lds_wait<(15 - cur < kFragAhead ? 15 - cur : kFragAhead)>(fr[cur]);
      const bf16x8_t af = __builtin_bit_cast(bf16x8_t, fr[cur]);
      static_for<0, 2>([&](auto TB) {
        constexpr int tb = decltype(TB)::value;
        const bf16x8_t t = __builtin_bit_cast(bf16x8_t, tf[tb][kk]);
        if constexpr (kk == 0) {
          const f32x16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          S[tb][h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, t, zero, 0, 0, 0);
        } else {
          S[tb][h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, t, S[tb][h], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        // group kk of the previous phase's 8 groups (token set kk >> 2, scores 4 (kk & 3) .. + 3), behind the first
        // MFMA of the pair
        constexpr int ctb = kk >> 2, q = kk & 3;
        if constexpr (tb == 0) group_step(S[ctb][1 - h], ctb, std::integral_constant<int, q>{});
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    // the scores just examined belong to the half before this one
    bhalf[0] = (best[0] > before0) ? half_id - 1 : bhalf[0];
    bhalf[1] = (best[1] > before1) ? half_id - 1 : bhalf[1];
  };
  const int nchunks = (a.C + kCB - 1) / kCB;
  stage(0, 0);
  for (int chunk = 0; chunk < nchunks; ++chunk) {
    __builtin_amdgcn_s_waitcnt(0);
    // block `chunk` has landed for every wave, and every wave has finished reading block chunk - 1, whose buffer the
    // next block may now overwrite; it has this block's 32 MFMAs per wave to arrive
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    if (chunk + 1 < nchunks) stage(chunk + 1, (chunk + 1) & 1);
    const uint32_t boff = (chunk & 1) * (kCB * 256);
    u32x4_t fr[16];
    static_for<0, kFragAhead>([&](auto I) { fr[decltype(I)::value] = frag(boff, I); });
    __builtin_amdgcn_sched_barrier(0);
    phase(std::integral_constant<int, 0>{}, boff, 2 * chunk, fr);
    phase(std::integral_constant<int, 1>{}, boff, 2 * chunk + 1, fr);
  }
  {   // the last half block
    const float before0 = best[0], before1 = best[1];
    static_for<0, 2>([&](auto TB) {
      static_for<0, 4>([&](auto Q) { group_step(S[decltype(TB)::value][1], decltype(TB)::value, Q); });
    });
    bhalf[0] = (best[0] > before0) ? 2 * nchunks - 1 : bhalf[0];
    bhalf[1] = (best[1] > before1) ? 2 * nchunks - 1 : bhalf[1];
  }
#pragma unroll
  for (int tb = 0; tb < 2; ++tb) {
    const int in_group = (keep0[tb] == best[tb]) ? 0 : (keep1[tb] == best[tb]) ? 1 : (keep2[tb] == best[tb]) ? 2 : 3;
    int bidx = bhalf[tb] * 32 + 4 * g + 8 * bgrp[tb] + in_group;
    float bv = best[tb];
    const float ob = __shfl_xor(bv, 32);
    const int oi = __shfl_xor(bidx, 32);
    if (ob > bv || (ob == bv && oi < bidx)) {
      bv = ob;
      bidx = oi;
    }
    const int n = tok0 + 32 * tb + c32;
    // cluster sizes come out of the counting sort that follows (per-tile histograms), not out of global atomics
    if (g == 0 && n < a.N) a.idx[(int64_t)g_id * a.i_sg + n] = bidx;
    if constexpr (TRACK) {
      const bool changed = g == 0 && n < a.N && old_idx[tb] != bidx;
      const unsigned long long m = __ballot(changed);
      if (m != 0) {   // wave-uniform
        int base = 0;
        if (lane == 0) base = atomicAdd(&s_chg_n, __popcll(m));
        base = __shfl(base, 0);
        if (changed) {
          const int pos = base + __popcll(m & ((1ull << lane) - 1ull));
          s_chg[pos] = make_uint2((uint32_t)n, ((uint32_t)old_idx[tb] << 16) | (uint32_t)bidx);
        }
      }
    }
  }
  if constexpr (TRACK) {
    __syncthreads();
    const int n_chg = s_chg_n;
    if (n_chg == 0) return;
    const int ch = tid & (kD - 1);
    const bool adds = tid < kD;
    const uint16_t* drow = db + ch;
    double* sg = a.keep_sum + (int64_t)g_id * a.C * kD + ch;
    int32_t* cg = a.keep_cnt + (int64_t)g_id * a.C;
    for (int i = 0; i < n_chg; ++i) {
      const uint2 e = s_chg[i];
      const int c = adds ? (int)(e.y & 0xffffu) : (int)(e.y >> 16);
      if (c >= a.C) continue;   // (an old assignment that is no cluster: nothing to take it out of)
      const double x = (double)bf16_bits_to_f32(drow[(int64_t)e.x * a.d_sn]);
      unsafeAtomicAdd(sg + (int64_t)c * kD, adds ? x : -x);
      if (ch == 0) atomicAdd(cg + c, adds ? 1 : -1);
    }
  }
}

// ------------------------------------------------------------------------- counting sort by cluster
struct SortArgs {
  const int32_t* idx;     // [G,N]
  int32_t* tile_hist;     // [G,nT,C]  in: per-tile histogram, after scan: exclusive prefix over tiles
  int32_t* total;         // [G,C]     cluster sizes (written by the scan)
  int32_t* dst;           // clusters [G,C,M]
  int64_t i_sg, dst_sg, dst_sc;
  int32_t N, C, nT, M;
};

__global__ __launch_bounds__(kTileTok) void sort_hist_kernel(SortArgs a) {
  extern __shared__ int32_t hist[];
  const int tile = blockIdx.x, g = blockIdx.y;
  for (int c = threadIdx.x; c < a.C; c += blockDim.x) hist[c] = 0;
  __syncthreads();
  const int n = tile * kTileTok + threadIdx.x;
  if (n < a.N) {
    const int c = a.idx[(int64_t)g * a.i_sg + n];
    if (c >= 0 && c < a.C) atomicAdd(&hist[c], 1);
  }
  __syncthreads();
  int32_t* out = a.tile_hist + ((int64_t)g * a.nT + tile) * a.C;
  for (int c = threadIdx.x; c < a.C; c += blockDim.x) out[c] = hist[c];
}

// Exclusive prefix over tiles of every cluster's per-tile count.  Workgroup = 32 clusters x 32 tile segments:
// each thread sums its segment, the 32 segment sums are scanned through LDS, then each thread rewrites its segment.
constexpr int kScanSegs = 32;
__global__ __launch_bounds__(32 * kScanSegs) void sort_scan_tiles_kernel(SortArgs a) {
  __shared__ int32_t seg_sum[kScanSegs][32];
  const int cl = threadIdx.x & 31, seg = threadIdx.x >> 5;
  const int c = blockIdx.x * 32 + cl, g = blockIdx.y;
  const int per = (a.nT + kScanSegs - 1) / kScanSegs;
  const int tb = seg * per, te = min(tb + per, a.nT);
  int32_t* h = a.tile_hist + (int64_t)g * a.nT * a.C + c;
  int sum = 0;
  if (c < a.C)
    for (int t = tb; t < te; ++t) sum += h[(int64_t)t * a.C];
  seg_sum[seg][cl] = sum;
  __syncthreads();
  int run = 0, total = 0;
#pragma unroll
  for (int q = 0; q < kScanSegs; ++q) {
    const int v = seg_sum[q][cl];
    if (q < seg) run += v;
    total += v;
  }
  if (c >= a.C) return;
  for (int t = tb; t < te; ++t) {
    const int v = h[(int64_t)t * a.C];
    h[(int64_t)t * a.C] = run;
    run += v;
  }
  if (seg == 0) a.total[(int64_t)g * a.C + c] = total;
}

__global__ __launch_bounds__(kTileTok) void sort_scatter_kernel(SortArgs a) {
  __shared__ int32_t cl[kTileTok];
  const int tile = blockIdx.x, g = blockIdx.y, t = threadIdx.x;
  const int n = tile * kTileTok + t;
  const int c = (n < a.N) ? a.idx[(int64_t)g * a.i_sg + n] : -1;
  cl[t] = c;
  __syncthreads();
  if (c < 0 || c >= a.C) return;
  int rank = 0;
  for (int u = 0; u < t; ++u) rank += (cl[u] == c);   // tokens of a tile keep their ascending order
  const int base = a.tile_hist[((int64_t)g * a.nT + tile) * a.C + c] + rank;
  if (base < a.M) a.dst[(int64_t)g * a.dst_sg + (int64_t)c * a.dst_sc + base] = n;
}

// Grouping without a global order, for the callers that only sum the rows of a cluster afterwards (centroid update,
// index_add): those sums are exact, so neither the order of the addends nor where a cluster's tokens lie matters.  A
// workgroup sorts its own tile of kBigTile tokens by cluster and nothing else: LDS histogram (the atomic's return value is
// the token's rank inside its (tile, cluster) range), exclusive prefix over the clusters, token ids written to
// order[tile * kBigTile + start[c] + rank].  start[tile][0..C] goes to memory; the sum kernel of cluster c walks the
// tiles and picks up order[tile][start[c] .. start[c + 1]) from each.  One launch, no pass that depends on all tiles.
//
// Clusters are summed by one workgroup each, so a cluster that has swallowed a large part of the tokens (the second
// Lloyd iteration from evenly spaced seeds does that: 50 000 of 131 072 tokens in one cluster, 0.5 ms in one workgroup)
// would hold up the whole step.  Tiles all have the same number of tokens, so the tile's workgroup takes that work: a
// (tile, cluster) range of kHeavy tokens or more is summed right here, in fp64, into rec[tile][start / kHeavy][128]
// (ranges that long cannot share a block of kHeavy positions, so the slot is unique), and the cluster's workgroup adds
// the records instead of the rows.
constexpr int kBigTok = 2;          // tokens per thread
constexpr int kBigTile = 1024 * kBigTok;        // tokens per workgroup
constexpr int kHeavy = 64;                      // tokens of one cluster in one tile from which the tile sums them itself
constexpr int kSlots = kBigTile / kHeavy;

struct GroupArgs {
  const int32_t* idx;     // [G,N]
  const uint16_t* src;    // [G,N,128] bf16 rows that will be summed
  int32_t* start;         // [G,nT,C+1]
  int32_t* order;         // [G,N]
  double* rec;            // [G,nT,kSlots,128]
  int64_t i_sg, s_sg, s_sn;
  int32_t N, C, nT;
};

__device__ __forceinline__ void add_row_bf16(double (&acc)[8], const uint4& raw) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t bits = (e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu);
    acc[e] += (double)bf16_bits_to_f32(bits);
  }
}

__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int o = __shfl_up(v, d);
    if (lane >= d) v += o;
  }
  return v;
}

constexpr int kMaxItems = 2 * kSlots;   // pieces of at most kHeavy rows: sum over ranges of ceil(m / kHeavy) <= kBigTile / kHeavy + ranges

__global__ __launch_bounds__(1024) void tile_group_kernel(GroupArgs a) {
  extern __shared__ double racc[];       // [kSlots][128] sums of the long ranges; then C counters / start positions; then the sorted ids
  __shared__ int32_t wsum[16];
  __shared__ int32_t item[kMaxItems][3]; // (first position, rows, slot) of a piece of a long range
  __shared__ int32_t used[kSlots];
  __shared__ int32_t n_items;
  int32_t* hist = (int32_t*)(racc + kSlots * kD);
  int32_t* ids = hist + a.C;
  const int tile = blockIdx.x, g = blockIdx.y, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  int c[kBigTok], rank[kBigTok];
#pragma unroll
  for (int u = 0; u < kBigTok; ++u) {
    const int n = tile * kBigTile + u * 1024 + t;
    c[u] = (n < a.N) ? a.idx[(int64_t)g * a.i_sg + n] : -1;
    if (c[u] >= a.C) c[u] = -1;
  }
  for (int i = t; i < a.C; i += 1024) hist[i] = 0;
  for (int i = t; i < kSlots * kD; i += 1024) racc[i] = 0;
  if (t < kSlots) used[t] = 0;
  if (t == 0) n_items = 0;
  __syncthreads();
#pragma unroll
  for (int u = 0; u < kBigTok; ++u) rank[u] = (c[u] >= 0) ? atomicAdd(&hist[c[u]], 1) : 0;
  __syncthreads();
  int32_t* out = a.start + ((int64_t)g * a.nT + tile) * (a.C + 1);
  int carry = 0;
  for (int c0 = 0; c0 < a.C; c0 += 1024) {
    const int i = c0 + t;
    const int v = (i < a.C) ? hist[i] : 0;
    const int inc = wave_inclusive_scan(v, lane);
    if (lane == 63) wsum[wave] = inc;
    __syncthreads();
    int wbase = 0, all = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int x = wsum[w];
      if (w < wave) wbase += x;
      all += x;
    }
    const int ex = carry + wbase + inc - v;
    if (i < a.C) {
      hist[i] = ex;
      out[i] = ex;
      if (v >= kHeavy) {
        const int pieces = (v + kHeavy - 1) / kHeavy, sl = ex / kHeavy;
        const int first = atomicAdd(&n_items, pieces);
        used[sl] = 1;
        for (int k = 0; k < pieces; ++k) {
          item[first + k][0] = ex + k * kHeavy;
          item[first + k][1] = min(kHeavy, v - k * kHeavy);
          item[first + k][2] = sl;
        }
      }
    }
    carry += all;
    __syncthreads();
  }
  if (t == 0) out[a.C] = carry;
  int32_t* ord = a.order + (int64_t)g * a.N + (int64_t)tile * kBigTile;
#pragma unroll
  for (int u = 0; u < kBigTok; ++u)
    if (c[u] >= 0) {
      const int pos = hist[c[u]] + rank[u], n = tile * kBigTile + u * 1024 + t;
      ord[pos] = n;
      ids[pos] = n;
    }
  __syncthreads();
  const int ni = n_items;
  if (ni == 0) return;
  // a piece per wave: four rows at a time (16 lanes of 16 bytes each), all of a lane's rows requested before the first is used
  const int o = lane & 15, rg = lane >> 4;
  const uint16_t* sb = a.src + (int64_t)g * a.s_sg + 8 * o;
  for (int it = wave; it < ni; it += 16) {
    const int p0 = item[it][0], m = item[it][1], sl = item[it][2];
    uint4 raw[kHeavy / 4];
#pragma unroll
    for (int u = 0; u < kHeavy / 4; ++u) {
      const int i = rg + 4 * u;
      raw[u] = make_uint4(0, 0, 0, 0);
      if (i < m) raw[u] = *(const uint4*)(sb + (int64_t)ids[p0 + i] * a.s_sn);
    }
    double acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < kHeavy / 4; ++u) add_row_bf16(acc, raw[u]);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      acc[e] += __shfl_xor(acc[e], 16);
      acc[e] += __shfl_xor(acc[e], 32);
    }
    if (lane < 16) {
#pragma unroll
      for (int e = 0; e < 8; ++e) atomicAdd(&racc[sl * kD + 8 * o + e], acc[e]);   // exact sums: the order does not matter
    }
  }
  __syncthreads();
  double* rec = a.rec + ((int64_t)g * a.nT + tile) * kSlots * kD;
  for (int i = t; i < kSlots * kD; i += 1024)
    if (used[i / kD]) rec[i] = racc[i];
}

// ------------------------------------------------------------------------- per-cluster sum + update
struct SumArgs {
  const uint16_t* src;    // [G,N,128] bf16 rows to sum (keys for the update, values for index_add)
  const int32_t* order;   // [G,N] token ids, every tile of kBigTile tokens grouped by cluster
  const int32_t* start;   // [G,nT,C+1] where a cluster's range begins inside its tile
  const double* rec;      // [G,nT,kSlots,128] sums of the ranges of kHeavy tokens or more
  uint16_t* dst;          // [G,C,128] bf16: centroids (update) or value sums (index_add)
  int32_t* cnt;           // [G,C] cluster sizes, or null
  int64_t s_sg, s_sn, d_sg, d_sc;
  int32_t N, C, nT, mode; // mode 0: plain sum cast to bf16; 1: mean; 2: mean + L2 normalise (1,2: only where cnt > 0)
  double* keep_sum;       // [G,C,128] or null: the exact sums, left for the iterations that only apply changes
  int32_t* keep_cnt;      // [G,C] or null
};

// From a cluster's exact sum (channel t of thread t < 128) and size to its stored row: sum rounded once to fp32, mean
// (kmeans.py:121), optional L2 normalisation with the squared norm summed in fp64 in a fixed tree (:122-123), bf16
// store only where the cluster has tokens (:120, 124).  Shared by the full re-sum and by the update from kept sums, so
// the two give the same bits.  All threads of the workgroup call it (it has barriers); ss_red: 128 doubles of LDS.
__device__ __forceinline__ void finish_cluster(double s, int cnt, int mode, double* ss_red, int t, uint16_t* dst_row, int32_t* cnt_out) {
  float x = 0.f;
  if (t < kD) {
    x = (float)s;                                   // exact sum rounded once to fp32
    if (mode >= 1) x = x / (float)cnt;
    ss_red[t] = (double)x * (double)x;
  }
  __syncthreads();
  if (mode == 2) {
    for (int d = kD / 2; d > 0; d >>= 1) {
      if (t < d) ss_red[t] += ss_red[t + d];
      __syncthreads();
    }
    if (t < kD) x = x / sqrtf((float)ss_red[0]);
  }
  if (t < kD && (mode == 0 || cnt > 0)) dst_row[t] = (uint16_t)f32_to_bf16_bits(x);
  if (cnt_out && t == 0) *cnt_out = cnt;
}

constexpr int kSumRows = 4;   // rows in flight per thread (8: slower, 2: the same)
constexpr int kListCap = 2048;   // token ids staged in LDS at a time

__global__ __launch_bounds__(256) void cluster_sum_kernel(SumArgs a) {
  __shared__ double red[4][kD];
  __shared__ double ss_red[kD];
  __shared__ int32_t list[kListCap];
  __shared__ int32_t wsum[4], wbig[4];
  __shared__ int32_t slot[64];
  const int c = blockIdx.x, g = blockIdx.y, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int o = t & 15, r = t >> 4;
  const int32_t* st = a.start + (int64_t)g * a.nT * (a.C + 1) + c;
  const int32_t* ord = a.order + (int64_t)g * a.N;
  const uint16_t* sb = a.src + (int64_t)g * a.s_sg + 8 * o;
  double acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  double extra = 0;   // channel t of the ranges the tiles have summed already
  int cnt = 0;
  for (int tb = 0; tb < a.nT; tb += 64) {   // 64 tiles at a time, four threads per tile
    const int tile = tb + (t >> 2), q = t & 3;
    int s0 = 0, mine = 0, big = 0;
    if (tile < a.nT) {
      s0 = st[(int64_t)tile * (a.C + 1)];
      mine = st[(int64_t)tile * (a.C + 1) + 1] - s0;
    }
    if (mine >= kHeavy) {
      big = mine;
      mine = 0;
    }
    if (q == 0) slot[t >> 2] = big ? s0 / kHeavy : -1;
    const int inc = wave_inclusive_scan(q == 0 ? mine : 0, lane);
    const int binc = wave_inclusive_scan(q == 0 ? big : 0, lane);
    if (lane == 63) {
      wsum[wave] = inc;
      wbig[wave] = binc;
    }
    __syncthreads();
    int base = __shfl(inc, lane & ~3) - mine, all = 0, all_big = 0;   // where this tile's ids go in the list
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int x = wsum[w];
      if (w < wave) base += x;
      all += x;
      all_big += wbig[w];
    }
    if (all_big > 0 && t < kD) {
      const int nt = min(64, a.nT - tb);
      for (int j = 0; j < nt; ++j)
        if (slot[j] >= 0) extra += a.rec[(((int64_t)g * a.nT + tb + j) * kSlots + slot[j]) * kD + t];
    }
    cnt += all_big;
    const int32_t* mo = ord + (int64_t)tile * kBigTile + s0;
    for (int w0 = 0; w0 < all; w0 += kListCap) {   // the ids of these tiles' tokens, kListCap at a time
      const int jb = max(0, w0 - base), je = min(mine, w0 + kListCap - base);
      for (int j = jb + q; j < je; j += 4) list[base + j - w0] = mo[j];
      __syncthreads();
      const int m = min(all - w0, kListCap);
      for (int i0 = r; i0 < m; i0 += 16 * kSumRows) {  // kSumRows rows in flight per thread
        uint4 raw[kSumRows];
#pragma unroll
        for (int u = 0; u < kSumRows; ++u) {
          const int i = i0 + 16 * u;
          raw[u] = make_uint4(0, 0, 0, 0);
          if (i < m) raw[u] = *(const uint4*)(sb + (int64_t)list[i] * a.s_sn);
        }
#pragma unroll
        for (int u = 0; u < kSumRows; ++u) add_row_bf16(acc, raw[u]);
      }
      __syncthreads();
    }
    cnt += all;
    __syncthreads();
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {   // the wave's four rows, then the four waves through LDS
    acc[e] += __shfl_xor(acc[e], 16);
    acc[e] += __shfl_xor(acc[e], 32);
  }
  if (lane < 16) {
#pragma unroll
    for (int e = 0; e < 8; ++e) red[wave][8 * o + e] = acc[e];
  }
  __syncthreads();
  double s = 0;
  if (t < kD) {
    s = extra;
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) s += red[rr][t];
    if (a.keep_sum) a.keep_sum[((int64_t)g * a.C + c) * kD + t] = s;
  }
  if (a.keep_cnt && t == 0) a.keep_cnt[(int64_t)g * a.C + c] = cnt;
  finish_cluster(s, cnt, a.mode, ss_red, t, a.dst + (int64_t)g * a.d_sg + (int64_t)c * a.d_sc, a.cnt ? a.cnt + (int64_t)g * a.C + c : nullptr);
}

// ------------------------------------------------------------------------- centroids from the carried sums
struct UpdateArgs {
  const double* sum;      // [G,C,128]
  const int32_t* cnt;     // [G,C]
  uint16_t* dst;          // centroids [G,C,128] bf16
  int32_t* cnt_out;       // [G,C]
  int64_t d_sg, d_sc;
  int32_t C, mode;
};

__global__ __launch_bounds__(kD) void kmeans_update_kernel(UpdateArgs a) {
  __shared__ double ss_red[kD];
  const int c = blockIdx.x, g = blockIdx.y, t = threadIdx.x;
  const double s = a.sum[((int64_t)g * a.C + c) * kD + t];
  const int cnt = a.cnt[(int64_t)g * a.C + c];
  finish_cluster(s, cnt, a.mode, ss_red, t, a.dst + (int64_t)g * a.d_sg + (int64_t)c * a.d_sc, a.cnt_out + (int64_t)g * a.C + c);
}

// ---------------------------------------------------------------------------------- top-k selection
struct TopkArgs {
  const uint16_t* query;   // [B,Hq,128] bf16
  const uint16_t* cent;    // [G,C,128] bf16
  const int32_t* clusters; // [G,C,M]
  const int32_t* size;     // [G,C]
  int32_t* out;            // [G,k], rows out_sg apart
  int64_t out_sg;
  float* score;            // workspace [G,C]
  int32_t* start;          // workspace [G,C] start position of each cluster in rank order (two-kernel path)
  uint32_t* arrive;        // workspace [G] arrival words of the shared score phase (one-launch path; same memory as `start`)
  int64_t q_sb, q_sh, c_sg, c_sc, cl_sg, cl_sc;
  int32_t C, M, k, Hkv, group;
};

// Cluster score = max over the kv head's q heads of <q_h, centroid>: one thread per centroid, the centroid row in
// registers (sixteen 16-byte loads), the group's queries in LDS as fp32; every dot product is one fp32 FMA chain over
// d = 0..127 in order.
__global__ __launch_bounds__(256) void topk_score_kernel(TopkArgs a) {
  __shared__ float qs[16][kD];
  const int g = blockIdx.y, b = g / a.Hkv, kvh = g % a.Hkv;
  const int nh = a.group < 16 ? a.group : 16;
  for (int i = threadIdx.x; i < nh * kD; i += blockDim.x) {
    const int h = i / kD, d = i % kD;
    qs[h][d] = bf16_bits_to_f32(a.query[(int64_t)b * a.q_sb + (int64_t)(kvh * a.group + h) * a.q_sh + d]);
  }
  __syncthreads();
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= a.C) return;
  const uint16_t* cp = a.cent + (int64_t)g * a.c_sg + (int64_t)c * a.c_sc;
  float best = -INFINITY;
  if (a.group <= 16) {
    float cf[kD];
#pragma unroll
    for (int j = 0; j < kD / 8; ++j) {
      const uint4 w = *(const uint4*)(cp + 8 * j);
      const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        cf[8 * j + 2 * e] = bf16_bits_to_f32(ww[e] & 0xffffu);
        cf[8 * j + 2 * e + 1] = bf16_bits_to_f32(ww[e] >> 16);
      }
    }
    for (int h = 0; h < nh; ++h) {
      float sacc = 0.f;
#pragma unroll
      for (int d = 0; d < kD; ++d) sacc += qs[h][d] * cf[d];
      best = fmaxf(best, sacc);
    }
  } else {   // more than 16 q heads per kv head: straight from memory
    for (int h = 0; h < a.group; ++h) {
      const uint16_t* qp = a.query + (int64_t)b * a.q_sb + (int64_t)(kvh * a.group + h) * a.q_sh;
      float sacc = 0.f;
      for (int d = 0; d < kD; ++d) sacc += bf16_bits_to_f32(qp[d]) * bf16_bits_to_f32(cp[d]);
      best = fmaxf(best, sacc);
    }
  }
  a.score[(int64_t)g * a.C + c] = best;
}

// Order the clusters by (score descending, index ascending), prefix-sum their sizes in that order and emit the first k
// token ids: one workgroup per group, everything in LDS.  The order comes from a bitonic sort of 64-bit keys
// (score mapped to an unsigned integer of the same order in the high word, ~index in the low word; a counting rank
// with C compares per cluster took 50 us at C = 1024).  Each output position finds its cluster by a binary search
// over the prefix; positions past the total number of tokens get -1.
__global__ __launch_bounds__(1024) void topk_emit_kernel(TopkArgs a) {
  extern __shared__ int32_t sh[];          // [P] 64-bit keys (P = C rounded up to a power of two), then [C + 1] prefix
  int P = 1;
  while (P < a.C) P <<= 1;
  unsigned long long* key = (unsigned long long*)sh;
  int32_t* pre = sh + 2 * P;
  __shared__ int32_t part[1024];
  const int g = blockIdx.x, t = threadIdx.x;
  const int32_t* size = a.size + (int64_t)g * a.C;
  for (int c = t; c < P; c += blockDim.x) {
    unsigned long long kk = 0;             // padding sorts behind every cluster
    if (c < a.C) {
      const uint32_t bits = __float_as_uint(a.score[(int64_t)g * a.C + c] + 0.0f);    // -0.0 counts as +0.0
      const uint32_t ord = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
      kk = ((unsigned long long)ord << 32) | (0xffffffffu - (uint32_t)c);
    }
    key[c] = kk;
  }
  __syncthreads();
  for (int len = 2; len <= P; len <<= 1)
    for (int d = len >> 1; d > 0; d >>= 1) {
      for (int i = t; i < P / 2; i += blockDim.x) {
        const int lo = ((i & ~(d - 1)) << 1) | (i & (d - 1)), hi = lo | d;
        const bool descending = (lo & len) == 0;
        const unsigned long long x = key[lo], y = key[hi];
        if ((x < y) == descending) {
          key[lo] = y;
          key[hi] = x;
        }
      }
      __syncthreads();
    }
  auto by_rank = [&](int r) { return (int)(0xffffffffu - (uint32_t)key[r]); };
  // exclusive prefix of the (clamped) sizes in rank order: per-thread runs of `per` ranks, a scan over the 1024 run sums
  const int per = (a.C + 1023) / 1024;
  int run = 0;
  for (int i = 0; i < per; ++i) {
    const int r = t * per + i;
    if (r < a.C) run += min(size[by_rank(r)], a.M);
  }
  part[t] = run;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {   // Hillis-Steele inclusive scan
    const int v = (t >= d) ? part[t - d] : 0;
    __syncthreads();
    part[t] += v;
    __syncthreads();
  }
  int acc = part[t] - run;
  for (int i = 0; i < per; ++i) {
    const int r = t * per + i;
    if (r < a.C) {
      pre[r] = acc;
      acc += min(size[by_rank(r)], a.M);
    }
  }
  if (t == 1023) pre[a.C] = part[1023];
  __syncthreads();
  const int total = pre[a.C];
  int32_t* out = a.out + (int64_t)g * a.out_sg;
  for (int p = t; p < a.k; p += blockDim.x) {
    int32_t id = -1;
    if (p < total) {
      int lo = 0, hi = a.C;               // the rank r with pre[r] <= p < pre[r + 1]
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (pre[mid] <= p) lo = mid;
        else hi = mid;
      }
      id = a.clusters[(int64_t)g * a.cl_sg + (int64_t)by_rank(lo) * a.cl_sc + (p - pre[lo])];
    }
    out[p] = id;
  }
}


// ---- the same selection in one launch, without ordering all clusters (at most 1024 clusters and 16 q heads per kv head;
// other shapes take the two kernels above).  One workgroup of 1024 threads per group, one cluster per thread:
//   1. scores of all clusters on the matrix cores (fp32 accumulation of exact bf16 products), maximum over the q heads;
//   2. the clusters that can take part are found by a radix select on the top 16 bits of the order-preserving score key,
//      weighted by cluster size: two rounds of a 256-bin histogram in LDS (sum of sizes per bin), each read from the top
//      bin down by one wave until k tokens are covered.  Every cluster whose 16-bit key is at or above the pivot is a
//      candidate: all clusters above the pivot together hold fewer than k tokens, those at the pivot complete them;
//   3. only the candidates (a few dozen of 1024 for k = 4096) are ordered by (score descending, index ascending): a
//      counting rank while there are at most 256 of them, the bitonic network otherwise;
//   4. prefix of the sizes in rank order by one wave, then every output position finds its cluster by binary search.
constexpr int kSelCount = 256;   // candidates ranked by counting; more go through the bitonic network

// executed by the 64 lanes of one wave: the highest bin d with (weight of bins above d) < need <= (that + weight of bin d)
__device__ __forceinline__ void find_pivot(const int32_t* hw, int need, int lane, int& digit, int& above) {
  int w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = hw[4 * lane + i];
  const int s = w[0] + w[1] + w[2] + w[3];
  int suf = s;                                   // weight of this lane's bins and of all higher lanes'
  for (int d = 1; d < 64; d <<= 1) {
    const int v = __shfl_down(suf, d);
    if (lane + d < 64) suf += v;
  }
  const unsigned long long m = __ballot(suf >= need);
  int dg = -1, ab = 0;
  if (m != 0) {
    const int lp = 63 - __builtin_clzll(m);      // suf falls with the lane index: the highest lane that still reaches `need`
    if (lane == lp) {
      int cum = suf - s;
      dg = 4 * lane;
      ab = cum + w[3] + w[2] + w[1];
#pragma unroll
      for (int i = 3; i >= 1; --i) {
        if (cum + w[i] >= need) {
          dg = 4 * lane + i;
          ab = cum;
          break;
        }
        cum += w[i];
      }
    }
    dg = __shfl(dg, lp);
    ab = __shfl(ab, lp);
  }
  digit = dg;    // -1: all bins together hold fewer than `need`
  above = ab;
}

// The score phase pulls a head's whole centroid matrix (256 KB at 1024 clusters) through the one CU its workgroup runs
// on, which is most of that phase's time.  With kTopkParts workgroups per (sequence, kv head), each scores its share
// of the clusters into the workspace, and the one that arrives last carries on alone with steps 2 - 4.  Nobody waits
// for anybody.
//
// The arrival counter of a head is a word in the caller's workspace, so calls that use different workspaces never meet.
// It needs no initialisation and no reset: the word counts as "k workgroups have arrived" only while it reads
// kArriveTag | k with 0 < k < parts; anything else -- whatever the memory held before, or the kArriveTag | parts a
// finished call leaves behind -- counts as zero.  (Only a call that was cut short between two arrivals could leave a
// live count behind; a launch that dies half-way takes the process's GPU context with it.)
//
// Ordering of the hand-over, step by step:
//   1. every wave that stored scores waits for its own stores to be acknowledged (s_waitcnt vmcnt(0)): they are then
//      in this XCD's L2, not somewhere between the wave and the L2;
//   2. the workgroup barrier puts all of that before thread 0's next instruction;
//   3. thread 0's device-scope fence writes the L2's dirty lines back, which covers every wave's scores of step 1,
//      and orders them before its atomic on the counter (the atomic executes at device scope);
//   4. the workgroup that reads parts - 1 earlier arrivals has thread 0 execute a device-scope fence after the atomic
//      (acquire: stale lines of other XCDs' data leave its L2), then the barrier, and only then the scores are read,
//      with device-scope loads that go past the CU's vector cache.
constexpr int kTopkParts = 4;   // divides 16: every part gets whole waves of 64 clusters
constexpr uint32_t kArriveTag = 0x5A70CB00u;   // low byte: number of arrivals so far

__global__ __launch_bounds__(1024) void topk_select_kernel(TopkArgs a) {
  __shared__ float sc[1024];
  __shared__ unsigned long long ckey[1024];
  __shared__ int32_t pre[1025], rank_cluster[1024], rank_size[1024], hw[256], misc[8];
  const int g = blockIdx.x, t = threadIdx.x, lane = t & 63;
  const int parts = gridDim.y, part = blockIdx.y;
  const int b = g / a.Hkv, kvh = g % a.Hkv;
  const int nh = a.group;
  if (t < 256) hw[t] = 0;
  if (t == 0) misc[0] = 0;
  const bool have = t < a.C;
  const int sz = have ? min(a.size[(int64_t)g * a.C + t], a.M) : 0;   // requested ahead of the score phase
  // ---- 1. scores on the matrix cores: wave w takes clusters 64 w .. 64 w + 63 in four blocks of 16; per block
  // S[cluster, head] = centroids . queries^T on v_mfma_f32_16x16x32_bf16 (the group's q heads padded to 16 columns).
  // Lane (r = lane % 16, q = lane / 16) feeds centroid row r, columns 32 kk + 8 q .. + 7 as the A operand and the same
  // columns of query head r as the B operand, and receives S[cluster 4 q + i][head r], i < 4.
  const int waves_per_part = 16 / parts;
  if ((t >> 6) < waves_per_part) {
    const int wave = part * waves_per_part + (t >> 6), r = lane & 15, q4 = lane >> 4;
    typedef __attribute__((ext_vector_type(4))) float f32x4;
    uint4 qf[4];
    const uint16_t* qp = a.query + (int64_t)b * a.q_sb + (int64_t)(kvh * a.group + min(r, nh - 1)) * a.q_sh + 8 * q4;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) qf[kk] = (r < nh) ? *(const uint4*)(qp + 32 * kk) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) {
      const int c0 = 64 * wave + 16 * blk;
      const int row = min(c0 + r, a.C - 1);
      const uint16_t* cp = a.cent + (int64_t)g * a.c_sg + (int64_t)row * a.c_sc + 8 * q4;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const uint4 cf = *(const uint4*)(cp + 32 * kk);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, cf), __builtin_bit_cast(bf16x8_t, qf[kk]), acc, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = (r < nh) ? acc[i] : -INFINITY;   // the padded columns take no part in the maximum over the q heads
        // maximum over the 16 lanes of a row by rotations within the row (DPP row_ror 1, 2, 4, 8): no LDS traffic
        v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false)));
        v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false)));
        v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false)));
        v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false)));
        if (r == 0) {
          if (parts == 1) sc[c0 + 4 * q4 + i] = v;
          else if (c0 + 4 * q4 + i < a.C) a.score[(int64_t)g * a.C + c0 + 4 * q4 + i] = v;
        }
      }
    }
  }
  if (parts > 1) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // step 1: this wave's score stores have reached the L2
    __syncthreads();                                    // step 2
    if (t == 0) {
      __threadfence();                                  // step 3
      uint32_t* ctr = a.arrive + g;
      uint32_t old = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), before;
      do {
        before = ((old & ~0xffu) == kArriveTag && (old & 0xffu) < (uint32_t)parts) ? (old & 0xffu) : 0u;
      } while (!__hip_atomic_compare_exchange_strong(ctr, &old, kArriveTag | (before + 1u), __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT));
      if ((int)before == parts - 1) __threadfence();    // step 4
      misc[4] = (int)before;
    }
    __syncthreads();
    if (misc[4] != parts - 1) return;    // uniform: somebody else finishes the job
    if (have) sc[t] = __hip_atomic_load(&a.score[(int64_t)g * a.C + t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  uint32_t key32 = 0;
  if (have) {
    const uint32_t bits = __float_as_uint(sc[t] + 0.0f);    // -0.0 counts as +0.0
    key32 = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
  }
  // ---- 2. radix select over the top 16 key bits, weighted by size
  if (sz > 0) atomicAdd(&hw[key32 >> 24], sz);
  __syncthreads();
  if (t < 64) {
    int d1, ab1;
    find_pivot(hw, a.k, lane, d1, ab1);
    if (t == 0) {
      misc[1] = d1;
      misc[2] = ab1;
    }
  }
  __syncthreads();
  const int d1 = misc[1], above1 = misc[2];
  if (t < 256) hw[t] = 0;
  __syncthreads();
  if (sz > 0 && d1 >= 0 && (int)(key32 >> 24) == d1) atomicAdd(&hw[(key32 >> 16) & 255], sz);
  __syncthreads();
  if (t < 64 && d1 >= 0) {
    int d2, ab2;
    find_pivot(hw, a.k - above1, lane, d2, ab2);   // bin d1 holds at least k - above1 tokens, so d2 >= 0
    if (t == 0) misc[3] = d2;
  }
  __syncthreads();
  const uint32_t pivot16 = d1 >= 0 ? (((uint32_t)d1 << 8) | (uint32_t)misc[3]) : 0u;   // fewer than k tokens in all: everything
  // ---- 3. candidates and their order
  if (sz > 0 && (key32 >> 16) >= pivot16) {
    const int pos = atomicAdd(&misc[0], 1);
    ckey[pos] = ((unsigned long long)key32 << 32) | (0xffffffffu - (uint32_t)t);
    rank_size[pos] = sz;    // by candidate slot for now
  }
  __syncthreads();
  const int m = misc[0];
  int my_rank = -1, my_cluster = 0, my_size = 0;
  if (m <= kSelCount) {
    if (t < m) {
      const unsigned long long mine = ckey[t];
      int r = 0;
      for (int j = 0; j < m; ++j) r += ckey[j] > mine;
      my_rank = r;
      my_cluster = (int)(0xffffffffu - (uint32_t)mine);
      my_size = rank_size[t];
    }
    __syncthreads();
    if (my_rank >= 0) {
      rank_cluster[my_rank] = my_cluster;
      rank_size[my_rank] = my_size;
    }
  } else {
    int P = 1;
    while (P < m) P <<= 1;
    if (t >= m && t < P) ckey[t] = 0;            // padding sorts behind every candidate
    __syncthreads();
    for (int len = 2; len <= P; len <<= 1)
      for (int d = len >> 1; d > 0; d >>= 1) {
        if (t < P / 2) {
          const int lo = ((t & ~(d - 1)) << 1) | (t & (d - 1)), hi = lo | d;
          const bool descending = (lo & len) == 0;
          const unsigned long long x = ckey[lo], y = ckey[hi];
          if ((x < y) == descending) {
            ckey[lo] = y;
            ckey[hi] = x;
          }
        }
        __syncthreads();
      }
    if (t < m) {
      const int c = (int)(0xffffffffu - (uint32_t)ckey[t]);
      rank_cluster[t] = c;
      rank_size[t] = min(a.size[(int64_t)g * a.C + c], a.M);
    }
  }
  __syncthreads();
  // ---- 4. exclusive prefix of the sizes in rank order (one wave), then the token ids
  if (t < 64) {
    const int per = (m + 63) / 64;
    int run = 0;
    for (int i = 0; i < per; ++i) {
      const int r = lane * per + i;
      if (r < m) run += rank_size[r];
    }
    int inc = run;
    for (int d = 1; d < 64; d <<= 1) {
      const int v = __shfl_up(inc, d);
      if (lane >= d) inc += v;
    }
    int acc = inc - run;
    for (int i = 0; i < per; ++i) {
      const int r = lane * per + i;
      if (r < m) {
        pre[r] = acc;
        acc += rank_size[r];
      }
    }
    if (lane == 63) pre[m] = inc;
  }
  __syncthreads();
  const int total = pre[m];
  int32_t* out = a.out + (int64_t)g * a.out_sg;
  constexpr int U = 4;   // positions per thread and round: their table reads are independent and overlap
  for (int p0 = t; p0 < a.k; p0 += U * 1024) {
    int64_t off[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = p0 + u * 1024;
      off[u] = -1;
      if (p < a.k && p < total) {
        int lo = 0, hi = m;               // the rank r with pre[r] <= p < pre[r + 1]
        while (hi - lo > 1) {
          const int mid = (lo + hi) >> 1;
          if (pre[mid] <= p) lo = mid;
          else hi = mid;
        }
        off[u] = (int64_t)g * a.cl_sg + (int64_t)rank_cluster[lo] * a.cl_sc + (p - pre[lo]);
      }
    }
    int32_t id[U];
#pragma unroll
    for (int u = 0; u < U; ++u) id[u] = off[u] >= 0 ? a.clusters[off[u]] : -1;
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (p0 + u * 1024 < a.k) out[p0 + u * 1024] = id[u];
  }
}

struct WsLayout {
  size_t off_bytes, hist_bytes, order_bytes, score_bytes, start_bytes, total_bytes, rec_bytes;
  size_t sum_bytes, cnt_bytes;   // the sums and sizes carried from step to step (sq_kmeans_train_stateful)
  int nT, C;
  size_t rec_offset() const { return off_bytes + hist_bytes + order_bytes + score_bytes + start_bytes + total_bytes; }
  size_t sum_offset() const { return rec_offset() + rec_bytes; }
  size_t cnt_offset() const { return sum_offset() + sum_bytes; }
  size_t all() const { return cnt_offset() + cnt_bytes; }
};

WsLayout ws_layout(int64_t G, int64_t N, int64_t C) {
  WsLayout w;
  auto up = [](size_t x) { return (x + 255) / 256 * 256; };
  w.nT = (int)((N + kTileTok - 1) / kTileTok);
  w.C = (int)C;
  w.off_bytes = up((size_t)G * (C + 1) * 4);
  w.hist_bytes = up((size_t)G * w.nT * (C + 1) * 4);   // per-tile histograms of the ordered sort, or range starts of the grouping
  w.order_bytes = up((size_t)G * N * 4);
  w.score_bytes = up((size_t)G * C * 4);
  w.start_bytes = up((size_t)G * C * 4);
  w.total_bytes = up((size_t)G * C * 4);
  w.rec_bytes = up((size_t)G * ((N + kBigTile - 1) / kBigTile) * kSlots * kD * 8);
  w.sum_bytes = up((size_t)G * C * kD * 8);
  w.cnt_bytes = up((size_t)G * C * 4);
  return w;
}

int check_ws(const DLTensor* ws, size_t need, int dev, const char* who) {
  SQ_REQUIRE(ws && on_gpu(ws) && ws->device.device_id == dev, SQ_EWORKSPACE, "%s: workspace missing or not on the device", who);
  SQ_REQUIRE((size_t)numel_of(ws) * (ws->dtype.bits / 8) >= need && is_compact(ws), SQ_EWORKSPACE,
             "%s: workspace too small: need %zu bytes", who, need);
  SQ_REQUIRE(((uintptr_t)data_of(ws) & 255) == 0, SQ_EWORKSPACE, "%s: workspace not 256-byte aligned", who);
  return SQ_OK;
}

int check_current_device(int dev, const char* who) {
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "%s: tensors live on device %d but the current device is %d", who, dev, cur);
  return SQ_OK;
}

// tokens of every cluster in ascending order into clusters[G,C,M] (reverse index), sizes into total_out
int run_sort(const DLTensor* idx, char* wsp, const WsLayout& w, int32_t* dst, int64_t dst_sg, int64_t dst_sc, int M,
             int32_t* total_out, int C, hipStream_t st) {
  const int64_t G = idx->shape[0], N = idx->shape[1];
  SortArgs s;
  s.idx = (const int32_t*)data_of(idx);
  s.tile_hist = (int32_t*)(wsp + w.off_bytes);
  s.total = total_out;
  s.dst = dst;
  s.i_sg = stride_of(idx, 0);
  s.dst_sg = dst_sg;
  s.dst_sc = dst_sc;
  s.N = (int)N;
  s.C = C;
  s.nT = w.nT;
  s.M = M;
  hipLaunchKernelGGL(sort_hist_kernel, dim3(w.nT, (unsigned)G), dim3(kTileTok), (size_t)C * 4, st, s);
  hipLaunchKernelGGL(sort_scan_tiles_kernel, dim3((C + 31) / 32, (unsigned)G), dim3(32 * kScanSegs), 0, st, s);
  hipLaunchKernelGGL(sort_scatter_kernel, dim3(w.nT, (unsigned)G), dim3(kTileTok), 0, st, s);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}

// every tile of kBigTile tokens grouped by cluster into `order`, the ranges' starts into the histogram region
int run_group(const DLTensor* idx, const DLTensor* src, char* wsp, const WsLayout& w, hipStream_t st) {
  const int64_t G = idx->shape[0], N = idx->shape[1];
  GroupArgs s;
  s.idx = (const int32_t*)data_of(idx);
  s.src = (const uint16_t*)data_of(src);
  s.start = (int32_t*)(wsp + w.off_bytes);
  s.order = (int32_t*)(wsp + w.off_bytes + w.hist_bytes);
  s.rec = (double*)(wsp + w.rec_offset());
  s.i_sg = stride_of(idx, 0);
  s.s_sg = stride_of(src, 0);
  s.s_sn = stride_of(src, 1);
  s.N = (int)N;
  s.C = w.C;
  s.nT = (int)((N + kBigTile - 1) / kBigTile);
  const size_t lds = (size_t)kSlots * kD * 8 + ((size_t)w.C + kBigTile) * 4;
  static bool raised[64] = {};
  int dev = 0;
  SQ_HIP(hipGetDevice(&dev));
  if (dev >= 0 && dev < 64 && !raised[dev]) {   // up to 72 KB for 8192 clusters, above the default limit
    SQ_HIP(hipFuncSetAttribute((const void*)tile_group_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)((size_t)kSlots * kD * 8 + ((size_t)kMaxC + kBigTile) * 4)));
    raised[dev] = true;
  }
  hipLaunchKernelGGL(tile_group_kernel, dim3(s.nT, (unsigned)G), dim3(1024), lds, st, s);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}

// sums of `src` rows per cluster after run_group
int run_cluster_sum(const DLTensor* src, char* wsp, const WsLayout& w, DLTensor* dst, int32_t* cnt, int mode, hipStream_t st, bool keep = false) {
  const int64_t G = src->shape[0], N = src->shape[1];
  SumArgs s;
  s.src = (const uint16_t*)data_of(src);
  s.start = (const int32_t*)(wsp + w.off_bytes);
  s.order = (const int32_t*)(wsp + w.off_bytes + w.hist_bytes);
  s.rec = (const double*)(wsp + w.rec_offset());
  s.dst = (uint16_t*)data_of(dst);
  s.cnt = cnt;
  s.s_sg = stride_of(src, 0);
  s.s_sn = stride_of(src, 1);
  s.d_sg = stride_of(dst, 0);
  s.d_sc = stride_of(dst, 1);
  s.N = (int)N;
  s.C = w.C;
  s.nT = (int)((N + kBigTile - 1) / kBigTile);
  s.mode = mode;
  s.keep_sum = keep ? (double*)(wsp + w.sum_offset()) : nullptr;
  s.keep_cnt = keep ? (int32_t*)(wsp + w.cnt_offset()) : nullptr;
  hipLaunchKernelGGL(cluster_sum_kernel, dim3((unsigned)w.C, (unsigned)G), dim3(256), 0, st, s);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}

int check_gnd(const DLTensor* t, const char* name, int dev) {
  int rc = check_tensor(t, name, 3, dev);
  if (rc) return rc;
  SQ_REQUIRE(dtype_of(t) == DType::BF16, SQ_EDTYPE, "%s must be bf16", name);
  SQ_REQUIRE(t->shape[2] == kD, SQ_EUNSUPPORTED, "%s: last dimension must be 128, got %lld", name, (long long)t->shape[2]);
  SQ_REQUIRE(stride_of(t, 0) % 8 == 0 && stride_of(t, 1) % 8 == 0, SQ_ESHAPE, "%s: strides must be multiples of 8 elements", name);
  return SQ_OK;
}

int check_i32(const DLTensor* t, const char* name, int ndim, int dev) {
  SQ_REQUIRE(t != nullptr, SQ_EINVAL, "%s is null", name);
  SQ_REQUIRE(on_gpu(t) && t->device.device_id == dev, SQ_EDEVICE, "%s is not on the same ROCm device", name);
  SQ_REQUIRE(dtype_of(t) == DType::I32 && t->ndim == ndim && is_compact(t), SQ_ESHAPE, "%s must be a compact int32 tensor of rank %d", name, ndim);
  return SQ_OK;
}

}  // namespace
}  // namespace sq

using namespace sq;

extern "C" size_t sq_kmeans_workspace_bytes(int64_t groups, int64_t num_tokens, int64_t num_centroids, int64_t dim) {
  (void)dim;
  if (groups <= 0 || num_tokens <= 0 || num_centroids <= 0) return 0;
  return ws_layout(groups, num_tokens, num_centroids).all();
}

namespace {
int kmeans_train_impl(const DLTensor* data, DLTensor* centroids, DLTensor* idx, DLTensor* cnt, DLTensor* workspace,
                      int32_t normalize, int32_t state, void* stream, const char* who) {
  SQ_REQUIRE(data && centroids && idx && cnt, SQ_EINVAL, "%s: data, centroids, idx and cnt must be non-null", who);
  SQ_REQUIRE(state >= SQ_KMEANS_STATELESS && state <= SQ_KMEANS_APPLY_CHANGES, SQ_EINVAL, "%s: state %d not supported", who, (int)state);
  const int dev = data->device.device_id;
  int rc;
  if ((rc = check_gnd(data, "data", dev)) || (rc = check_gnd(centroids, "centroids", dev)) || (rc = check_i32(idx, "idx", 2, dev)) ||
      (rc = check_i32(cnt, "cnt", 2, dev)))
    return rc;
  const int64_t G = data->shape[0], N = data->shape[1], C = centroids->shape[1];
  SQ_REQUIRE(G > 0 && N > 0 && C > 0, SQ_ESHAPE, "%s: empty tensor", who);
  SQ_REQUIRE(centroids->shape[0] == G && idx->shape[0] == G && idx->shape[1] == N && cnt->shape[0] == G && cnt->shape[1] == C,
             SQ_ESHAPE, "%s: shapes of data/centroids/idx/cnt disagree", who);
  SQ_REQUIRE(C % 32 == 0, SQ_ESHAPE, "num_centroids %% 32 != 0 (num_centroids = %lld)", (long long)C);
  SQ_REQUIRE(C <= kMaxC, SQ_EUNSUPPORTED, "%s: more than %d centroids", who, kMaxC);
  SQ_REQUIRE(N < (1ll << 31) - 65536, SQ_EUNSUPPORTED, "%s: too many tokens", who);
  const WsLayout w = ws_layout(G, N, C);
  if ((rc = check_ws(workspace, w.all(), dev, who)) || (rc = check_current_device(dev, who))) return rc;
  hipStream_t st = (hipStream_t)stream;
  char* wsp = data_of(workspace);

  AssignArgs a;
  a.data = (const uint16_t*)data_of(data);
  a.cent = (const uint16_t*)data_of(centroids);
  a.idx = (int32_t*)data_of(idx);
  a.d_sg = stride_of(data, 0);
  a.d_sn = stride_of(data, 1);
  a.c_sg = stride_of(centroids, 0);
  a.c_sc = stride_of(centroids, 1);
  a.i_sg = stride_of(idx, 0);
  a.N = (int)N;
  a.C = (int)C;
  a.keep_sum = (double*)(wsp + w.sum_offset());
  a.keep_cnt = (int32_t*)(wsp + w.cnt_offset());
  const dim3 agrid((unsigned)((N + kTileTok - 1) / kTileTok), (unsigned)G);
  const int mode = normalize ? 2 : 1;
  if (state == SQ_KMEANS_APPLY_CHANGES) {
    hipLaunchKernelGGL(kmeans_assign_kernel<true>, agrid, dim3(kAssignWaves * 64), 0, st, a);
    UpdateArgs u;
    u.sum = a.keep_sum;
    u.cnt = a.keep_cnt;
    u.dst = (uint16_t*)data_of(centroids);
    u.cnt_out = (int32_t*)data_of(cnt);
    u.d_sg = stride_of(centroids, 0);
    u.d_sc = stride_of(centroids, 1);
    u.C = (int)C;
    u.mode = mode;
    hipLaunchKernelGGL(kmeans_update_kernel, dim3((unsigned)C, (unsigned)G), dim3(kD), 0, st, u);
    SQ_HIP(hipGetLastError());
    return SQ_OK;
  }
  hipLaunchKernelGGL(kmeans_assign_kernel<false>, agrid, dim3(kAssignWaves * 64), 0, st, a);
  SQ_HIP(hipGetLastError());
  if ((rc = run_group(idx, data, wsp, w, st))) return rc;
  return run_cluster_sum(data, wsp, w, centroids, (int32_t*)data_of(cnt), mode, st, state == SQ_KMEANS_KEEP_SUMS);   // cnt = cluster sizes
}
}  // namespace

extern "C" int sq_kmeans_train(const DLTensor* data, DLTensor* centroids, DLTensor* idx, DLTensor* cnt, DLTensor* workspace,
                               int32_t normalize, void* stream) {
  return kmeans_train_impl(data, centroids, idx, cnt, workspace, normalize, SQ_KMEANS_STATELESS, stream, "sq_kmeans_train");
}

extern "C" int sq_kmeans_train_stateful(const DLTensor* data, DLTensor* centroids, DLTensor* idx, DLTensor* cnt, DLTensor* workspace,
                                        int32_t normalize, int32_t state, void* stream) {
  return kmeans_train_impl(data, centroids, idx, cnt, workspace, normalize, state, stream, "sq_kmeans_train_stateful");
}

extern "C" int sq_reverse_index(const DLTensor* idx, DLTensor* clusters, DLTensor* cluster_size, DLTensor* workspace, void* stream) {
  SQ_REQUIRE(idx && clusters && cluster_size, SQ_EINVAL, "sq_reverse_index: idx, clusters and cluster_size must be non-null");
  const int dev = idx->device.device_id;
  int rc;
  if ((rc = check_i32(idx, "idx", 2, dev)) || (rc = check_i32(clusters, "clusters", 3, dev)) ||
      (rc = check_i32(cluster_size, "cluster_size", 2, dev)))
    return rc;
  const int64_t G = idx->shape[0], N = idx->shape[1], C = clusters->shape[1], M = clusters->shape[2];
  SQ_REQUIRE(G > 0 && N > 0 && C > 0 && M > 0, SQ_ESHAPE, "sq_reverse_index: empty tensor");
  SQ_REQUIRE(clusters->shape[0] == G && cluster_size->shape[0] == G && cluster_size->shape[1] == C, SQ_ESHAPE,
             "sq_reverse_index: shapes of idx/clusters/cluster_size disagree");
  SQ_REQUIRE(C <= kMaxC, SQ_EUNSUPPORTED, "sq_reverse_index: more than %d centroids", kMaxC);
  const WsLayout w = ws_layout(G, N, C);
  if ((rc = check_ws(workspace, w.all(), dev, "sq_reverse_index")) || (rc = check_current_device(dev, "sq_reverse_index"))) return rc;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(fill_i32_kernel, dim3(256), dim3(256), 0, st, (int32_t*)data_of(clusters), G * C * M, 0);
  return run_sort(idx, data_of(workspace), w, (int32_t*)data_of(clusters), C * M, M, (int)M,
                  (int32_t*)data_of(cluster_size), (int)C, st);
}

extern "C" int sq_index_add(const DLTensor* value, const DLTensor* idx, DLTensor* out, DLTensor* workspace, void* stream) {
  SQ_REQUIRE(value && idx && out, SQ_EINVAL, "sq_index_add: value, idx and out must be non-null");
  const int dev = value->device.device_id;
  int rc;
  if ((rc = check_gnd(value, "value", dev)) || (rc = check_gnd(out, "out", dev)) || (rc = check_i32(idx, "idx", 2, dev))) return rc;
  const int64_t G = value->shape[0], N = value->shape[1], C = out->shape[1];
  SQ_REQUIRE(G > 0 && N > 0 && C > 0, SQ_ESHAPE, "sq_index_add: empty tensor");
  SQ_REQUIRE(out->shape[0] == G && idx->shape[0] == G && idx->shape[1] == N, SQ_ESHAPE, "sq_index_add: shapes disagree");
  SQ_REQUIRE(C <= kMaxC, SQ_EUNSUPPORTED, "sq_index_add: more than %d centroids", kMaxC);
  const WsLayout w = ws_layout(G, N, C);
  if ((rc = check_ws(workspace, w.all(), dev, "sq_index_add")) || (rc = check_current_device(dev, "sq_index_add"))) return rc;
  hipStream_t st = (hipStream_t)stream;
  char* wsp = data_of(workspace);
  if ((rc = run_group(idx, value, wsp, w, st))) return rc;
  return run_cluster_sum(value, wsp, w, out, nullptr, 0, st);
}

extern "C" int sq_topk_select(const DLTensor* query, const DLTensor* centroids, const DLTensor* clusters,
                              const DLTensor* cluster_size, DLTensor* out, DLTensor* workspace, int32_t num_kv_groups,
                              void* stream) {
  SQ_REQUIRE(query && centroids && clusters && cluster_size && out, SQ_EINVAL, "sq_topk_select: null tensor argument");
  const int dev = query->device.device_id;
  int rc;
  if ((rc = check_gnd(query, "query", dev)) || (rc = check_gnd(centroids, "centroids", dev)) ||
      (rc = check_i32(clusters, "clusters", 3, dev)) || (rc = check_i32(cluster_size, "cluster_size", 2, dev)))
    return rc;
  // out may be the leading columns of a wider int32 matrix (a decode list that continues with other tokens)
  SQ_REQUIRE(on_gpu(out) && out->device.device_id == dev, SQ_EDEVICE, "out is not on the same ROCm device");
  SQ_REQUIRE(dtype_of(out) == DType::I32 && out->ndim == 2 && stride_of(out, 1) == 1 && stride_of(out, 0) >= out->shape[1], SQ_ESHAPE,
             "out must be int32 [G, k] with contiguous rows");
  const int64_t B = query->shape[0], Hq = query->shape[1], G = centroids->shape[0], C = centroids->shape[1];
  const int64_t M = clusters->shape[2], k = out->shape[1];
  SQ_REQUIRE(num_kv_groups > 0 && Hq % num_kv_groups == 0, SQ_EINVAL, "sq_topk_select: num_kv_groups %d does not divide Hq", num_kv_groups);
  const int64_t Hkv = Hq / num_kv_groups;
  SQ_REQUIRE(G == B * Hkv, SQ_ESHAPE, "sq_topk_select: centroids has %lld groups, expected B*Hkv = %lld", (long long)G, (long long)(B * Hkv));
  SQ_REQUIRE(clusters->shape[0] == G && clusters->shape[1] == C && cluster_size->shape[0] == G && cluster_size->shape[1] == C &&
                 out->shape[0] == G && k > 0 && M > 0,
             SQ_ESHAPE, "sq_topk_select: shapes disagree");
  SQ_REQUIRE(C <= kMaxC, SQ_EUNSUPPORTED, "sq_topk_select: more than %d centroids", kMaxC);
  const WsLayout w = ws_layout(G, 1, C);
  if ((rc = check_ws(workspace, w.all(), dev, "sq_topk_select")) || (rc = check_current_device(dev, "sq_topk_select"))) return rc;
  hipStream_t st = (hipStream_t)stream;
  char* wsp = data_of(workspace);
  TopkArgs a;
  a.query = (const uint16_t*)data_of(query);
  a.cent = (const uint16_t*)data_of(centroids);
  a.clusters = (const int32_t*)data_of(clusters);
  a.size = (const int32_t*)data_of(cluster_size);
  a.out = (int32_t*)data_of(out);
  a.out_sg = stride_of(out, 0);
  a.score = (float*)(wsp + w.off_bytes + w.hist_bytes + w.order_bytes);
  a.start = (int32_t*)(wsp + w.off_bytes + w.hist_bytes + w.order_bytes + w.score_bytes);
  a.arrive = (uint32_t*)a.start;   // the one-launch path does not use `start`
  a.q_sb = stride_of(query, 0);
  a.q_sh = stride_of(query, 1);
  a.c_sg = stride_of(centroids, 0);
  a.c_sc = stride_of(centroids, 1);
  a.cl_sg = C * M;
  a.cl_sc = M;
  a.C = (int)C;
  a.M = (int)M;
  a.k = (int)k;
  a.Hkv = (int)Hkv;
  a.group = num_kv_groups;
  if (C <= 1024 && num_kv_groups <= 16) {   // one launch, only the clusters that can fill k are ordered
    const unsigned parts = (C >= 64 * 16) ? kTopkParts : 1;   // fewer clusters: not worth sharing
    hipLaunchKernelGGL(topk_select_kernel, dim3((unsigned)G, parts), dim3(1024), 0, st, a);
    SQ_HIP(hipGetLastError());
    return SQ_OK;
  }
  hipLaunchKernelGGL(topk_score_kernel, dim3((unsigned)((C + 255) / 256), (unsigned)G), dim3(256), 0, st, a);
  int P = 1;
  while (P < C) P <<= 1;
  const size_t emit_lds = (size_t)(2 * P + C + 1) * 4;
  if (emit_lds > 48 * 1024)   // beyond the default limit of dynamic LDS (C > 4096)
    SQ_HIP(hipFuncSetAttribute((const void*)topk_emit_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)emit_lds));
  hipLaunchKernelGGL(topk_emit_kernel, dim3((unsigned)G), dim3(1024), emit_lds, st, a);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}
