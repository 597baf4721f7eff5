// Decode-step ("token") attention over a paged KV pool for gfx950.
//
//   q [batch, heads, d]            one query token per sequence
//   k, v [slots, kv_heads, d]      the pool; a token's heads are adjacent (d contiguous)
//   b_loc [batch, >= max_len]      slot table, right-aligned: sequence b's t-th token is at
//                                  column max_len - seq_len[b] + t
//   b_start_loc, b_seq_len [batch]
//
// out[b,h,:] = softmax_t(q[b,h,:] . k[slot_t,h,:] / sqrt(d)) . v[slot_t,h,:]
// (dicp/dicp/vendor/AscendGraph/ext_ops.py:100-133, slots gathered through b_loc).
//
// The fused kernel is HBM-bound: every K and V row of the sequence is read exactly once
// (d * itemsize bytes each), nothing else of size is touched. Mapping:
//   * a head row of d elements is covered by LPT = d*itemsize/16 lanes with one 16-byte
//     load each, so one wave-wide load fetches 64/LPT head rows: consecutive heads of one token
//     (one contiguous piece of the slot; the workgroup then owns 64/LPT heads) when the head count
//     is a multiple of that, otherwise 64/LPT tokens of one head;
//   * every lane group keeps its OWN running (max, sum, acc[8]) online-softmax state, so the
//     inner loop needs no cross-group traffic: per token only the log2(LPT) butterfly steps
//     of the dot product;
//   * two-deep pipeline: while iteration i does its math, the K and V rows of iteration i + 1
//     (2 + 2 wave-loads, 4 KiB per wave) and the slot indices of iteration i + 2 are in flight,
//     so neither the row latency nor the index -> address dependency is exposed. A deeper queue is
//     slower, not faster: 4 + 4 loads per wave measured 458 us where 2 + 2 take 432 (8 + 8: 509);
//   * a workgroup = 4 waves owns a chunk of the sequence (split-KV: chunks of 512 tokens, shorter ones, down to 64,
//     when there would otherwise be too few workgroups for the chip, at most 256 per sequence); states are merged by
//     wave butterflies, then through LDS, then across chunks by a small lane-parallel second kernel.
//
// The two halves of the two-call form (scores to memory, then softmax and the sum over V from stored scores) are the same
// streaming kernel with the other half of the work compiled out: 588 -> 462 us for both at batch 64 with 156 000 cached
// tokens, and the second half no longer walks a long sequence with one workgroup (1 x 32768 tokens: 1709 -> 60 us).
//
// Head rows of whole 16-byte pieces up to 512 bytes at 16-byte aligned strides take the kernels above (rows of other
// lengths than 128, 256 or 512 bytes on the lanes of the next of those, the lanes past the row's end masked); any
// other head size or alignment (up to 1024 elements) takes the generic kernels at the end: one workgroup per (sequence, head), 256 tokens
// at a time, one token's dot product per thread and P.V with the threads over d. A correctness path.
#include <algorithm>
#include <mutex>

#include "common.hpp"

namespace amd {

constexpr float kLog2eTA = 1.4426950408889634f;
constexpr int kTaWaves = 4;
constexpr int kTaUnroll = 2;
constexpr int kTaChunk = 512;  // tokens of one sequence handled by one workgroup (grows for very long sequences)
constexpr int kTaMaxSplit = 256;  // decodeMergeWideKernel holds four splits' weights per lane (decodeMergeKernel: one, up to 64 splits)
constexpr int kTaMinChunk = 128;  // shorter chunks cost more in prologues, partial results and merging than they gain ...
constexpr int kTaTinyChunk = 64;  // ... unless even those leave CUs without a workgroup
constexpr int kTaWgsPerCu = 8;    // workgroups per CU the chunk length aims for

__device__ __forceinline__ int64_t ldIndex(const void* p, int64_t i, bool is64) {
  return is64 ? reinterpret_cast<const int64_t*>(p)[i] : static_cast<int64_t>(reinterpret_cast<const int32_t*>(p)[i]);
}

struct TaArgs {
  const void* q;
  const void* k;
  const void* v;
  const void* bLoc;
  const void* bStart;
  const void* bLen;
  bool loc64, start64, len64;
  bool generic;  // head rows the vector kernels do not take: the generic kernels run
  int64_t locRowStride;  // elements
  int64_t kSlotStride, kHeadStride, vSlotStride, vHeadStride;  // elements
  int64_t qBatchStride, qHeadStride;
  int64_t slots;
  int heads, kvHeads, d, maxLen, nsplit, chunk;
  float scaleLog2e;  // log2(e) / sqrt(d)
  const void* logits;  // two-call form: scores [heads, total_tokens], row h at logits + h * logitsHeadStride (elements)
  int64_t logitsHeadStride;
  int qGroups;  // grouped-query layouts: workgroups that share the query heads of one K/V head between them
  int batch;    // sequences (the grouped-query kernels decode a one-dimensional grid)
};

// Merge (m, l, acc) of another online-softmax stream into this one.
template <int E>
__device__ __forceinline__ void mergeState(float& m, float& l, float (&acc)[E], float m2, float l2,
                                           const float (&acc2)[E]) {
  float mn = fmaxf(m, m2);
  float c1 = (m == -INFINITY) ? 0.f : exp2f(m - mn);
  float c2 = (m2 == -INFINITY) ? 0.f : exp2f(m2 - mn);
  l = l * c1 + l2 * c2;
#pragma unroll
  for (int e = 0; e < E; ++e) acc[e] = acc[e] * c1 + acc2[e] * c2;
  m = mn;
}

// Sum over the LPT (8, 16 or 32) adjacent lanes that share a head row, left in all of them: within a row of 16 lanes
// the steps are lane permutations folded into the additions (see waveSum), no trips through the LDS crossbar. Decode
// attention at batch 64 (156 000 cached tokens): 373.7 -> 371.6 us; at batch 256: 1054 -> 1046 us.
template <int LPT>
__device__ __forceinline__ float headRowSum(float v) {
  static_assert(LPT == 8 || LPT == 16 || LPT == 32, "a head row is shared by 8, 16 or 32 lanes");
  v += lanePermuted<kDppQuadSwap1>(v);
  v += lanePermuted<kDppQuadSwap2>(v);
  v += lanePermuted<kDppHalfMirror>(v);
  if (LPT >= 16) v += lanePermuted<kDppMirror>(v);
  if (LPT >= 32) v += __shfl_xor(v, 16, 64);
  return v;
}

// c + a[0] b[0] + a[1] b[1] for two packed 16-bit pairs, in one instruction (fp32 accumulation).
template <typename T>
__device__ __forceinline__ float dotPair(uint32_t a, uint32_t b, float c) {
  static_assert(sizeof(T) == 2, "packed pairs of 16-bit elements");
  if constexpr (std::is_same<T, bf16_t>::value) {
    typedef __bf16 Pair __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(Pair, a), __builtin_bit_cast(Pair, b), c, false);
  } else {
    typedef _Float16 Pair __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(Pair, a), __builtin_bit_cast(Pair, b), c, false);
  }
}
template <typename T>
__device__ __forceinline__ uint32_t packPair(float lo, float hi) {
  const T l = static_cast<T>(lo), h = static_cast<T>(hi);
  return (uint32_t)__builtin_bit_cast(uint16_t, l) | ((uint32_t)__builtin_bit_cast(uint16_t, h) << 16);
}

// The three things the streaming kernel below can do with a chunk of a sequence: the whole decode attention (scores,
// online softmax and the sum over V), only the scores (first half of the two-call form: att[h, start_b + t]), or the
// softmax and the sum over V from scores computed earlier (second half of the two-call form).
enum TaMode { kTaFused = 0, kTaLogitsOut = 1, kTaReduceV = 2 };

// The value lane J of every aligned group of four lanes holds, in all four (one DPP move; every lane active).
template <int J>
__device__ __forceinline__ uint32_t quadBroadcast(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, J * 0x55, 0xf, 0xf, false);
}
template <int J>
__device__ __forceinline__ float quadBroadcast(float v) {
  return __builtin_bit_cast(float, quadBroadcast<J>(__builtin_bit_cast(uint32_t, v)));
}

// T: bf16_t / half_t (8 per 16 B) or float (4 per 16 B). LPT lanes cover one head row. LT: the type of the scores in
// memory (the two-call modes). QPK: query heads that share this workgroup's K/V head and are all served from one read
// of its rows (grouped-query layouts; 1 otherwise). With QPK > 1 the grid is one-dimensional and decoded so that the
// workgroups that share a K/V head's rows run next to each other on one XCD.
template <typename T, int LPT, bool HIW, int MODE = kTaFused, typename LT = float, int QPK = 1, bool PART = false>
__global__ __launch_bounds__(kTaWaves * 64) void decodeSplitKernel(TaArgs a, T* __restrict__ out,
                                                                     float* __restrict__ partial) {
  static_assert(QPK == 1 || !HIW, "several query heads per lane group: the lane groups of a wave take tokens, not heads");
  using V = typename Vec16<T>::type;
  constexpr int N = Vec16<T>::N;
  constexpr int TPW = 64 / LPT;  // tokens per wave-wide load
  constexpr bool kNeedK = MODE != kTaReduceV, kNeedV = MODE != kTaLogitsOut;
  // rows per wave in flight: 2 K + 2 V in the fused mode, 2 K or 2 V in the halves of the two-call form (at batch 64,
  // 156 000 tokens: scores 215 us with 2, 219 with 4, 229 with 6; second half 204 with 2, 212 with 3, 221 with 4)
  constexpr int UNR = kTaUnroll;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPT, grp = lane / LPT;
  // HIW: the lane groups of a wave take TPW consecutive heads of the same token (a wave load is TPW head rows, contiguous
  // in a slot) instead of TPW tokens of one head
  // Dispatch order: the chunk index is the slowest grid dimension and runs backwards, so the ragged part of the work
  // (the last, partly filled chunk of every sequence and the chunks only long sequences have) is handed out first and
  // the launch ends on whole chunks that finish together. Against sequence-major order, batch 64 x (512..4096):
  // 410.7 -> 406.8 us; 32 x (100..8192): 332 -> 323; 256 x (1024..2048): 1040 -> 1025, and with 8 K/V heads 413 -> 361.
  int split = (int)gridDim.z - 1 - (int)blockIdx.z, b = blockIdx.y;
  const int perKv = a.heads / a.kvHeads;
  int h, kvh, nq = 1;  // h: this lane group's (first) query head; nq: how many it serves (at most QPK)
  if constexpr (QPK == 1) {
    h = HIW ? blockIdx.x * TPW + grp : blockIdx.x;
    kvh = h / perKv;
  } else {
    // One-dimensional grid. A unit is a (K/V head, sequence, chunk); its qGroups workgroups read the same rows, so they
    // get consecutive places on one XCD (workgroup ids go round the 8 XCDs) and find the rows in that L2 after the
    // first of them has fetched them. Units go round the XCDs in the order the three-dimensional grid has: K/V head
    // fastest, then sequence, chunks from the last to the first.
    const int f = blockIdx.x, idx = f >> 3;
    const int g = idx % a.qGroups, u = (idx / a.qGroups) * 8 + (f & 7);
    if (u >= a.kvHeads * a.batch * a.nsplit) return;  // the grid is rounded up to whole rounds of the XCDs
    kvh = u % a.kvHeads;
    const int rest = u / a.kvHeads;
    b = rest % a.batch, split = a.nsplit - 1 - rest / a.batch;
    // the perKv sharers of a K/V head are dealt over the qGroups workgroups as evenly as they go (7 = 4 + 3); a group
    // short of QPK heads computes its last head again in the spare places and stores nothing from them
    const int base = perKv / a.qGroups, rem = perKv % a.qGroups;
    h = kvh * perKv + g * base + min(g, rem);
    nq = base + (g < rem ? 1 : 0);
  }
  auto headOf = [&](int j) { return QPK == 1 ? 0 : min(j, nq - 1); };  // offset of place j's head from h
  const int len = min(max((int)ldIndex(a.bLen, b, a.len64), 0), a.maxLen);  // a length beyond the table's width is cut to it
  const int begin = split * a.chunk;
  if (begin >= len && !(split == 0 && MODE != kTaLogitsOut)) return;  // nothing to do; split 0 still writes zeros for len == 0
  const int end = min(len, begin + a.chunk);
  const int64_t locBase = (int64_t)b * a.locRowStride + (a.maxLen - len);
  // the scores of this lane's (first) head for the tokens of sequence b (two-call modes); head h + j is j rows further
  LT* scores = nullptr;
  if constexpr (MODE != kTaFused)
    scores = static_cast<LT*>(const_cast<void*>(a.logits)) + h * a.logitsHeadStride + ldIndex(a.bStart, b, a.start64);

  // Two-call modes: the scores of the chunk pass through LDS, so memory sees them as whole rows of the chunk (one
  // coalesced read before the walk, one coalesced write after it) instead of four floats per wave and row on the way
  // (at batch 64, 156 000 tokens: scores 225 -> 219 us, second half 234 -> 205 us). Chunks longer than the buffer
  // (sequences past 131 072 tokens) keep the direct accesses.
  constexpr int kLdsScores = 1024;
  __shared__ float sbuf[MODE != kTaFused ? QPK * kLdsScores : 1];
  const bool useLds = MODE != kTaFused && a.chunk <= kLdsScores;
  // The slot indices of a 512-token chunk take the same way in those modes: one coalesced read of the chunk's piece of
  // b_loc, then the walk finds its slots in LDS instead of asking memory for one index per wave and row (indices
  // outside the pool are stored as -1): scores 216 -> 209 us, second half 205 -> 199 us at batch 64; 621 -> 595 and
  // 565 -> 549 us at batch 256 (8 x 4096 tokens, one round of workgroups: 48.5 -> 50.4 us). Not for the shorter chunks
  // of small batches, where the wait for the whole piece before the first row is requested weighs more, and not for
  // the fused mode, whose time moves by a few percent either way with anything that shifts the tail of the grid
  // (batch 64: 371 -> 392 us, batch 256: 1045 -> 1022 us, 8 x 4096: 90.6 -> 96.7 us).
  __shared__ int sidx[MODE != kTaFused ? kLdsScores : 1];
  const bool idxInLds = MODE != kTaFused && a.chunk >= kTaChunk && a.chunk <= kLdsScores && a.slots <= 0x7fffffff;
  if (idxInLds) {
    for (int i = threadIdx.x; i < end - begin; i += kTaWaves * 64) {
      const int64_t s = ldIndex(a.bLoc, locBase + begin + i, a.loc64);
      sidx[i] = s >= 0 && s < a.slots ? (int)s : -1;
    }
    if (!(MODE == kTaReduceV && useLds)) __syncthreads();  // (that mode's barrier below publishes both)
  }
  if constexpr (MODE == kTaReduceV) {
    if (useLds) {
#pragma unroll
      for (int j = 0; j < QPK; ++j)
        for (int i = threadIdx.x; i < end - begin; i += kTaWaves * 64)
          sbuf[j * kLdsScores + i] = static_cast<float>(scores[headOf(j) * a.logitsHeadStride + begin + i]) * kLog2eTA;
      __syncthreads();
    }
  }
  // Several query heads on 16-bit rows: the products are taken two at a time on the packed pairs as they come from
  // memory (q.k: a pair of q against a pair of k; p.v: the probabilities of the two rows in flight, rounded to 16
  // bits, against the two rows' values of one element), which halves the arithmetic instructions and needs no
  // conversions of K and V. 32 query heads on 8 K/V heads, batch 64 x (512..4096), fused: 184 -> 157 us (147 -> 110
  // registers, three -> four waves per SIMD); batch 256 x (1024..2048): 484 -> 413 us.
  constexpr bool kPairs = QPK > 1 && sizeof(T) == 2 && UNR == 2;
  // PART: a head row shorter than the LPT pieces the lane group spans (head sizes between the powers of two). The lanes
  // past its end read the row's first piece instead (memory that exists), hold zeros for q, so that they add nothing
  // to a score, and store nothing. (A variant of its own: with these selects in the kernel for whole rows the launch
  // at batch 64 reads 377 us against 366.)
  const bool live = !PART || sub * N < a.d;
  const int subIn = PART ? (live ? sub : 0) : sub;
  // scores leave the kernel in natural units, inside it they are in units of log2
  const float qScale = MODE == kTaLogitsOut ? a.scaleLog2e / kLog2eTA : a.scaleLog2e;
  float qf[kPairs ? 1 : QPK][N];
  uint32_t qp[kPairs ? QPK : 1][4];
  if constexpr (kNeedK) {
#pragma unroll
    for (int j = 0; j < QPK; ++j) {
      V qv = *reinterpret_cast<const V*>(reinterpret_cast<const T*>(a.q) + b * a.qBatchStride + (h + headOf(j)) * a.qHeadStride + subIn * N);
      if constexpr (kPairs) {
        const u32x4 raw = __builtin_bit_cast(u32x4, qv);
#pragma unroll
        for (int c = 0; c < 4; ++c) qp[j][c] = live ? raw[c] : 0u;
      } else {
#pragma unroll
        for (int e = 0; e < N; ++e) qf[j][e] = live ? static_cast<float>(qv[e]) * qScale : 0.f;
      }
    }
  }
  const T* kBase = kNeedK ? reinterpret_cast<const T*>(a.k) + kvh * a.kHeadStride + subIn * N : nullptr;
  const T* vBase = kNeedV ? reinterpret_cast<const T*>(a.v) + kvh * a.vHeadStride + subIn * N : nullptr;

  constexpr bool kShared = QPK == 4 && kPairs && MODE == kTaFused;
  float mOwn = -INFINITY, lOwn = 0.f;  // kShared: the state of head (sub & 3), see the loop
  float m[QPK], l[QPK], acc[QPK][N];
#pragma unroll
  for (int j = 0; j < QPK; ++j) {
    m[j] = -INFINITY, l[j] = 0.f;
#pragma unroll
    for (int e = 0; e < N; ++e) acc[j][e] = 0.f;
  }

  constexpr int TPI = HIW ? 1 : TPW;  // tokens per wave-wide load
  constexpr int STEP = kTaWaves * UNR * TPI;  // tokens per workgroup iteration
  // Two-deep software pipeline: while the rows of iteration i are being reduced, the K/V rows
  // of iteration i+1 and the slot indices of iteration i+2 are already in flight.
  int64_t slot[UNR];
  int slotTok[UNR];  // the token each slot index belongs to (the stored scores are addressed by it)
  V kr[UNR], vr[UNR], kn[UNR], vn[UNR];
  float lr[QPK][UNR], ln[QPK][UNR];  // stored scores of the rows (kTaReduceV)
  bool ok[UNR], okn[UNR];
  auto loadSlots = [&](int it) {
    int t0 = it + wave * UNR * TPI + (HIW ? 0 : grp);
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      int t = t0 + u * TPI;
      slotTok[u] = t;
      slot[u] = t >= end ? -1 : (idxInLds ? (int64_t)sidx[t - begin] : ldIndex(a.bLoc, locBase + t, a.loc64));
    }
  };
  auto loadRows = [&](V (&kk)[UNR], V (&vv)[UNR], float (&lg)[QPK][UNR], bool (&okk)[UNR]) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      okk[u] = slot[u] >= 0 && slot[u] < a.slots;  // slots outside the pool are skipped, never dereferenced
      int64_t s = okk[u] ? slot[u] : 0;
      if constexpr (kNeedK) kk[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(kBase + s * a.kSlotStride));
      if constexpr (kNeedV) vv[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(vBase + s * a.vSlotStride));
      if constexpr (MODE == kTaReduceV) {
#pragma unroll
        for (int j = 0; j < QPK; ++j)
          lg[j][u] = !okk[u] ? -INFINITY
                             : (useLds ? sbuf[j * kLdsScores + slotTok[u] - begin]
                                       : static_cast<float>(scores[headOf(j) * a.logitsHeadStride + slotTok[u]]) * kLog2eTA);
      }
    }
  };
  loadSlots(begin);
  loadRows(kr, vr, lr, ok);
  loadSlots(begin + STEP);
  for (int it = begin; it < end; it += STEP) {
    loadRows(kn, vn, ln, okn);    // rows of the next iteration (all masked past the end)
    loadSlots(it + 2 * STEP);     // indices of the one after
    float kf[kNeedK && QPK > 1 && !kPairs ? UNR : 1][N];  // several query heads on fp32 rows: the K rows are converted once
    if constexpr (kNeedK && QPK > 1 && !kPairs) {
#pragma unroll
      for (int u = 0; u < UNR; ++u)
#pragma unroll
        for (int e = 0; e < N; ++e) kf[u][e] = static_cast<float>(kr[u][e]);
    }
    // kPairs: element 2 c and 2 c + 1 of the two V rows, regrouped as (row 0, row 1) pairs of one element each
    uint32_t vlo[kPairs && kNeedV ? 4 : 1], vhi[kPairs && kNeedV ? 4 : 1];
    if constexpr (kPairs && kNeedV) {
      const u32x4 r0 = __builtin_bit_cast(u32x4, vr[0]), r1 = __builtin_bit_cast(u32x4, vr[1]);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        vlo[c] = __builtin_amdgcn_perm(r1[c], r0[c], 0x05040100u);
        vhi[c] = __builtin_amdgcn_perm(r1[c], r0[c], 0x07060302u);
      }
    }
    // kShared: four query heads on 16-bit rows in the fused mode. Every lane of a lane group holds the scores of all
    // four heads after the row sums, so the softmax update of head i is done by lanes i, i + 4, ... alone (their own
    // running maximum and sum: mOwn, lOwn) and the factors reach the other lanes by one quad broadcast each: three
    // exponentials per lane and pair of rows instead of twelve. The same arithmetic per head as the loop below.
    if constexpr (kShared) {
      float scAll[QPK][UNR];
#pragma unroll
      for (int j = 0; j < QPK; ++j)
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          const u32x4 kraw = __builtin_bit_cast(u32x4, kr[u]);
          float d = 0.f;
#pragma unroll
          for (int c = 0; c < 4; ++c) d = dotPair<T>(qp[j][c], kraw[c], d);
          d = headRowSum<LPT>(d) * qScale;
          scAll[j][u] = ok[u] ? d : -INFINITY;
        }
      const int own = sub & 3;
      float my[UNR];
#pragma unroll
      for (int u = 0; u < UNR; ++u)
        my[u] = own == 0 ? scAll[0][u] : (own == 1 ? scAll[1][u] : (own == 2 ? scAll[2][u] : scAll[3][u]));
      const float mn = fmaxf(mOwn, fmaxf(my[0], my[UNR - 1]));
      const bool any = mn != -INFINITY;
      const float corr = any ? __builtin_amdgcn_exp2f(mOwn - mn) : 1.f;  // mOwn == -inf gives 0: acc and l are 0 then anyway
      const float p0 = any ? __builtin_amdgcn_exp2f(my[0] - mn) : 0.f, p1 = any ? __builtin_amdgcn_exp2f(my[UNR - 1] - mn) : 0.f;
      lOwn = lOwn * corr + (p0 + p1);
      mOwn = mn;
      const uint32_t ppOwn = packPair<T>(p0, p1);
      staticFor<QPK>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const float cj = quadBroadcast<j>(corr);
        const uint32_t pp = quadBroadcast<j>(ppOwn);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          acc[j][2 * c] = dotPair<T>(pp, vlo[c], acc[j][2 * c] * cj);
          acc[j][2 * c + 1] = dotPair<T>(pp, vhi[c], acc[j][2 * c + 1] * cj);
        }
      });
    } else {
#pragma unroll
    for (int j = 0; j < QPK; ++j) {
      float sc[UNR];
      float mn = m[j];
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        if constexpr (kNeedK) {
          float d = 0.f;
          if constexpr (kPairs) {
            const u32x4 kraw = __builtin_bit_cast(u32x4, kr[u]);
#pragma unroll
            for (int c = 0; c < 4; ++c) d = dotPair<T>(qp[j][c], kraw[c], d);
            d = headRowSum<LPT>(d) * qScale;
          } else {
#pragma unroll
            for (int e = 0; e < N; ++e) d += qf[j][e] * (QPK > 1 ? kf[u][e] : static_cast<float>(kr[u][e]));
            d = headRowSum<LPT>(d);
          }
          sc[u] = ok[u] ? d : -INFINITY;
        } else {
          sc[u] = lr[j][u];
        }
        mn = fmaxf(mn, sc[u]);
      }
      if constexpr (MODE == kTaLogitsOut) {
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          const int t = it + wave * UNR * TPI + (HIW ? 0 : grp) + u * TPI;
          if (sub == 0 && t < end) {
            if (useLds) sbuf[j * kLdsScores + t - begin] = sc[u];
            else if (j < nq) scores[j * a.logitsHeadStride + t] = static_cast<LT>(sc[u]);
          }
        }
      } else if (mn != -INFINITY) {
        float corr = __builtin_amdgcn_exp2f(m[j] - mn);  // m == -inf gives 0, acc and l are 0 then anyway
        float p[UNR], ps = 0.f;
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          p[u] = __builtin_amdgcn_exp2f(sc[u] - mn);
          ps += p[u];
        }
        l[j] = l[j] * corr + ps;
        if constexpr (kPairs) {
          const uint32_t pp = packPair<T>(p[0], p[UNR - 1]);
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            acc[j][2 * c] = dotPair<T>(pp, vlo[c], acc[j][2 * c] * corr);
            acc[j][2 * c + 1] = dotPair<T>(pp, vhi[c], acc[j][2 * c + 1] * corr);
          }
        } else {
#pragma unroll
          for (int e = 0; e < N; ++e) {
            float s = acc[j][e] * corr;
#pragma unroll
            for (int u = 0; u < UNR; ++u) s += p[u] * static_cast<float>(vr[u][e]);
            acc[j][e] = s;
          }
        }
        m[j] = mn;
      }
    }
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      kr[u] = kn[u], vr[u] = vn[u], ok[u] = okn[u];
#pragma unroll
      for (int j = 0; j < QPK; ++j) lr[j][u] = ln[j][u];
    }
  }
  if constexpr (kShared) {  // every lane gets the four heads' maxima and sums back for the merges below
    staticFor<QPK>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      m[j] = quadBroadcast<j>(mOwn);
      l[j] = quadBroadcast<j>(lOwn);
    });
  }
  if constexpr (MODE == kTaLogitsOut) {
    if (useLds) {
      __syncthreads();
#pragma unroll
      for (int j = 0; j < QPK; ++j)
        if (j < nq)
          for (int i = threadIdx.x; i < end - begin; i += kTaWaves * 64)
            scores[j * a.logitsHeadStride + begin + i] = static_cast<LT>(sbuf[j * kLdsScores + i]);
    }
    return;
  }

  // merge the TPW lane groups of the wave (each holds other tokens of the same head)
  if (!HIW)
#pragma unroll
  for (int j = 0; j < QPK; ++j)
#pragma unroll
  for (int off = LPT; off < 64; off <<= 1) {
    float m2 = __shfl_xor(m[j], off, 64), l2 = __shfl_xor(l[j], off, 64), acc2[N];
#pragma unroll
    for (int e = 0; e < N; ++e) acc2[e] = __shfl_xor(acc[j][e], off, 64);
    mergeState<N>(m[j], l[j], acc[j], m2, l2, acc2);
  }
  // merge the waves through LDS: [wave][2 + LPT*N], one query head after the other
  constexpr int RG = HIW ? TPW : 1;  // lane groups with a state of their own
  const int rg = HIW ? grp : 0;
  __shared__ float red[kTaWaves][RG][2 + LPT * N];
#pragma unroll
  for (int j = 0; j < QPK; ++j) {
    if (j > 0) __syncthreads();  // wave 0 has read the previous head's states
    if (HIW || grp == 0) {
      if (sub == 0) red[wave][rg][0] = m[j], red[wave][rg][1] = l[j];
#pragma unroll
      for (int e = 0; e < N; ++e) red[wave][rg][2 + sub * N + e] = acc[j][e];
    }
    __syncthreads();
    if (wave == 0 && (HIW || grp == 0) && j < nq) {
#pragma unroll
      for (int w = 1; w < kTaWaves; ++w) {
        float acc2[N];
#pragma unroll
        for (int e = 0; e < N; ++e) acc2[e] = red[w][rg][2 + sub * N + e];
        mergeState<N>(m[j], l[j], acc[j], red[w][rg][0], red[w][rg][1], acc2);
      }
      if (a.nsplit == 1) {
        float inv = l[j] > 0.f ? 1.f / l[j] : 0.f;
        V o;
#pragma unroll
        for (int e = 0; e < N; ++e) o[e] = static_cast<T>(acc[j][e] * inv);
        if (live) *reinterpret_cast<V*>(out + ((int64_t)b * a.heads + h + j) * a.d + sub * N) = o;
      } else {
        float* dst = partial + (((int64_t)b * a.heads + h + j) * a.nsplit + split) * (2 + a.d);
        if (sub == 0) dst[0] = m[j], dst[1] = l[j];
        if (live) {
#pragma unroll
          for (int e = 0; e < N; ++e) dst[2 + sub * N + e] = acc[j][e];
        }
      }
    }
  }
}

// out[b,h,:] = merge over the chunks that hold tokens. One wave per (b,h): lane s takes the (max, sum) of
// split s, a butterfly gives the global max and normaliser, then every lane combines its elements over the
// splits. Nothing here waits for anything else before it is requested: the sequence length, the (max, sum)
// pairs and the first eight splits' elements are all loaded up front (splits that hold no tokens were never
// written; what is read from them is discarded by a select, never multiplied).
template <typename T>
__global__ __launch_bounds__(256) void decodeMergeKernel(T* __restrict__ out, const float* __restrict__ partial,
                                                          const void* bLen, bool len64, int64_t pairs, int heads,
                                                          int d, int nsplit, int chunk) {
  constexpr int kBatch = 8, kMaxPerLane = 4;  // d <= 256
  const int lane = threadIdx.x & 63;
  const int64_t pair = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int b = (int)(pair / heads);
  const int row = 2 + d;
  const float* src = partial + pair * nsplit * row;
  float ms = -INFINITY, ls = 0.f;
  if (lane < nsplit) {
    ms = src[lane * row];
    ls = src[lane * row + 1];
  }
  const int len = (int)ldIndex(bLen, b, len64);
  float acc[kMaxPerLane] = {0.f, 0.f, 0.f, 0.f};
  float m = 0.f, wgt = 0.f;
  int used = 0;
  for (int sb = 0; sb < nsplit; sb += kBatch) {
    float v[kBatch][kMaxPerLane];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const float* r = src + (int64_t)min(sb + u, nsplit - 1) * row + 2;
#pragma unroll
      for (int k = 0; k < kMaxPerLane; ++k) {
        const int e = lane + 64 * k;
        v[u][k] = e < d ? r[e] : 0.f;
      }
    }
    if (sb == 0) {  // the weights of all splits, once, while the loads above are in flight
      used = len <= 0 ? 1 : min(nsplit, (len + chunk - 1) / chunk);
      if (lane >= used) ms = -INFINITY, ls = 0.f;
      m = waveMax(ms);
      wgt = (ms == -INFINITY) ? 0.f : exp2f(ms - m);
      const float l = waveSum(ls * wgt);
      wgt *= l > 0.f ? 1.f / l : 0.f;
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int sp = sb + u;
      const float w = __shfl(wgt, sp & 63, 64);
#pragma unroll
      for (int k = 0; k < kMaxPerLane; ++k) acc[k] += sp < used ? w * v[u][k] : 0.f;
    }
  }
#pragma unroll
  for (int k = 0; k < kMaxPerLane; ++k) {
    const int e = lane + 64 * k;
    if (e < d) out[pair * d + e] = static_cast<T>(acc[k]);
  }
}

// The same merge for 65 to 256 splits (few sequences with long contexts, cut fine to fill the chip): one workgroup per
// (b, h). Every wave works out the weights of all splits (lane s holds splits s, s + 64, s + 128, s + 192), then wave w
// combines splits w, w + 4, ... and the four sums meet in LDS.
template <typename T>
__global__ __launch_bounds__(256) void decodeMergeWideKernel(T* __restrict__ out, const float* __restrict__ partial,
                                                              const void* bLen, bool len64, int heads, int d, int nsplit,
                                                              int chunk) {
  constexpr int kBatch = 8, kMaxPerLane = 4, kPerLane = kTaMaxSplit / 64;  // d <= 256
  __shared__ float red[4][64 * kMaxPerLane];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t pair = blockIdx.x;
  const int b = (int)(pair / heads);
  const int row = 2 + d;
  const float* src = partial + pair * nsplit * row;
  const int len = (int)ldIndex(bLen, b, len64);
  const int used = len <= 0 ? 1 : min(nsplit, (len + chunk - 1) / chunk);
  float ms[kPerLane], ls[kPerLane], wgt[kPerLane];
  float m = -INFINITY;
#pragma unroll
  for (int k = 0; k < kPerLane; ++k) {
    const int sp = lane + 64 * k;
    ms[k] = sp < used ? src[sp * row] : -INFINITY;  // splits that hold no tokens were never written
    ls[k] = sp < used ? src[sp * row + 1] : 0.f;
    m = fmaxf(m, ms[k]);
  }
  m = waveMax(m);
  float lsum = 0.f;
#pragma unroll
  for (int k = 0; k < kPerLane; ++k) {
    wgt[k] = ms[k] == -INFINITY ? 0.f : exp2f(ms[k] - m);
    lsum += ls[k] * wgt[k];
  }
  const float l = waveSum(lsum);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  float acc[kMaxPerLane] = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = wave; s0 < used; s0 += 4 * kBatch) {
    float v[kBatch][kMaxPerLane];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const float* r = src + (int64_t)min(s0 + 4 * u, nsplit - 1) * row + 2;
#pragma unroll
      for (int k = 0; k < kMaxPerLane; ++k) {
        const int e = lane + 64 * k;
        v[u][k] = e < d ? r[e] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int sp = s0 + 4 * u, owner = sp >> 6;  // wave-uniform
      float w = wgt[0];
#pragma unroll
      for (int k = 1; k < kPerLane; ++k) w = owner == k ? wgt[k] : w;
      w = __shfl(w, sp & 63, 64) * inv;
#pragma unroll
      for (int k = 0; k < kMaxPerLane; ++k) acc[k] += sp < used ? w * v[u][k] : 0.f;
    }
  }
#pragma unroll
  for (int k = 0; k < kMaxPerLane; ++k) red[wave][lane + 64 * k] = acc[k];
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int k = 0; k < kMaxPerLane; ++k) {
      const int e = lane + 64 * k;
      if (e < d) out[pair * d + e] = static_cast<T>(red[0][e] + red[1][e] + red[2][e] + red[3][e]);
    }
  }
}

// ------------------------------------------------ any head size: generic kernels --
constexpr int kTaGenericMaxD = 1024;  // four elements of the head row per thread

// max / sum of one value per thread over the workgroup of 256 (red: 4 floats of LDS; two barriers)
__device__ __forceinline__ float blockMax256(float v, float* red) {
  v = waveMax(v);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  return v;
}
__device__ __forceinline__ float blockSum256(float v, float* red) {
  v = waveSum(v);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  v = red[0] + red[1] + red[2] + red[3];
  __syncthreads();
  return v;
}

// Fused decode attention, one workgroup per (sequence, head) (ext_ops.py:100-133). Tokens whose slot lies outside the
// pool are skipped, as in the vector kernels; a sequence of length 0 gives zeros.
template <typename T>
__global__ __launch_bounds__(256) void decodeGenericKernel(TaArgs a, T* __restrict__ out) {
  __shared__ float prob[256];
  __shared__ int64_t slotOf[256];
  __shared__ float red[4];
  const int h = blockIdx.x, b = blockIdx.z, tid = threadIdx.x;
  const int len = min(max((int)ldIndex(a.bLen, b, a.len64), 0), a.maxLen);
  const int kvh = h / (a.heads / a.kvHeads);
  const int64_t locBase = (int64_t)b * a.locRowStride + (a.maxLen - len);
  const T* q = reinterpret_cast<const T*>(a.q) + b * a.qBatchStride + h * a.qHeadStride;
  const T* kHead = reinterpret_cast<const T*>(a.k) + kvh * a.kHeadStride;
  const T* vHead = reinterpret_cast<const T*>(a.v) + kvh * a.vHeadStride;
  float m = -INFINITY, l = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};  // acc[j]: element tid + 256 j of the output row
  for (int t0 = 0; t0 < len; t0 += 256) {
    const int t = t0 + tid;
    int64_t slot = t < len ? ldIndex(a.bLoc, locBase + t, a.loc64) : -1;
    if (slot >= a.slots) slot = -1;
    float sc = -INFINITY;  // in the scaled log2 domain
    if (slot >= 0) {
      const T* k = kHead + slot * a.kSlotStride;
      float d = 0.f;
      for (int e = 0; e < a.d; ++e) d += static_cast<float>(q[e]) * static_cast<float>(k[e]);
      sc = d * a.scaleLog2e;
    }
    const float mn = fmaxf(m, blockMax256(sc, red));
    const float pr = sc == -INFINITY ? 0.f : exp2f(sc - mn);
    prob[tid] = pr;
    slotOf[tid] = slot;
    const float bs = blockSum256(pr, red);  // its barriers also publish prob / slotOf
    const float corr = m == -INFINITY ? 0.f : exp2f(m - mn);
    l = l * corr + bs;
    const int cnt = min(256, len - t0);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = tid + 256 * j;
      if (e < a.d) {
        float x = acc[j] * corr;
        for (int i = 0; i < cnt; ++i)
          if (slotOf[i] >= 0) x += prob[i] * static_cast<float>(vHead[slotOf[i] * a.vSlotStride + e]);
        acc[j] = x;
      }
    }
    m = mn;
    __syncthreads();  // prob / slotOf are rewritten by the next block of tokens
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int e = tid + 256 * j;
    if (e < a.d) out[((int64_t)b * a.heads + h) * a.d + e] = static_cast<T>(acc[j] * inv);
  }
}

// Two-call form, first half: att[h, start_b + t] = q[b,h,:] . k[slot_t,h,:] / sqrt(d); -inf for a slot outside the pool.
template <typename T, typename OT>
__global__ __launch_bounds__(256) void tokenLogitsGenericKernel(TaArgs a, OT* __restrict__ att, int64_t attHeadStride) {
  const int h = blockIdx.x, b = blockIdx.z;
  const int len = min(max((int)ldIndex(a.bLen, b, a.len64), 0), a.maxLen);
  const int64_t start = ldIndex(a.bStart, b, a.start64);
  const int begin = blockIdx.y * a.chunk, end = min(len, begin + a.chunk);
  const int kvh = h / (a.heads / a.kvHeads);
  const int64_t locBase = (int64_t)b * a.locRowStride + (a.maxLen - len);
  const T* q = reinterpret_cast<const T*>(a.q) + b * a.qBatchStride + h * a.qHeadStride;
  const T* kHead = reinterpret_cast<const T*>(a.k) + kvh * a.kHeadStride;
  const float scale = a.scaleLog2e / kLog2eTA;
  for (int t = begin + threadIdx.x; t < end; t += 256) {
    const int64_t slot = ldIndex(a.bLoc, locBase + t, a.loc64);
    float v = -INFINITY;
    if (slot >= 0 && slot < a.slots) {
      const T* k = kHead + slot * a.kSlotStride;
      float d = 0.f;
      for (int e = 0; e < a.d; ++e) d += static_cast<float>(q[e]) * static_cast<float>(k[e]);
      v = d * scale;
    }
    att[h * attHeadStride + start + t] = static_cast<OT>(v);
  }
}

// Two-call form, second half: out[b,h,:] = softmax(logics[h, start_b : start_b + len]) . v[slots].
template <typename T, typename LT>
__global__ __launch_bounds__(256) void softmaxReduceVGenericKernel(TaArgs a, T* __restrict__ out, const LT* __restrict__ logics,
                                                                    int64_t logHeadStride) {
  __shared__ float prob[256];
  __shared__ int64_t slotOf[256];
  __shared__ float red[4];
  const int h = blockIdx.x, b = blockIdx.z, tid = threadIdx.x;
  const int len = min(max((int)ldIndex(a.bLen, b, a.len64), 0), a.maxLen);
  const int64_t start = ldIndex(a.bStart, b, a.start64);
  const int kvh = h / (a.heads / a.kvHeads);
  const int64_t locBase = (int64_t)b * a.locRowStride + (a.maxLen - len);
  const LT* lg = logics + h * logHeadStride + start;
  const T* vHead = reinterpret_cast<const T*>(a.v) + kvh * a.vHeadStride;
  float m = -INFINITY;
  for (int t = tid; t < len; t += 256) m = fmaxf(m, static_cast<float>(lg[t]));
  m = blockMax256(m, red);
  const float mS = m == -INFINITY ? 0.f : m * kLog2eTA;
  float sum = 0.f;
  for (int t = tid; t < len; t += 256) sum += exp2f(static_cast<float>(lg[t]) * kLog2eTA - mS);
  sum = blockSum256(sum, red);
  const float inv = sum > 0.f ? 1.f / sum : 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int t0 = 0; t0 < len; t0 += 256) {
    const int t = t0 + tid;
    int64_t slot = t < len ? ldIndex(a.bLoc, locBase + t, a.loc64) : -1;
    if (slot >= a.slots) slot = -1;
    prob[tid] = slot >= 0 ? exp2f(static_cast<float>(lg[t]) * kLog2eTA - mS) : 0.f;
    slotOf[tid] = slot;
    __syncthreads();
    const int cnt = min(256, len - t0);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = tid + 256 * j;
      if (e < a.d) {
        float x = acc[j];
        for (int i = 0; i < cnt; ++i)
          if (slotOf[i] >= 0) x += prob[i] * static_cast<float>(vHead[slotOf[i] * a.vSlotStride + e]);
        acc[j] = x;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int e = tid + 256 * j;
    if (e < a.d) out[((int64_t)b * a.heads + h) * a.d + e] = static_cast<T>(acc[j] * inv);
  }
}

// ---------------------------------------------------------------- host side --
struct TaViews {
  TensorView q, k, v, loc, start, len;
};

static diopiError_t checkIndex(const TensorView& t, const char* name) {
  AMD_CHECK(t.defined(), "token attention: %s is null", name);
  AMD_CHECK(t.dtype == diopi_dtype_int32 || t.dtype == diopi_dtype_int64, "token attention: %s must be int32/int64, got %s",
            name, dtypeName(t.dtype));
  AMD_CHECK(t.isContiguous() || t.ndim == 2, "token attention: %s must be dense", name);
  return diopiSuccess;
}

static diopiError_t fillArgs(const TaViews& t, bool needK, bool needV, int maxLen, TaArgs* a) {
  const TensorView& q = t.q;
  AMD_CHECK(q.defined() && q.ndim == 3, "token attention: q must be [batch, heads, head_dim]");
  AMD_CHECK(q.stride[2] == 1 || q.shape[2] == 1, "token attention: q head_dim must be contiguous");
  const TensorView& kv = needK ? t.k : t.v;
  AMD_CHECK(kv.defined() && kv.ndim == 3, "token attention: k/v must be [slots, kv_heads, head_dim]");
  AMD_CHECK(kv.dtype == q.dtype, "token attention: k/v dtype %s differs from q dtype %s", dtypeName(kv.dtype),
            dtypeName(q.dtype));
  AMD_CHECK(kv.shape[2] == q.shape[2], "token attention: head_dim mismatch (%ld vs %ld)", (long)kv.shape[2],
            (long)q.shape[2]);
  AMD_CHECK(kv.shape[1] > 0 && q.shape[1] % kv.shape[1] == 0, "token attention: %ld heads are not a multiple of %ld kv heads",
            (long)q.shape[1], (long)kv.shape[1]);
  AMD_CHECK(kv.stride[2] == 1, "token attention: k/v head_dim must be contiguous");
  AMD_CHECK(kv.shape[0] > 0, "token attention: the KV pool has no slots");
  if (needK && needV) {
    AMD_CHECK(t.v.defined() && t.v.ndim == 3 && t.v.dtype == q.dtype && t.v.stride[2] == 1, "token attention: bad v");
    for (int d = 0; d < 3; ++d) AMD_CHECK(t.v.shape[d] == t.k.shape[d], "token attention: k and v shapes differ");
  }
  AMD_TRY(checkIndex(t.loc, "b_loc"));
  AMD_TRY(checkIndex(t.start, "b_start_loc"));
  AMD_TRY(checkIndex(t.len, "b_seq_len"));
  const int64_t batch = q.shape[0];
  AMD_CHECK(t.loc.ndim == 2 && t.loc.shape[0] == batch && (t.loc.stride[1] == 1 || t.loc.shape[1] == 1),
            "token attention: b_loc must be [batch, n] with a contiguous last dim");
  AMD_CHECK(maxLen >= 0 && t.loc.shape[1] >= maxLen, "token attention: b_loc has %ld columns, max_input_len is %d",
            (long)t.loc.shape[1], maxLen);
  AMD_CHECK(t.start.numel == batch && t.len.numel == batch, "token attention: b_start_loc/b_seq_len must have %ld entries",
            (long)batch);
  AMD_CHECK(q.dtype == diopi_dtype_bfloat16 || q.dtype == diopi_dtype_float16 || q.dtype == diopi_dtype_float32,
            "token attention: unsupported dtype %s", dtypeName(q.dtype));
  const int64_t bytes = q.shape[2] * q.itemsize;
  // head rows of whole 16-byte pieces up to 512 bytes: the streaming kernels span them with 8, 16 or 32 lanes
  bool vector = bytes % 16 == 0 && bytes >= 16 && bytes <= 512 && q.aligned16() && kv.aligned16() &&
                (kv.stride[0] * kv.itemsize) % 16 == 0 && (kv.stride[1] * kv.itemsize) % 16 == 0 &&
                (q.stride[0] * q.itemsize) % 16 == 0 && (q.stride[1] * q.itemsize) % 16 == 0;
  if (needK && needV)
    vector = vector && t.v.aligned16() && (t.v.stride[0] * q.itemsize) % 16 == 0 && (t.v.stride[1] * q.itemsize) % 16 == 0;
  a->generic = !vector;
  AMD_CHECK(vector || q.shape[2] <= kTaGenericMaxD, "token attention: head_dim %ld exceeds %d", (long)q.shape[2], kTaGenericMaxD);
  a->q = q.data;
  a->k = needK ? t.k.data : nullptr;
  a->v = needV ? t.v.data : nullptr;
  a->bLoc = t.loc.data;
  a->bStart = t.start.data;
  a->bLen = t.len.data;
  a->loc64 = t.loc.dtype == diopi_dtype_int64;
  a->start64 = t.start.dtype == diopi_dtype_int64;
  a->len64 = t.len.dtype == diopi_dtype_int64;
  a->locRowStride = t.loc.stride[0];
  a->kSlotStride = needK ? t.k.stride[0] : 0;
  a->kHeadStride = needK ? t.k.stride[1] : 0;
  a->vSlotStride = needV ? t.v.stride[0] : 0;
  a->vHeadStride = needV ? t.v.stride[1] : 0;
  a->qBatchStride = q.stride[0];
  a->qHeadStride = q.stride[1];
  a->slots = kv.shape[0];
  a->heads = (int)q.shape[1];
  a->kvHeads = (int)kv.shape[1];
  a->d = (int)q.shape[2];
  a->maxLen = maxLen;
  a->nsplit = 1;
  a->logits = nullptr, a->logitsHeadStride = 0, a->qGroups = 1, a->batch = (int)q.shape[0];
  // at most kTaMaxSplit chunks per sequence; chunks stay a multiple of 64 tokens
  a->chunk = kTaChunk;
  if ((int64_t)maxLen > (int64_t)kTaChunk * kTaMaxSplit) a->chunk = (int)(ceilDiv(ceilDiv(maxLen, kTaMaxSplit), 64) * 64);
  a->scaleLog2e = kLog2eTA / sqrtf((float)q.shape[2]);
  return diopiSuccess;
}

// Chunk length of the split over a sequence for the streaming kernels (decodeSplitKernel in its three modes).
static void chooseChunk(TaArgs* a, int64_t groupsPerSeq, int64_t batch, int maxInputLen) {
  // A workgroup walks its chunk with two loads per wave in flight, so the rate comes from the number of workgroups a
  // CU holds at once. Few sequences or short ones are cut into smaller chunks until there are about kTaWgsPerCu
  // workgroups per CU; large batches keep the 512-token chunks, whose partial results are fewer. Measured (us, 32 heads
  // x 128, bf16, with 512-token chunks -> with these): 1 x 2048 tokens 72 -> 20, 1 x 32768 130 -> 96, 8 x 4096 130 -> 91,
  // 4 x (100 .. 16384) 123 -> 86, 64 x (256 .. 512) 101 -> 80; 64 x (512 .. 4096) and 256 x (1024 .. 2048) keep their chunks.
  const int64_t groups = groupsPerSeq * batch, cus = computeUnits(), len = std::max(maxInputLen, 1);
  const int64_t wantSplits = std::max<int64_t>(1, ceilDiv(kTaWgsPerCu * cus, groups));
  const int64_t fine = ceilDiv(ceilDiv(len, wantSplits), 64) * 64;
  const int64_t capped = ceilDiv(ceilDiv(len, (int64_t)kTaMaxSplit), 64) * 64;  // at most kTaMaxSplit chunks
  const int64_t shortest = groups * ceilDiv(len, (int64_t)kTaMinChunk) < cus ? kTaTinyChunk : kTaMinChunk;
  a->chunk = (int)std::max(std::max(capped, shortest), std::min<int64_t>(a->chunk, fine));
}

#define TA_DISPATCH(DTYPE, BYTES, CALL)                                                        \
  do {                                                                                         \
    if (DTYPE == diopi_dtype_bfloat16) {                                                       \
      if (BYTES == 128) { CALL(bf16_t, 8); } else if (BYTES == 256) { CALL(bf16_t, 16); } else { CALL(bf16_t, 32); } \
    } else if (DTYPE == diopi_dtype_float16) {                                                 \
      if (BYTES == 128) { CALL(half_t, 8); } else if (BYTES == 256) { CALL(half_t, 16); } else { CALL(half_t, 32); } \
    } else if (DTYPE == diopi_dtype_float32) {                                                 \
      if (BYTES == 128) { CALL(float, 8); } else if (BYTES == 256) { CALL(float, 16); } else { CALL(float, 32); }   \
    } else {                                                                                   \
      setLastError("token attention: unsupported dtype %s", dtypeName(DTYPE));                 \
      return diopiErrorOccurred;                                                               \
    }                                                                                          \
  } while (0)

#define TA_GENERIC_DISPATCH(DTYPE, CALL)                                \
  do {                                                                  \
    if (DTYPE == diopi_dtype_bfloat16) { CALL(bf16_t); }                \
    else if (DTYPE == diopi_dtype_float16) { CALL(half_t); }            \
    else { CALL(float); }                                               \
  } while (0)

// Split-KV partial results for the entry point that allocates nothing. Every device the library's code object is
// loaded on holds its own copy of this array, at its own address, until the process ends.
constexpr int64_t kDecodeScratchBytes = 32ll << 20;
static __device__ __align__(256) unsigned char scratch[kDecodeScratchBytes];

// The array's name is a host-side stand-in; its device address is looked up once per device, with that device
// current, and only that address is ever handed to a kernel.
static diopiError_t decodeScratch(float** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static void* addr[kMaxDevices] = {};
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  AMD_CHECK(e == hipSuccess && dev >= 0 && dev < kMaxDevices, "token attention: no current device (%s)", hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(mu);
  if (addr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    AMD_CHECK(e == hipSuccess && p != nullptr, "token attention: hipGetSymbolAddress of the scratch array failed on device %d (%s)",
              dev, hipGetErrorString(e));
    addr[dev] = p;
  }
  *out = static_cast<float*>(addr[dev]);
  return diopiSuccess;
}

}  // namespace amd

using namespace amd;

// staticScratch: partial results go to the library's own device array instead of workspace from the context.
// Launches decodeSplitKernel in one of its modes over (head groups, chunks, sequences) and, for the modes that produce
// the attention output, merges the chunks. scoresF32: the stored scores of the two-call modes are float32 (else T).
template <int MODE>
static diopiError_t streamChunks(diopiContextHandle_t ctx, hipStream_t stream, TaArgs a, diopiDtype_t dtype, int64_t bytes,
                                 int64_t batch, int maxInputLen, void* outPtr, bool scoresF32, bool staticScratch,
                                 float* ownScratch) {
  // a head row is spanned by 8, 16 or 32 lanes of 16 bytes: the next of 128 / 256 / 512 bytes (the kernel masks the rest)
  const bool partRows = bytes != 128 && bytes != 256 && bytes != 512;
  bytes = bytes <= 128 ? 128 : bytes <= 256 ? 256 : 512;
  // The lane groups of a wave take consecutive heads of one token when the head count allows it: a wave load is then
  // one contiguous piece of a slot (1 KiB) instead of head rows of four different slots (431 -> 421 us at batch 64,
  // 32 heads x 128, 156 043 cached tokens).
  const int tpw = (int)(64 / std::max<int64_t>(1, bytes / 16));
  // (the two-call modes keep four tokens of one head per wave load and a workgroup per head: at batch 64, 156 000
  // tokens, with the chunk's scores staged in LDS either way, four heads per workgroup read 244 against 219 us for the
  // scores and 238 against 205 us for the second half)
  // Grouped-query layouts: one read of a K/V row serves four (or two) of the query heads that share it, with their
  // softmax states side by side in the lane group's registers; more sharers than that are dealt over several
  // workgroups that run on the same XCD. At batch 64 x (512..4096) tokens, 32 query heads on 8 K/V heads (every query
  // head used to read the rows for itself): fused 236 -> 157 us, scores 214 -> 74 us, second half 205 -> 106 us; 64
  // query heads on 8: 405 -> 240 us fused. Sharing factors that are no multiple of four are dealt over the workgroups
  // as evenly as they go (28 query heads on 4 K/V heads: 4 + 3 per K/V head).
  const int perKv = a.heads / a.kvHeads;
  const int qpk = perKv >= 3 ? 4 : perKv;  // 1, 2 or 4 query heads per read
  a.qGroups = (perKv + qpk - 1) / qpk;
  const bool hiw = qpk == 1 && MODE == kTaFused && (bytes == 128 || bytes == 256 || bytes == 512) && a.heads % tpw == 0;
  const int groupsPerSeq = qpk > 1 ? a.kvHeads * a.qGroups : (hiw ? a.heads / tpw : a.heads);
  chooseChunk(&a, groupsPerSeq, batch, maxInputLen);
  a.nsplit = (int)std::max<int64_t>(1, ceilDiv(maxInputLen, a.chunk));
  AMD_CHECK(batch <= 65535 && a.nsplit <= 65535, "token attention: batch %ld / splits %d exceed the grid limits", (long)batch,
            a.nsplit);
  float* partial = nullptr;
  if (MODE != kTaLogitsOut && a.nsplit > 1) {
    const int64_t need = (int64_t)batch * a.heads * a.nsplit * (2 + a.d) * (int64_t)sizeof(float);
    if (staticScratch) {
      AMD_CHECK(need <= kDecodeScratchBytes,
                "token attention: batch %ld x %d heads x %d splits of %d tokens needs %ld bytes of partial results, the "
                "entry point that allocates nothing holds %ld; use diopiTokenDecodeAttentionInference",
                (long)batch, a.heads, a.nsplit, a.chunk, (long)need, (long)kDecodeScratchBytes);
      // Nothing has to start at zero: the split kernel writes every (max, sum, acc) row the merge kernel uses, and
      // rows of splits that hold no tokens are read but discarded by a select.
      partial = ownScratch;
    } else {
      void* ws = nullptr;
      AMD_TRY(requireWorkspace(ctx, need, &ws));
      partial = static_cast<float*>(ws);
    }
  }
  dim3 grid((unsigned)groupsPerSeq, (unsigned)batch, a.nsplit), block(kTaWaves * 64);
  if (qpk > 1) {
    const int64_t units = (int64_t)a.kvHeads * batch * a.nsplit, wgs = ceilDiv(units, (int64_t)8) * 8 * a.qGroups;
    AMD_CHECK(wgs < ((int64_t)1 << 31), "token attention: %ld workgroups exceed the grid limits", (long)wgs);
    grid = dim3((unsigned)wgs, 1, 1);
  }
#define STREAM_CALL_PART(T, LPT, LT, PART)                                                                                           \
  if (qpk == 4) hipLaunchKernelGGL((decodeSplitKernel<T, LPT, false, MODE, LT, 4, PART>), grid, block, 0, stream, a, static_cast<T*>(outPtr), partial); \
  else if (qpk == 2) hipLaunchKernelGGL((decodeSplitKernel<T, LPT, false, MODE, LT, 2, PART>), grid, block, 0, stream, a, static_cast<T*>(outPtr), partial); \
  else if (hiw) hipLaunchKernelGGL((decodeSplitKernel<T, LPT, true, MODE, LT, 1, PART>), grid, block, 0, stream, a, static_cast<T*>(outPtr), partial); \
  else hipLaunchKernelGGL((decodeSplitKernel<T, LPT, false, MODE, LT, 1, PART>), grid, block, 0, stream, a, static_cast<T*>(outPtr), partial)
#define STREAM_CALL_AS(T, LPT, LT)            \
  if (partRows) {                             \
    STREAM_CALL_PART(T, LPT, LT, true);       \
  } else {                                    \
    STREAM_CALL_PART(T, LPT, LT, false);      \
  }
#define STREAM_CALL(T, LPT)                                \
  if (MODE == kTaFused || scoresF32) {                     \
    STREAM_CALL_AS(T, LPT, float);                         \
  } else {                                                 \
    STREAM_CALL_AS(T, LPT, T);                             \
  }
  TA_DISPATCH(dtype, bytes, STREAM_CALL);
#undef STREAM_CALL
#undef STREAM_CALL_AS
#undef STREAM_CALL_PART
  AMD_LAUNCH_CHECK();
  if (MODE == kTaLogitsOut) return diopiSuccess;
  if (a.nsplit > 64) {
    const int64_t pairs = batch * a.heads;
    AMD_CHECK(a.nsplit <= kTaMaxSplit && a.d <= 256, "token attention: %d splits of head size %d cannot be merged", a.nsplit, a.d);
#define MERGE_WIDE_CALL(T, LPT)                                                                                                      \
  hipLaunchKernelGGL((decodeMergeWideKernel<T>), dim3((unsigned)pairs), dim3(256), 0, stream, static_cast<T*>(outPtr), partial, a.bLen, \
                     a.len64, a.heads, a.d, a.nsplit, a.chunk)
    TA_DISPATCH(dtype, bytes, MERGE_WIDE_CALL);
#undef MERGE_WIDE_CALL
    AMD_LAUNCH_CHECK();
  } else if (a.nsplit > 1) {
    int64_t pairs = batch * a.heads;
    dim3 mgrid((unsigned)ceilDiv(pairs, 4)), mblock(256);
#define MERGE_CALL(T, LPT)                                                                                                     \
  hipLaunchKernelGGL((decodeMergeKernel<T>), mgrid, mblock, 0, stream, static_cast<T*>(outPtr), partial, a.bLen, a.len64, pairs, \
                     a.heads, a.d, a.nsplit, a.chunk)
    TA_DISPATCH(dtype, bytes, MERGE_CALL);
#undef MERGE_CALL
    AMD_LAUNCH_CHECK();
  }
  return diopiSuccess;
}

static diopiError_t decodeAttention(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t qH,
                                    diopiConstTensorHandle_t kH, diopiConstTensorHandle_t vH, diopiConstTensorHandle_t locH,
                                    diopiConstTensorHandle_t startH, diopiConstTensorHandle_t lenH, int maxInputLen,
                                    bool staticScratch) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TaViews t;
  TensorView out;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(qH, &t.q, "q"));
  AMD_TRY(getView(kH, &t.k, "k"));
  AMD_TRY(getView(vH, &t.v, "v"));
  AMD_TRY(getView(locH, &t.loc, "b_loc"));
  AMD_TRY(getView(startH, &t.start, "b_start_loc"));
  AMD_TRY(getView(lenH, &t.len, "b_seq_len"));
  TaArgs a;
  AMD_TRY(fillArgs(t, true, true, maxInputLen, &a));
  AMD_CHECK(out.defined() && out.dtype == t.q.dtype && out.numel == t.q.numel && out.isContiguous(),
            "token attention: out must be a dense tensor shaped like q");
  const int64_t batch = t.q.shape[0];
  // The device address of the library's own array is looked up by the first call of either entry point on a device,
  // so that a caller who records the allocation-free one into a graph only has to have run decode attention once,
  // eagerly, on that device before: the lookup itself is then never made while a stream is being captured.
  float* ownScratch = nullptr;
  AMD_TRY(decodeScratch(&ownScratch));
  if (batch == 0 || t.q.numel == 0) return diopiSuccess;
  if (a.generic) {
    AMD_CHECK(batch <= 65535, "token attention: batch %ld exceeds the grid limits", (long)batch);
    dim3 grid(a.heads, 1, (unsigned)batch);
#define GENERIC_CALL(T) hipLaunchKernelGGL((decodeGenericKernel<T>), grid, dim3(256), 0, stream, a, out.ptr<T>())
    TA_GENERIC_DISPATCH(t.q.dtype, GENERIC_CALL);
#undef GENERIC_CALL
    AMD_LAUNCH_CHECK();
    return diopiSuccess;
  }
  return streamChunks<kTaFused>(ctx, stream, a, t.q.dtype, t.q.shape[2] * t.q.itemsize, batch, maxInputLen, out.data, true,
                                staticScratch, ownScratch);
}

extern "C" __attribute__((visibility("default"))) diopiError_t diopiTokenDecodeAttentionInference(
    diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t qH, diopiConstTensorHandle_t kH,
    diopiConstTensorHandle_t vH, diopiConstTensorHandle_t locH, diopiConstTensorHandle_t startH,
    diopiConstTensorHandle_t lenH, int maxInputLen) {
  return decodeAttention(ctx, outH, qH, kH, vH, locH, startH, lenH, maxInputLen, false);
}

// The same kernels with the split-KV partial results in the library's own device array: no hipMalloc, no hipFree, no
// workspace request. Calls that overlap on one device (two streams, two threads) share the array and race.
extern "C" __attribute__((visibility("default"))) diopiError_t diopiTokenDecodeAttentionInferenceNoAlloc(
    diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t qH, diopiConstTensorHandle_t kH,
    diopiConstTensorHandle_t vH, diopiConstTensorHandle_t locH, diopiConstTensorHandle_t startH,
    diopiConstTensorHandle_t lenH, int maxInputLen) {
  return decodeAttention(ctx, outH, qH, kH, vH, locH, startH, lenH, maxInputLen, true);
}

extern "C" __attribute__((visibility("default"))) diopiError_t diopiTokenAttentionInference(
    diopiContextHandle_t ctx, diopiTensorHandle_t attH, diopiConstTensorHandle_t qH, diopiConstTensorHandle_t kH,
    diopiConstTensorHandle_t locH, diopiConstTensorHandle_t startH, diopiConstTensorHandle_t lenH, int maxInputLen) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TaViews t;
  TensorView att;
  AMD_TRY(getView(attH, &att, "attention_out"));
  AMD_TRY(getView(qH, &t.q, "q"));
  AMD_TRY(getView(kH, &t.k, "k"));
  AMD_TRY(getView(locH, &t.loc, "b_loc"));
  AMD_TRY(getView(startH, &t.start, "b_start_loc"));
  AMD_TRY(getView(lenH, &t.len, "b_seq_len"));
  TaArgs a;
  AMD_TRY(fillArgs(t, true, false, maxInputLen, &a));
  AMD_CHECK(att.defined() && att.ndim == 2 && att.shape[0] == a.heads && (att.stride[1] == 1 || att.shape[1] == 1),
            "token attention: attention_out must be [heads, total_tokens] with a contiguous last dim");
  AMD_CHECK(att.dtype == diopi_dtype_float32 || att.dtype == t.q.dtype,
            "token attention: attention_out dtype must be float32 or the q dtype");
  const int64_t batch = t.q.shape[0];
  if (batch == 0 || maxInputLen == 0) return diopiSuccess;
  int nchunk = (int)ceilDiv(maxInputLen, a.chunk);
  AMD_CHECK(batch <= 65535 && nchunk <= 65535, "token attention: grid limits exceeded");
  dim3 grid(a.heads, nchunk, (unsigned)batch), block(256);
  const int64_t bytes = t.q.shape[2] * t.q.itemsize;
  if (a.generic) {
    if (att.dtype == diopi_dtype_float32) {
#define GENERIC_CALL(T) \
  hipLaunchKernelGGL((tokenLogitsGenericKernel<T, float>), grid, block, 0, stream, a, att.ptr<float>(), att.stride[0])
      TA_GENERIC_DISPATCH(t.q.dtype, GENERIC_CALL);
#undef GENERIC_CALL
    } else {
#define GENERIC_CALL(T) hipLaunchKernelGGL((tokenLogitsGenericKernel<T, T>), grid, block, 0, stream, a, att.ptr<T>(), att.stride[0])
      TA_GENERIC_DISPATCH(t.q.dtype, GENERIC_CALL);
#undef GENERIC_CALL
    }
    AMD_LAUNCH_CHECK();
    return diopiSuccess;
  }
  a.logits = att.data, a.logitsHeadStride = att.stride[0];
  return streamChunks<kTaLogitsOut>(ctx, stream, a, t.q.dtype, bytes, batch, maxInputLen, nullptr,
                                    att.dtype == diopi_dtype_float32, false, nullptr);
}

extern "C" __attribute__((visibility("default"))) diopiError_t diopiTokenSoftmaxReduceVInference(
    diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t logicsH, diopiConstTensorHandle_t vH,
    diopiConstTensorHandle_t locH, diopiConstTensorHandle_t startH, diopiConstTensorHandle_t lenH, int maxInputLen,
    int otherKvIndex) {
  (void)otherKvIndex;
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TaViews t;
  TensorView out, lg;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(logicsH, &lg, "logics"));
  AMD_TRY(getView(vH, &t.v, "v"));
  AMD_TRY(getView(locH, &t.loc, "b_loc"));
  AMD_TRY(getView(startH, &t.start, "b_start_loc"));
  AMD_TRY(getView(lenH, &t.len, "b_seq_len"));
  AMD_CHECK(out.defined() && out.ndim == 3 && out.isContiguous(), "token attention: out must be a dense [batch, heads, head_dim]");
  t.q = out;  // out has q's geometry
  TaArgs a;
  AMD_TRY(fillArgs(t, false, true, maxInputLen, &a));
  AMD_CHECK(lg.defined() && lg.ndim == 2 && lg.shape[0] == a.heads && (lg.stride[1] == 1 || lg.shape[1] == 1),
            "token attention: logics must be [heads, total_tokens] with a contiguous last dim");
  AMD_CHECK(lg.dtype == diopi_dtype_float32 || lg.dtype == out.dtype, "token attention: logics dtype must be float32 or out's");
  const int64_t batch = out.shape[0];
  if (batch == 0 || out.numel == 0) return diopiSuccess;
  AMD_CHECK(batch <= 65535, "token attention: grid limits exceeded");
  dim3 grid(a.heads, 1, (unsigned)batch), block(256);
  const int64_t bytes = out.shape[2] * out.itemsize;
  if (a.generic) {
    if (lg.dtype == diopi_dtype_float32) {
#define GENERIC_CALL(T) \
  hipLaunchKernelGGL((softmaxReduceVGenericKernel<T, float>), grid, block, 0, stream, a, out.ptr<T>(), lg.ptr<float>(), lg.stride[0])
      TA_GENERIC_DISPATCH(out.dtype, GENERIC_CALL);
#undef GENERIC_CALL
    } else {
#define GENERIC_CALL(T) \
  hipLaunchKernelGGL((softmaxReduceVGenericKernel<T, T>), grid, block, 0, stream, a, out.ptr<T>(), lg.ptr<T>(), lg.stride[0])
      TA_GENERIC_DISPATCH(out.dtype, GENERIC_CALL);
#undef GENERIC_CALL
    }
    AMD_LAUNCH_CHECK();
    return diopiSuccess;
  }
  a.logits = lg.data, a.logitsHeadStride = lg.stride[0];
  return streamChunks<kTaReduceV>(ctx, stream, a, out.dtype, bytes, batch, maxInputLen, out.data,
                                  lg.dtype == diopi_dtype_float32, false, nullptr);
}
