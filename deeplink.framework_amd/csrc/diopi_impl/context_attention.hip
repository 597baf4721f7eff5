// Prefill ("context") causal attention over packed sequences for gfx950.
//
//   q [tokens, heads, d], k/v [tokens, kv_heads, d]; sequence b = rows
//   [b_start_loc[b], b_start_loc[b] + b_seq_len[b]);
//   out = softmax(q k^T / sqrt(d) + causal mask) v, scores and softmax in fp32
//   (dicp/dicp/vendor/AscendGraph/ext_ops.py:62-87).
//
// MFMA kernel (bf16 / fp16, d = 64 or 128): a workgroup of 4 waves owns 128 queries of one
// (sequence, head); each wave owns 32 of them and walks the keys in tiles of 64.
//   * S^T = K . Q^T is computed instead of S: the 32x32 accumulator then holds, in every
//     lane, 16 scores of ONE query (its column), so the online-softmax row statistics are
//     an in-lane reduction plus a single xor-32 shuffle, and the O^T accumulators of the
//     lane belong to that same query: rescaling needs no cross-lane traffic at all.
//   * The accumulator registers of S^T, converted to bf16, are already a valid B operand
//     (P^T) for O^T += V^T . P^T: consecutive groups of 8 accumulator registers are the 8
//     K-slots of a lane, for a fixed permutation of the 16 keys of the step. The A operand
//     (V^T) comes from V kept row-major [keys][d] in LDS through the transposing LDS read
//     (ds_read_b64_tr_b16): the addresses the lanes supply pick that same permutation, two
//     8-byte reads per operand and no transposition work anywhere.
//   * K and V tiles go from memory straight into LDS (buffer_load ... lds): no staging registers, no
//     LDS stores. Rows are XOR-swizzled per 16-byte chunk on the global side of the copy: K for
//     conflict-free ds_read_b128, V so that the 16 row pieces one transposing read touches spread
//     evenly over the banks.
//   * two workgroups per CU (<= 256 registers per lane) so one wave's softmax VALU work overlaps
//     another's MFMAs; exp2 is the bare hardware instruction fed by one FMA; the O^T rescale is
//     skipped while the running max does not move;
//   * two LDS stages; the copy of tile t + 1 is issued when tile t starts and waited for when it ends
//     (buffer descriptors: no per-row address arithmetic, rows past the sequence read as zero), one
//     barrier per tile;
//   * causal work grows with the query block index: a workgroup processes the heaviest remaining
//     block and then the lightest, so all workgroups stream the same number of key tiles; the
//     one-dimensional grid is decoded so the workgroups of a head share one XCD (one L2).
//   * the epilogue transposes O^T through LDS so global stores are 16-byte and coalesced.
//
// Scalar kernel: any dtype / head_dim, one workgroup per (query, head); correctness path
// for fp32 and odd head sizes.
#include <algorithm>

#include "common.hpp"

namespace amd {

constexpr float kLog2eCA = 1.4426950408889634f;

__device__ __forceinline__ int64_t ldIdxCA(const void* p, int64_t i, bool is64) {
  return is64 ? reinterpret_cast<const int64_t*>(p)[i] : static_cast<int64_t>(reinterpret_cast<const int32_t*>(p)[i]);
}

struct CaArgs {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  const void* bStart;
  const void* bLen;
  bool start64, len64;
  int64_t qTok, qHead, kTok, kHead, vTok, vHead, oTok, oHead;  // element strides
  int heads, kvHeads, d;
  float scale;  // 1/sqrt(d)
};

template <typename T>
struct CaMfma;
template <>
struct CaMfma<bf16_t> {
  typedef bf16x8 Frag;
  typedef bf16x4 Half;
  static __device__ __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct CaMfma<half_t> {
  typedef f16x8 Frag;
  typedef f16x4 Half;
  static __device__ __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// XOR applied to the 16-byte chunk index of K row `key` in LDS; the patterns are the ones that
// measure conflict-free for ds_read_b128 with 32 consecutive rows per half-wave: 256-byte rows
// (d = 128; 512-byte rows alias the banks the same way) need key & 15, 128-byte rows (d = 64) need (key >> 1) & 7.
template <int D>
__device__ __forceinline__ int kSwizzle(int key) {
  return D >= 128 ? (key & 15) : ((key >> 1) & 7);
}

// XOR applied to the 16-byte chunk index of V row `key` in LDS (a multiple of 4, so the 32 bytes a 16-lane
// group takes from one row stay together). A transposing read is served half a wave at a time: 4
// consecutive keys x 2 pieces of 32 bytes, which these patterns put on 8 different 32-byte bank groups.
template <int D>
__device__ __forceinline__ int vSwizzle(int key) {
  return D >= 128 ? 4 * (key & 3) : 4 * ((key >> 1) & 1);
}

constexpr int kCaBQ = 128, kCaBKV = 64;
// A new row maximum replaces the running one only when it exceeds it by more than this (log2 domain). Until then the
// probabilities of a tile are taken against the stale maximum (at most 2^8: harmless in the fp32 sums and in bf16 / fp16
// operands) and the softmax is the same; the rescale of O^T, which otherwise runs in most tiles (one of a wave's 32
// queries nearly always sees a new maximum), becomes rare.
constexpr float kCaRescaleStep = 8.0f;

// One 128-query block of one (sequence, head): the whole flash-attention pass over its key tiles.
// D is the head size the tiles are laid out for (64, 128 or 256); with PART the tensors' own head size a.d is any
// multiple of 8 below D: the pieces of a row at or past a.d are zeros in the Q fragments and in the K and V tiles (they add
// nothing to a score and produce output columns that are not stored).
template <typename T, int D, bool PART>
__device__ __forceinline__ void contextAttnBlock(const CaArgs& a, const int qb, const int h, const int b) {
  using Frag = typename CaMfma<T>::Frag;
  using Half = typename CaMfma<T>::Half;
  constexpr int KS = D / 16;        // MFMA k-steps over the head dim
  constexpr int DT = D / 32;        // 32-row tiles of O^T
  constexpr int CPR = D / 8;        // 16-byte chunks per row
  constexpr int RPL = 64 / CPR;     // rows one wave-wide copy instruction covers (1 KiB)
  constexpr int NLD = kCaBKV / RPL / 4;     // copy instructions per wave, per matrix, per tile
  constexpr int STAGE = kCaBKV * D;         // elements
  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* sK = reinterpret_cast<T*>(smem);   // [2][64][D] swizzled
  T* sV = sK + 2 * STAGE;               // [2][64][D] swizzled

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l31 = lane & 31, half = lane >> 5;
  const int64_t start = ldIdxCA(a.bStart, b, a.start64);
  const int len = (int)ldIdxCA(a.bLen, b, a.len64);
  const int q0 = qb * kCaBQ;
  if (q0 >= len) return;
  const int kvh = h / (a.heads / a.kvHeads);
  const T* qg = reinterpret_cast<const T*>(a.q) + start * a.qTok + (int64_t)h * a.qHead;
  const T* kg = reinterpret_cast<const T*>(a.k) + start * a.kTok + (int64_t)kvh * a.kHead;
  const T* vg = reinterpret_cast<const T*>(a.v) + start * a.vTok + (int64_t)kvh * a.vHead;

  const int qi = q0 + wave * 32 + l31;      // this lane's query (column of S^T)
  const int qiC = min(qi, len - 1);          // rows past the sequence compute on the last row, never stored
  const int dReal = PART ? a.d : D;  // (PART: a variant of its own, so that whole rows pay nothing for the tests below)
  Frag qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (ks * 16 + half * 8 < dReal) {
      qf[ks] = *reinterpret_cast<const Frag*>(qg + (int64_t)qiC * a.qTok + ks * 16 + half * 8);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[ks][e] = static_cast<T>(0.f);
    }
  }

  const int ntiles = (min(len, q0 + kCaBQ) + kCaBKV - 1) / kCaBKV;
  const int waveMaxQ = min(q0 + wave * 32 + 31, len - 1);

  // ---- tile copies. K and V rows come through buffer descriptors that end at the sequence's last
  // row: a lane's offset is computed once (32 bits), the tile advances a scalar offset, and rows past
  // the sequence read as zeros without any clamping arithmetic. Copy instruction i of this wave fills
  // the 1 KiB block (i * 4 + wave) of a stage: lane l owns physical slot (row l / CPR, chunk l % CPR) and
  // fetches the logical chunk the swizzle puts there.
  int kVoff[NLD], vVoff[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int key = (i * 4 + wave) * RPL + lane / CPR, pc = lane % CPR;
    const int kc = (pc ^ kSwizzle<D>(key)) << 3, vc = (pc ^ vSwizzle<D>(key)) << 3;  // first element of the piece
    constexpr int kPastEnd = (int)0x80000000u;  // beyond every descriptor: the copy writes zeros
    kVoff[i] = kc < dReal ? (key * (int)a.kTok + kc) * (int)sizeof(T) : kPastEnd;
    vVoff[i] = vc < dReal ? (key * (int)a.vTok + vc) * (int)sizeof(T) : kPastEnd;
  }
  auto descriptor = [](const T* base, int64_t bytes) {
    const uint64_t p = reinterpret_cast<uint64_t>(base);
    u32x4 d = {(uint32_t)p, (uint32_t)(p >> 32) & 0xffffu, (uint32_t)bytes, 0x00020000u};
    return d;
  };
  const u32x4 rsK = descriptor(kg, ((int64_t)(len - 1) * a.kTok + dReal) * sizeof(T));
  const u32x4 rsV = descriptor(vg, ((int64_t)(len - 1) * a.vTok + dReal) * sizeof(T));
  const unsigned ldsK = (unsigned)(uintptr_t)sK, ldsV = (unsigned)(uintptr_t)sV;

  auto copyK = [&](int t, int stage) {
    const int kS = t * kCaBKV * (int)a.kTok * (int)sizeof(T);
    const unsigned to = ldsK + (unsigned)(stage * STAGE * sizeof(T)) + (unsigned)wave * 1024u;
#pragma unroll
    for (int i = 0; i < NLD; ++i) loadToLds16(rsK, kVoff[i], kS, to + i * 4096u);
  };
  auto copyV = [&](int t, int stage) {
    const int vS = t * kCaBKV * (int)a.vTok * (int)sizeof(T);
    const unsigned to = ldsV + (unsigned)(stage * STAGE * sizeof(T)) + (unsigned)wave * 1024u;
#pragma unroll
    for (int i = 0; i < NLD; ++i) loadToLds16(rsV, vVoff[i], vS, to + i * 4096u);
  };

  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;
  float m = -INFINITY, l = 0.f;
  const float scale2 = a.scale * kLog2eCA;

  // Everything this wave has in flight (its share of the copies, its LDS reads) is done, then the
  // workgroup meets: past the barrier the tiles those copies fill are complete in LDS.
  auto tileBarrier = []() {
    __builtin_amdgcn_s_waitcnt(0x0070);
    __builtin_amdgcn_s_barrier();
  };
  // K fragment i of a tile: key half i & 1 (32 keys), head-dim step i >> 1. A ring of them runs kKAhead
  // MFMAs ahead of the score MFMAs, and the first kKAhead of the NEXT tile are read at the end of the
  // P.V loop, so no score MFMA waits for LDS.
  // Addresses: the XOR swizzles touch only bits that the rest of a fragment's address leaves zero, so the LDS byte
  // address is (lane constant + stage) ^ (step constant) plus an immediate: one register per matrix, made opaque per
  // tile so that the derived addresses are recomputed (one XOR each) rather than kept or re-derived with several adds.
  constexpr int NS = 2 * KS, kKAhead = 4, ROWB = D * (int)sizeof(T);
  constexpr unsigned kStageBytes = STAGE * sizeof(T);
  Frag kfr[kKAhead + 1];
  const int kswz = kSwizzle<D>(l31);
  const unsigned kLane = (unsigned)(l31 * ROWB + ((half ^ (kswz & 1)) << 4) + ((kswz >> 1) << 5));
  typedef __attribute__((address_space(3))) const Frag* LdsFrag;
  auto kfragAt = [&](unsigned kBase, int i) {  // kBase = kLane + LDS byte address of the stage
    return *(LdsFrag)(uintptr_t)((kBase ^ (unsigned)((i >> 1) << 5)) + (unsigned)((i & 1) * 32 * ROWB));
  };
  auto opaque = [](unsigned x) {
    asm volatile("" : "+v"(x));
    return x;
  };
  const unsigned ldsK0 = (unsigned)(uintptr_t)sK, ldsV0 = (unsigned)(uintptr_t)sV;
  // The barrier of tile t sits between its softmax and its P.V: it publishes K of tile t + 1 and V of tile t,
  // and it says that every wave is done with K of tile t and V of tile t - 1, whose stages the copies
  // issued right after it (K of t + 2, V of t + 1) overwrite. Every copy has a whole tile to land.
  copyK(0, 0);
  copyV(0, 0);
  tileBarrier();
  if (ntiles > 1) copyK(1, 1);
#pragma unroll
  for (int i = 0; i < kKAhead; ++i) kfr[i] = kfragAt(kLane + ldsK0, i);

  for (int t = 0; t < ntiles; ++t) {
    const int cur = t & 1;
    const int k0 = t * kCaBKV;
    const bool live = k0 <= waveMaxQ;  // wave-uniform; once false it stays false
    const unsigned kCur = opaque(kLane + ldsK0 + cur * kStageBytes), kOther = opaque(kLane + ldsK0 + (cur ^ 1) * kStageBytes);
    f32x16 s[2];
    if (live) {
#pragma unroll
      for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[kt2][r] = 0.f;
      // A wave in an MFMA phase outranks one in its softmax when both want to issue: the matrix pipe then never
      // waits behind the other wave's exp2 and conversions (measured: 169 -> 161 us on 4 x 2048 x 32 x 128).
      __builtin_amdgcn_s_setprio(1);
      // the two 32-key halves are independent accumulation chains: alternate them so that no MFMA
      // waits for the one issued just before it
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        if (i + kKAhead < NS) kfr[(i + kKAhead) % (kKAhead + 1)] = kfragAt(kCur, i + kKAhead);
        s[i & 1] = CaMfma<T>::run(kfr[i % (kKAhead + 1)], qf[i >> 1], s[i & 1]);
        __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_s_setprio(0);
      // ---- online softmax for this lane's query over the 64 keys of the tile
      // (m and mn are kept in the scaled log2 domain: score * scale * log2 e)
      const bool needMask = (k0 + kCaBKV - 1 > q0 + wave * 32) || (k0 + kCaBKV > len);
      if (needMask) {  // wave-uniform: only the diagonal and the last tile pay for masking
#pragma unroll
        for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            int kj = k0 + kt2 * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
            if (kj > qiC || kj >= len) s[kt2][r] = -INFINITY;
          }
      }
      float mt = -INFINITY;
#pragma unroll
      for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
        for (int r = 0; r < 16; ++r) mt = fmaxf(mt, s[kt2][r]);
      {  // the other half-wave holds the other 16 scores of the query: one lane swap, no trip through LDS
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mt), __float_as_uint(mt), false, false);
        mt = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1])) * scale2;  // scale2 > 0, so the max commutes with the scaling
      }
      // key 0 is visible to every query, so mn is finite from tile 0 on (m = -inf there: the difference is +inf)
      const float mn = mt - m > kCaRescaleStep ? mt : m;
#pragma unroll
      for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          // one fused multiply-add and one hardware exp2 per score; masked scores give exp2(-inf) = 0
          s[kt2][r] = __builtin_amdgcn_exp2f(fmaf(s[kt2][r], scale2, -mn));
        }
      // the running max rarely moves after the first tiles: rescale only when some lane needs it
      if (__builtin_amdgcn_ballot_w64(mn > m) != 0) {
        const float corr = __builtin_amdgcn_exp2f(m - mn);
        l *= corr;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[dt][r] *= corr;
        m = mn;
      }
    }
    tileBarrier();
    if (t + 2 < ntiles) copyK(t + 2, cur);
    if (t + 1 < ntiles) copyV(t + 1, cur ^ 1);
    if (live) {
      __builtin_amdgcn_s_setprio(2);
      // ---- O^T += V^T . P^T: 4 key groups of 16 x DT row tiles. The V^T fragment of MFMA i + kVAhead is
      // read while MFMA i issues, and a scheduling fence after every MFMA keeps that order, so the LDS
      // latency of a fragment is covered by the MFMAs in front of it.
      {
        constexpr int NPV = 4 * DT, kVAhead = 3;
        // Transposing read: the 16 lanes of a group each supply the address of 4 consecutive d of one key,
        // source lane j -> (key j >> 2, d 4 * (j & 3)), and lane i of the group receives d = i of those 4
        // keys. Group G serves the half-wave G >> 1 and the d range 16 * (G & 1); read r of the two takes
        // keys 8 r + 4 half + 0..3 of the step: the order the P^T operand holds them in.
        const int trKey = half * 4 + ((lane & 15) >> 2);
        const int trChunk = ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1), trIn = (lane & 1) * 4;
        const int vsw = D >= 128 ? (trKey & 3) : ((trKey >> 1) & 1);  // vSwizzle<D>(key) / 4: the low bits of the d tile
        const unsigned vCur = opaque((unsigned)(trKey * ROWB + (trChunk << 4) + trIn * 2 + (vsw << 6)) + ldsV0 + cur * kStageBytes);
        typedef __attribute__((address_space(3))) s16x4* LdsTr;
        auto vfrag = [&](int i) {
          const int g = i / DT, dt = i % DT;  // key group (kt2 * 2 + t2), d tile
          Half part[2];
#pragma unroll
          for (int r = 0; r < 2; ++r)
            part[r] = __builtin_bit_cast(Half, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                                   (LdsTr)(uintptr_t)((vCur ^ (unsigned)(dt << 6)) + (unsigned)((g * 16 + r * 8) * ROWB))));
          Frag vf;
          vf[0] = part[0][0], vf[1] = part[0][1], vf[2] = part[0][2], vf[3] = part[0][3];
          vf[4] = part[1][0], vf[5] = part[1][1], vf[6] = part[1][2], vf[7] = part[1][3];
          return vf;
        };
        Frag vfr[kVAhead + 1];
#pragma unroll
        for (int i = 0; i < kVAhead; ++i) vfr[i] = vfrag(i);
        // The softmax denominator comes off the matrix pipe too: a V^T row of ones makes every
        // accumulator of lsum the sum of this query's (rounded) probabilities over the 16 keys of a
        // group, which takes 32 additions per tile off the VALU, the unit this kernel is bound by.
        Frag pf, ones;
#pragma unroll
        for (int j = 0; j < 8; ++j) ones[j] = static_cast<T>(1.0f);
        f32x16 lsum;
#pragma unroll
        for (int r = 0; r < 16; ++r) lsum[r] = 0.f;
#pragma unroll
        for (int i = 0; i < NPV; ++i) {
          const int g = i / DT, dt = i % DT;
          if (dt == 0) {
#pragma unroll
            for (int j = 0; j < 8; ++j) pf[j] = static_cast<T>(s[g >> 1][8 * (g & 1) + j]);
            lsum = CaMfma<T>::run(ones, pf, lsum);
          }
          if (i + kVAhead < NPV) vfr[(i + kVAhead) % (kVAhead + 1)] = vfrag(i + kVAhead);
          // the next tile's first K fragments (after the last tile: a harmless read of the other stage)
          if (i >= NPV - kKAhead) kfr[i - (NPV - kKAhead)] = kfragAt(kOther, i - (NPV - kKAhead));
          o[dt] = CaMfma<T>::run(vfr[i % (kVAhead + 1)], pf, o[dt]);
          __builtin_amdgcn_sched_barrier(0);
        }
        l += lsum[0];
      }
    }
  }
  __builtin_amdgcn_s_setprio(0);
  __syncthreads();  // the output staging below aliases the stages other waves may still be reading

  // ---- epilogue: O^T (lane = query) -> LDS [query][d] -> coalesced 16-byte stores
  constexpr int OS = D + 8;  // padded row, elements
  T* sO = reinterpret_cast<T*>(smem) + wave * 32 * OS;
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      Half p;
#pragma unroll
      for (int e = 0; e < 4; ++e) p[e] = static_cast<T>(o[dt][g * 4 + e] * inv);
      *reinterpret_cast<Half*>(sO + l31 * OS + dt * 32 + g * 8 + half * 4) = p;
    }
  __syncthreads();
  T* og = reinterpret_cast<T*>(a.out) + start * a.oTok + (int64_t)h * a.oHead;
#pragma unroll
  for (int i = 0; i < 32 * CPR / 64; ++i) {
    int chunk = lane + 64 * i;
    int row = chunk / CPR, c = chunk % CPR;
    int qrow = q0 + wave * 32 + row;
    if (qrow < len && c * 8 < dReal) *reinterpret_cast<Frag*>(og + (int64_t)qrow * a.oTok + c * 8) = *reinterpret_cast<const Frag*>(sO + row * OS + c * 8);
  }
}

// Causal work grows linearly with the query block index, so a workgroup takes the heaviest remaining
// block and then the lightest one: every workgroup streams the same number of key tiles, the grid is
// an exact multiple of what the chip holds at typical shapes, and the blocks of one head still run
// side by side and share their K/V tiles in L2.
//
// Workgroups are dealt to the 8 XCDs round-robin by their linear id, and each XCD has its own L2. The
// grid is therefore one-dimensional and decoded so that all workgroups of one (sequence, head), and
// of neighbouring heads (which share K/V under grouped-query attention), land on the same XCD next to
// each other in time: a K/V tile is fetched from HBM once and then served from that L2.
template <typename T, int D, bool PART>
__global__ __launch_bounds__(256, D > 128 ? 1 : 2) void contextAttnMfmaKernel(CaArgs a, int numQBlocks, int numSeq) {
  const int pairs = (numQBlocks + 1) / 2, hb = a.heads * numSeq;
  const int flat = (int)blockIdx.x;
  int h, b, pair;
  if ((a.heads & 7) == 0) {
    // every sequence's heads are dealt over the 8 XCDs, a contiguous eighth of them each, so that a batch of unequal
    // sequences loads the XCDs alike (with whole sequences per XCD, one long sequence among short ones kept a single
    // XCD busy: 4096 + 12 x 340 tokens 843 us against 146 for 4 x 2048, which is the same work)
    const int xcd = flat & 7, idx = flat >> 3, perXcd = a.heads >> 3;
    const int hs = idx / pairs;
    pair = idx - hs * pairs;
    b = hs / perXcd;
    h = xcd * perXcd + (hs - b * perXcd);
  } else if ((hb & 7) == 0) {
    const int xcd = flat & 7, idx = flat >> 3;
    const int headSeq = xcd * (hb >> 3) + idx / pairs;
    pair = idx % pairs;
    h = headSeq % a.heads, b = headSeq / a.heads;
  } else {
    const int headSeq = flat / pairs;
    pair = flat % pairs;
    h = headSeq % a.heads, b = headSeq / a.heads;
  }
  const int heavy = numQBlocks - 1 - pair, light = pair;
  for (int pass = 0; pass < 2; ++pass) {
    if (pass == 1) {
      if (light == heavy) break;
      __syncthreads();  // the first block's output staging aliases the K/V stages the second one fills
    }
    contextAttnBlock<T, D, PART>(a, pass == 0 ? heavy : light, h, b);
  }
}

// The same blocks one per workgroup, the heaviest first, for launches whose pairs would leave CUs without work or with
// twice their share (a single prompt of a few hundred tokens; a few sequences whose pairs are a little more than one
// per CU). The dispatcher hands a free CU the heaviest block left, so the load evens out the way a longest-job-first
// list does, and a short prompt has twice the workgroups. The blocks of one head are no longer neighbours in time
// and share less in L2, which is why launches whose pairs already fill the chip evenly keep the paired form. Measured
// (us, 32 heads x 128, bf16, pairs -> this): 1 x 256 tokens 14.6 -> 9.1, 1 x 512 19.1 -> 13.6, 1 x 1024 28.0 -> 22.8,
// 3 x 700 30.9 -> 24.4, 1 x 3000 89.7 -> 84.9; against it: 1 x 2048 46.8 -> 51.0, 32 x 512 134 -> 155, 8 x 1000 88 -> 103.
template <typename T, int D, bool PART>
__global__ __launch_bounds__(256, D > 128 ? 1 : 2) void contextAttnSingleBlockKernel(CaArgs a, int numQBlocks, int numSeq) {
  const int flat = (int)blockIdx.x;
  int rank, b, h;
  if ((a.heads & 7) == 0) {  // a contiguous eighth of every sequence's heads per XCD, as in the paired form
    const int xcd = flat & 7, idx = flat >> 3, perXcd = a.heads >> 3;
    const int hsPerXcd = perXcd * numSeq;
    rank = idx / hsPerXcd;
    const int hs = idx - rank * hsPerXcd;
    b = hs / perXcd, h = xcd * perXcd + (hs - b * perXcd);
  } else {
    const int hb = a.heads * numSeq;
    rank = flat / hb;
    const int hs = flat - rank * hb;
    b = hs / a.heads, h = hs - b * a.heads;
  }
  contextAttnBlock<T, D, PART>(a, numQBlocks - 1 - rank, h, b);
}

// One workgroup per (query token, head): scores to LDS, softmax, then P.V with lanes over d.
template <typename T>
__global__ __launch_bounds__(256) void contextAttnScalarKernel(CaArgs a, int maxLen) {
  extern __shared__ float sc[];  // maxLen scores + 8 reduction slots
  float* red = sc + maxLen;
  const int qi = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int64_t start = ldIdxCA(a.bStart, b, a.start64);
  const int len = (int)ldIdxCA(a.bLen, b, a.len64);
  if (qi >= len) return;
  const int kvh = h / (a.heads / a.kvHeads);
  const T* q = reinterpret_cast<const T*>(a.q) + (start + qi) * a.qTok + (int64_t)h * a.qHead;
  const T* kg = reinterpret_cast<const T*>(a.k) + start * a.kTok + (int64_t)kvh * a.kHead;
  const T* vg = reinterpret_cast<const T*>(a.v) + start * a.vTok + (int64_t)kvh * a.vHead;
  const int n = qi + 1;  // causal: keys 0..qi
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float mx = -INFINITY;
  for (int j = threadIdx.x; j < n; j += 256) {
    const T* kr = kg + (int64_t)j * a.kTok;
    float d = 0.f;
    for (int e = 0; e < a.d; ++e) d += static_cast<float>(q[e]) * static_cast<float>(kr[e]);
    d *= a.scale;
    sc[j] = d;
    mx = fmaxf(mx, d);
  }
  mx = waveMax(mx);
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float sum = 0.f;
  for (int j = threadIdx.x; j < n; j += 256) {
    float p = expf(sc[j] - mx);
    sc[j] = p;
    sum += p;
  }
  sum = waveSum(sum);
  if (lane == 0) red[4 + wave] = sum;
  __syncthreads();
  const float inv = 1.f / (red[4] + red[5] + red[6] + red[7]);
  T* og = reinterpret_cast<T*>(a.out) + (start + qi) * a.oTok + (int64_t)h * a.oHead;
  for (int e = threadIdx.x; e < a.d; e += 256) {
    float acc = 0.f;
    for (int j = 0; j < n; ++j) acc += sc[j] * static_cast<float>(vg[(int64_t)j * a.vTok + e]);
    og[e] = static_cast<T>(acc * inv);
  }
}

template <typename T, int D, bool PART>
static diopiError_t launchCaMfmaAs(hipStream_t stream, const CaArgs& a, int maxLen, int64_t batch) {
  constexpr size_t lds = 2 * (size_t)(2 * kCaBKV * D) * sizeof(T);
  static_assert(lds >= 4 * 32 * (D + 8) * sizeof(T), "epilogue staging must fit in the tile buffers");
  AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&contextAttnMfmaKernel<T, D, PART>), (int)lds));
  const int numQBlocks = (int)ceilDiv(maxLen, kCaBQ);
  const int64_t blocks = (int64_t)((numQBlocks + 1) / 2) * a.heads * batch;
  AMD_CHECK(blocks < ((int64_t)1 << 31), "context attention: grid limits exceeded");
  // Busiest CU's load in units of one key-block column of a query block (block i costs i + 1): pairs of numQBlocks + 1
  // dealt round-robin, against single blocks handed out heaviest first (the mean load, or the heaviest block alone).
  const int64_t cus = computeUnits(), hb = (int64_t)a.heads * batch;
  const int64_t pairedLoad = ceilDiv(blocks, cus) * (numQBlocks + 1);
  const int64_t singleLoad = std::max<int64_t>(ceilDiv(hb * numQBlocks * (numQBlocks + 1) / 2, cus), numQBlocks);
  if (numQBlocks > 1 && singleLoad * 11 < pairedLoad * 10 && hb * numQBlocks < ((int64_t)1 << 31)) {
    AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&contextAttnSingleBlockKernel<T, D, PART>), (int)lds));
    hipLaunchKernelGGL((contextAttnSingleBlockKernel<T, D, PART>), dim3((unsigned)(hb * numQBlocks)), dim3(256), lds, stream, a, numQBlocks,
                       (int)batch);
    AMD_LAUNCH_CHECK();
    return diopiSuccess;
  }
  hipLaunchKernelGGL((contextAttnMfmaKernel<T, D, PART>), dim3((unsigned)blocks), dim3(256), lds, stream, a, numQBlocks, (int)batch);
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

template <typename T, int D>
static diopiError_t launchCaMfma(hipStream_t stream, const CaArgs& a, int maxLen, int64_t batch) {
  return a.d == D ? launchCaMfmaAs<T, D, false>(stream, a, maxLen, batch) : launchCaMfmaAs<T, D, true>(stream, a, maxLen, batch);
}

}  // namespace amd

using namespace amd;

extern "C" __attribute__((visibility("default"))) diopiError_t diopiContextAttentionInference(
    diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t qH, diopiConstTensorHandle_t kH,
    diopiConstTensorHandle_t vH, diopiConstTensorHandle_t startH, diopiConstTensorHandle_t lenH, int maxInputLen) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, q, k, v, st, ln;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(qH, &q, "q"));
  AMD_TRY(getView(kH, &k, "k"));
  AMD_TRY(getView(vH, &v, "v"));
  AMD_TRY(getView(startH, &st, "b_start_loc"));
  AMD_TRY(getView(lenH, &ln, "b_seq_len"));
  AMD_CHECK(out.defined() && q.defined() && k.defined() && v.defined() && st.defined() && ln.defined(),
            "context attention: null tensor");
  AMD_CHECK(q.ndim == 3 && k.ndim == 3 && v.ndim == 3 && out.ndim == 3, "context attention: q/k/v/out must be [tokens, heads, head_dim]");
  AMD_CHECK(q.dtype == k.dtype && q.dtype == v.dtype && q.dtype == out.dtype, "context attention: dtypes differ");
  for (int d = 0; d < 3; ++d) {
    AMD_CHECK(out.shape[d] == q.shape[d], "context attention: out shape differs from q at dim %d", d);
    AMD_CHECK(k.shape[d] == v.shape[d], "context attention: k and v shapes differ at dim %d", d);
  }
  AMD_CHECK(k.shape[0] == q.shape[0] && k.shape[2] == q.shape[2], "context attention: k must cover the same tokens and head_dim as q");
  AMD_CHECK(k.shape[1] > 0 && q.shape[1] % k.shape[1] == 0, "context attention: %ld heads are not a multiple of %ld kv heads",
            (long)q.shape[1], (long)k.shape[1]);
  AMD_CHECK((st.dtype == diopi_dtype_int32 || st.dtype == diopi_dtype_int64) &&
                (ln.dtype == diopi_dtype_int32 || ln.dtype == diopi_dtype_int64),
            "context attention: b_start_loc / b_seq_len must be int32 or int64");
  AMD_CHECK(st.isContiguous() && ln.isContiguous() && st.numel == ln.numel, "context attention: b_start_loc / b_seq_len must be dense and equally long");
  const int64_t batch = ln.numel;
  if (batch == 0 || q.numel == 0 || maxInputLen <= 0) return diopiSuccess;
  AMD_CHECK(batch <= 65535 && q.shape[1] <= 65535, "context attention: grid limits exceeded");
  auto unit = [](const TensorView& t) { return t.stride[2] == 1 || t.shape[2] == 1; };
  TensorView cq = q, ck = k, cv = v, co = out;
  if (!unit(q)) AMD_TRY(makeContiguous(ctx, stream, q, &cq));
  if (!unit(k)) AMD_TRY(makeContiguous(ctx, stream, k, &ck));
  if (!unit(v)) AMD_TRY(makeContiguous(ctx, stream, v, &cv));
  bool outTemp = !unit(out);
  if (outTemp) {
    diopiTensorHandle_t th;
    AMD_TRY(requireTensor(ctx, out.shape, 3, out.dtype, &th, &co));
  }
  CaArgs a;
  a.q = cq.data, a.k = ck.data, a.v = cv.data, a.out = co.data;
  a.bStart = st.data, a.bLen = ln.data;
  a.start64 = st.dtype == diopi_dtype_int64, a.len64 = ln.dtype == diopi_dtype_int64;
  a.qTok = cq.stride[0], a.qHead = cq.stride[1], a.kTok = ck.stride[0], a.kHead = ck.stride[1];
  a.vTok = cv.stride[0], a.vHead = cv.stride[1], a.oTok = co.stride[0], a.oHead = co.stride[1];
  a.heads = (int)q.shape[1], a.kvHeads = (int)k.shape[1], a.d = (int)q.shape[2];
  a.scale = 1.0f / sqrtf((float)a.d);
  const bool half = q.dtype == diopi_dtype_bfloat16 || q.dtype == diopi_dtype_float16;
  auto al = [](const TensorView& t) {
    return t.aligned16() && (t.stride[0] * t.itemsize) % 16 == 0 && (t.stride[1] * t.itemsize) % 16 == 0;
  };
  diopiError_t err;
  // the MFMA kernel addresses K and V rows of one sequence with 32-bit byte offsets
  const bool fits32 = ((int64_t)maxInputLen + kCaBKV) * std::max(a.kTok, a.vTok) * (int64_t)q.itemsize < (int64_t)1 << 31;
  // head sizes that are a multiple of 8 (whole 16-byte pieces) take the tile layout of the next of 64 / 128 / 256
  if (half && a.d % 8 == 0 && a.d <= 256 && al(cq) && al(ck) && al(cv) && al(co) && fits32) {
    if (q.dtype == diopi_dtype_bfloat16)
      err = a.d <= 64    ? launchCaMfma<bf16_t, 64>(stream, a, maxInputLen, batch)
            : a.d <= 128 ? launchCaMfma<bf16_t, 128>(stream, a, maxInputLen, batch)
                         : launchCaMfma<bf16_t, 256>(stream, a, maxInputLen, batch);
    else
      err = a.d <= 64    ? launchCaMfma<half_t, 64>(stream, a, maxInputLen, batch)
            : a.d <= 128 ? launchCaMfma<half_t, 128>(stream, a, maxInputLen, batch)
                         : launchCaMfma<half_t, 256>(stream, a, maxInputLen, batch);
  } else {
    AMD_CHECK(maxInputLen <= 12000, "context attention: the scalar path supports sequences up to 12000 tokens, got %d", maxInputLen);
    AMD_CHECK(maxInputLen <= 65535, "context attention: grid limits exceeded");
    size_t lds = ((size_t)maxInputLen + 8) * sizeof(float);
    dim3 grid((unsigned)maxInputLen, a.heads, (unsigned)batch);
    switch (q.dtype) {
      case diopi_dtype_float32: hipLaunchKernelGGL(contextAttnScalarKernel<float>, grid, dim3(256), lds, stream, a, maxInputLen); break;
      case diopi_dtype_bfloat16: hipLaunchKernelGGL(contextAttnScalarKernel<bf16_t>, grid, dim3(256), lds, stream, a, maxInputLen); break;
      case diopi_dtype_float16: hipLaunchKernelGGL(contextAttnScalarKernel<half_t>, grid, dim3(256), lds, stream, a, maxInputLen); break;
      default: setLastError("context attention: unsupported dtype %s", dtypeName(q.dtype)); return diopiErrorOccurred;
    }
    err = hipGetLastError() == hipSuccess ? diopiSuccess : diopiErrorOccurred;
    if (err != diopiSuccess) setLastError("context attention: scalar kernel launch failed");
  }
  AMD_TRY(err);
  if (outTemp) AMD_TRY(stridedCopy(stream, co, out));
  return diopiSuccess;
}
