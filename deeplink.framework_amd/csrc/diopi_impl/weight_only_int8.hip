// diopiWeightOnlyInt8Linear for gfx950: out[M,N] = x[M,K] . (W_int8[N,K] * scale[N])^T + bias.
//
// Skinny-M (decode) shape: the int8 weight matrix is streamed from HBM exactly once and is
// the only traffic of size (K*N bytes). The kernel is a GEMV-shaped MFMA kernel:
//   * a workgroup owns NTW tiles of 16 output channels; each tile has 4 waves that split K
//     four ways, so a workgroup is NTW*4 waves. NTW grows with N until the grid is about
//     one workgroup per CU: the activations are then fetched once per CU instead of once
//     per 16 channels (at M = 16 they are 3x the bytes of a 16-channel weight tile);
//   * the (up to 64) activation rows the workgroup needs are staged once in LDS by direct-to-LDS
//     loads (rows padded by 16 bytes so the 16 rows of a fragment read fall in different banks)
//     and read from there as MFMA A operands; K larger than the LDS budget is processed in chunks;
//   * v_mfma_f32_16x16x32_{bf16,f16}: the B operand is the weight tile -- lane (n = lane%16,
//     kgrp = lane/16) loads 32 consecutive int8 of row n (two 16-byte loads; the 4 kgrps of a
//     row cover 128 contiguous bytes) and converts them to bf16/fp16 in registers while
//     the next loads are in flight: the dequantisation is fused into the operand load.
//     The first weight loads of a chunk are issued before the activations are staged;
//   * fp32 accumulators of the 4 K-split waves are summed through LDS; the per-channel scale
//     is applied to the fp32 sum (identical to scaling the weights first, one rounding fewer),
//     then bias, then one conversion to the output dtype.
// Up to 64 rows of x (4 groups of 16) share every weight fragment while it is in registers; rows
// beyond 64 are handled by more workgroups along grid.y (weights are then re-read per 64 rows;
// large-M prefill should dequantise once and use the dense GEMM).
#include <algorithm>

#include "gemm.hpp"

namespace amd {

template <typename T>
struct W8Mfma;
template <>
struct W8Mfma<bf16_t> {
  typedef bf16x8 Frag;
  static __device__ __forceinline__ f32x4 run(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct W8Mfma<half_t> {
  typedef f16x8 Frag;
  static __device__ __forceinline__ f32x4 run(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

struct W8Args {
  const void* x;
  const int8_t* w;
  const void* scale;
  const void* bias;
  void* out;
  int64_t ldx, ldw, ldo;
  int M, N, K;
  int scaleDtype, biasDtype;
  int colsPerWg;  // w8LinearLdsKernel: output channels per workgroup
  // w8LinearLdsKernel with K split over gridDim.z: workgroup z multiplies stagesPerSlice stages of K from stage
  // z * stagesPerSlice on and leaves its unscaled fp32 sums in partial[z][M][N] (w8SliceReduceKernel finishes);
  // partial == nullptr: the whole K, the result scaled and stored
  float* partial = nullptr;
  int stagesPerSlice = 0;
};

// The four int8 of one dword as floats: one SDWA conversion per byte (left to itself the compiler shifts
// bytes 1 and 3 into place first, two more VALU instructions per dword in a loop that has no slack).
__device__ __forceinline__ void cvt4(uint32_t w, float& f0, float& f1, float& f2, float& f3) {
  asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(f0) : "v"(w));
  asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(f1) : "v"(w));
  asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(f2) : "v"(w));
  asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(f3) : "v"(w));
}

// converts 8 consecutive int8 (two dwords) to an MFMA operand fragment
template <typename T>
__device__ __forceinline__ typename W8Mfma<T>::Frag cvt8(uint32_t lo, uint32_t hi) {
  float f[8];
  cvt4(lo, f[0], f[1], f[2], f[3]);
  cvt4(hi, f[4], f[5], f[6], f[7]);
  typename W8Mfma<T>::Frag r;
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = static_cast<T>(f[j]);
  return r;
}

constexpr int kW8Block = 128;   // K elements one wave consumes per step (4 kgrps x 32)
// One step (two 16-byte loads per lane) is in flight ahead of the one being multiplied, no more: measured,
// a deeper queue is slower (9.7 us with four steps ahead, 10.4 with eight, 8.8 with one or two at M = 1).
constexpr int kW8KSplit = 4;    // waves per 16-channel tile = K splits
constexpr int kW8MaxTiles = 4;  // 16-channel tiles per workgroup (16 waves at most)
constexpr int kW8Pad = 8;       // elements appended to every staged activation row (16 bytes)
constexpr int kW8RowsK = 16 * 4096; // staged rows x columns per pass: 16 G x (4096 / G + 8) x 2 B <= 129 KiB

// G groups of 16 activation rows share every weight fragment while it is in registers (K is then staged in chunks
// of 4096 / G columns so that the rows fit in LDS); more than 16 G rows go to further workgroups along grid.y.
template <typename T, int NTW, int G>
__global__ __launch_bounds__(NTW * kW8KSplit * 64) void w8LinearKernel(W8Args a) {
  using Frag = typename W8Mfma<T>::Frag;
  constexpr int THREADS = NTW * kW8KSplit * 64, kW8ChunkK = kW8RowsK / (16 * G);
  extern __shared__ __attribute__((aligned(16))) char w8smem[];
  T* sx = reinterpret_cast<T*>(w8smem);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = wave / kW8KSplit, ks = wave % kW8KSplit;
  const int r16 = lane & 15, kgrp = lane >> 4;
  const int n0 = (blockIdx.x * NTW + tile) * 16, m0 = blockIdx.y * 16 * G;
  const int rows = min(16 * G, a.M - m0);
  const int8_t* wrow = a.w + (int64_t)min(n0 + r16, a.N - 1) * a.ldw + kgrp * 32;
  const uint64_t xp = reinterpret_cast<uint64_t>(reinterpret_cast<const T*>(a.x) + (int64_t)m0 * a.ldx);
  const u32x4 rsX = {(uint32_t)xp, (uint32_t)(xp >> 32) & 0xffffu, (uint32_t)(((int64_t)(rows - 1) * a.ldx + a.K) * sizeof(T)),
                     0x00020000u};
  const unsigned ldsBase = (unsigned)(size_t)(__attribute__((address_space(3))) char*)w8smem;
  // scale and bias of this lane's output channel: requested now, used after the last weight has been consumed
  const int col = n0 + r16;
  float sc = 0.f, bv = 0.f;
  if (ks == 0 && col < a.N) {
    sc = loadAs<float>(a.scale, col, a.scaleDtype);
    if (a.bias) bv = loadAs<float>(a.bias, col, a.biasDtype);
  }
  f32x4 acc[G];
#pragma unroll
  for (int gi = 0; gi < G; ++gi) acc[gi] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int kc = 0; kc < a.K; kc += kW8ChunkK) {
    const int kcLen = min(kW8ChunkK, a.K - kc);  // a multiple of 128, as K is
    const int ldx = kcLen + kW8Pad;
    // this wave's share of the chunk: a contiguous run of 128-element steps
    const int steps = kcLen / kW8Block;
    const int per = (steps + kW8KSplit - 1) / kW8KSplit;
    const int sBegin = ks * per, sEnd = min(steps, sBegin + per);
    const int8_t* wk = wrow + kc;
    // the first weight loads go out before the activations are staged
    u32x4 w0, w1;
    if (sBegin < sEnd) {  // wave-uniform
      w0 = *reinterpret_cast<const u32x4*>(wk + sBegin * kW8Block);
      w1 = *reinterpret_cast<const u32x4*>(wk + sBegin * kW8Block + 16);
    }
    if (kc > 0) __syncthreads();  // everyone is done with the previous chunk's activations
    // The activations go from memory straight into LDS, 512 columns of one row (1 KiB) per wave instruction:
    // the row and column of a piece are wave-uniform and travel in the scalar offset and in M0.
    const int segs = (kcLen + 511) / 512;
    for (int i = __builtin_amdgcn_readfirstlane(wave); i < rows * segs; i += THREADS / 64) {
      const int r = i / segs, c0 = (i - r * segs) * 512;
      const int from = __builtin_amdgcn_readfirstlane((int)(((int64_t)r * a.ldx + kc + c0) * sizeof(T)));
      const unsigned to = __builtin_amdgcn_readfirstlane(ldsBase + (unsigned)((r * ldx + c0) * sizeof(T)));
      if (c0 + lane * 8 < kcLen) loadToLds16(rsX, lane * 16, from, to);
    }
    __builtin_amdgcn_s_waitcnt(0x0070);  // this wave's pieces have landed
    __syncthreads();
    const T* xrow[G];  // fragment rows past M repeat the last row and are discarded
#pragma unroll
    for (int gi = 0; gi < G; ++gi) xrow[gi] = sx + min(gi * 16 + r16, rows - 1) * ldx + kgrp * 32;
    for (int s = sBegin; s < sEnd; ++s) {
      const u32x4 c0 = w0, c1 = w1;
      if (s + 1 < sEnd) {
        w0 = *reinterpret_cast<const u32x4*>(wk + (s + 1) * kW8Block);
        w1 = *reinterpret_cast<const u32x4*>(wk + (s + 1) * kW8Block + 16);
      }
      const Frag f0 = cvt8<T>(c0[0], c0[1]), f1 = cvt8<T>(c0[2], c0[3]), f2 = cvt8<T>(c1[0], c1[1]), f3 = cvt8<T>(c1[2], c1[3]);
#pragma unroll
      for (int gi = 0; gi < G; ++gi) {
        const T* xp = xrow[gi] + s * kW8Block;
        acc[gi] = W8Mfma<T>::run(*reinterpret_cast<const Frag*>(xp), f0, acc[gi]);
        acc[gi] = W8Mfma<T>::run(*reinterpret_cast<const Frag*>(xp + 8), f1, acc[gi]);
        acc[gi] = W8Mfma<T>::run(*reinterpret_cast<const Frag*>(xp + 16), f2, acc[gi]);
        acc[gi] = W8Mfma<T>::run(*reinterpret_cast<const Frag*>(xp + 24), f3, acc[gi]);
      }
    }
  }
  // the partial sums of the K split meet where the activations were
  __syncthreads();
  float* red = reinterpret_cast<float*>(w8smem);  // [NTW * kW8KSplit][G][4][64]
#pragma unroll
  for (int gi = 0; gi < G; ++gi)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[((wave * G + gi) * 4 + r) * 64 + lane] = acc[gi][r];
  __syncthreads();
  if (ks == 0 && col < a.N) {
    T* out = reinterpret_cast<T*>(a.out);
#pragma unroll
    for (int gi = 0; gi < G; ++gi)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = m0 + gi * 16 + kgrp * 4 + r;
        if (row < a.M) {
          float v = 0.f;
#pragma unroll
          for (int w = 0; w < kW8KSplit; ++w) v += red[(((tile * kW8KSplit + w) * G + gi) * 4 + r) * 64 + lane];
          out[(int64_t)row * a.ldo + col] = static_cast<T>(v * sc + bv);
        }
      }
  }
}

// Wide weights: both operands staged through LDS, the int8 counterpart of the bf16 decode kernel.
//   * Weight loads that deliver MFMA fragments straight into registers touch 16 rows x 32 bytes per instruction, a pattern
//     that streams far below what whole-row pieces reach. Here a copy instruction takes 256 contiguous bytes of 4 weight
//     rows (or 512 bytes of 2 activation rows) and lands in LDS without passing through registers, 16-byte pieces
//     XOR-swizzled by row on the global side so that the fragment reads are conflict-free. The weight copies are
//     non-temporal (read once; they must not push the activations out of L2).
//   * The host deals the output channels evenly over the CUs: a workgroup of eight waves owns colsPerWg of them (at most
//     32 NTP) for the whole of K and at most 64 rows (grid.y walks further row groups). K moves in stages of BK = 256
//     (stages of 512, deeper rings of either operand and two stages per barrier all measured slower): wave w
//     takes columns 64 (w % 4) .. + 63 of every stage, lane (n, kgrp) 16 consecutive int8 of them (one 16-byte LDS read,
//     converted in registers into the operands of two MFMAs), all G row groups against the NTP channel tiles of its half.
//     The four shares meet in LDS at the end, where wave w finishes row group w % 4: per-channel scale on the fp32 sum,
//     bias, one rounding.
//   * Loads return to a wave in the order it issued them, so weights (HBM) and activations (L2) are copied by
//     different waves, 0-3 and 4-7, each waiting only for its own stage; one barrier per stage publishes both.
//     Workgroup b starts its walk over K at stage (13 b) mod stages, so that the requests of a moment spread over
//     the memory channels.
constexpr int kW8LdsStagger = 13;

template <typename T, int G, int NTP, int BK, int WST, int XST>
__global__ __launch_bounds__(512) void w8LinearLdsKernel(W8Args a) {
  using Frag = typename W8Mfma<T>::Frag;
  constexpr int BN = 32 * NTP;
  constexpr int LW = BK / 16, LX = BK * (int)sizeof(T) / 16;   // 16-byte pieces (= lanes of a copy instruction) per weight / activation row
  constexpr int RW = 64 / LW, RX = 64 / LX;                    // rows one copy instruction covers
  constexpr int WIPW = BN / RW / 4, XIPW = G * 16 / RX / 4;    // copy instructions (1 KiB) per wave and stage: weights, activations
  constexpr int WBUF = BN * BK, XBUF = G * 16 * BK * (int)sizeof(T);  // bytes per stage buffer
  constexpr int UNROLL = WST % XST == 0 ? WST : (XST % WST == 0 ? XST : WST * XST);
  constexpr int IPW = WIPW > XIPW ? WIPW : XIPW;
  constexpr int PPW = BK / 64 / 4;   // 64-column pieces of a stage per wave
  static_assert(PPW >= 1 && LX <= 64, "a stage is 256 or 512 columns");
  extern __shared__ __attribute__((aligned(16))) char w8smem[];
  char* sw = w8smem;                 // WST weight buffers: BN rows x BK bytes
  char* sx = sw + WST * WBUF;        // XST activation buffers: 16 G rows x 2 BK bytes
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, kgrp = lane >> 4;
  const int ci = wave & 3, kq = wave & 3, nb = wave >> 2;
  const int n0 = blockIdx.x * a.colsPerWg, nCols = min(a.colsPerWg, a.N - n0);
  const int m0 = blockIdx.y * 16 * G, rows = min(16 * G, a.M - m0);
  // the host sends only K that are multiples of BK here; with K split over gridDim.z this workgroup takes the stages
  // from firstStage on (every slice holds at least one)
  const int allStages = a.K / BK;
  const int firstStage = a.partial ? (int)blockIdx.z * a.stagesPerSlice : 0;
  const int nStages = a.partial ? min(a.stagesPerSlice, allStages - firstStage) : allStages;
  const int kStart = (int)((blockIdx.x * (unsigned)kW8LdsStagger) % (unsigned)nStages);
  auto descriptor = [](const void* base, int64_t bytes) {
    const uint64_t p = reinterpret_cast<uint64_t>(base);
    u32x4 d = {(uint32_t)p, (uint32_t)(p >> 32) & 0xffffu, (uint32_t)bytes, 0x00020000u};
    return d;
  };
  const bool copiesW = wave < 4;
  const u32x4 rs = copiesW ? descriptor(a.w, (int64_t)(a.N - 1) * a.ldw + a.K)
                           : descriptor(reinterpret_cast<const T*>(a.x) + (int64_t)m0 * a.ldx, ((int64_t)(rows - 1) * a.ldx + a.K) * sizeof(T));
  const int ipw = copiesW ? WIPW : XIPW;
  const unsigned ldsBase = (unsigned)(size_t)(__attribute__((address_space(3))) char*)(copiesW ? sw : sx);
  const unsigned bufBytes = copiesW ? WBUF : XBUF;
  // copy instruction q = ci + 4 i fills 1 KiB of a buffer: RW weight rows (LW pieces each) or RX activation rows (LX
  // pieces each); a lane owns one physical piece and fetches the logical piece the swizzle puts there.
  // Weight rows past this workgroup's channels and activation rows past M get an offset past the end of the descriptor,
  // which reads zeros without traffic.
  unsigned voff[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int q = ci + 4 * i;
    if (copiesW) {
      const int row = RW * q + lane / LW, piece = (lane % LW) ^ (row & 15);
      voff[i] = row < nCols ? (unsigned)((int64_t)(n0 + row) * a.ldw + piece * 16) : 0x80000000u;
    } else {
      const int row = RX * q + lane / LX, piece = (lane % LX) ^ (row & 15);
      voff[i] = row < rows ? (unsigned)(((int64_t)row * a.ldx) * sizeof(T) + piece * 16) : 0x80000000u;
    }
  }
  auto copyStage = [&](int c, int buf) {  // a stage past the end copies the last one again, into a buffer nobody reads any more
    int cc = min(c, nStages - 1) + kStart;
    if (cc >= nStages) cc -= nStages;
    const int from = __builtin_amdgcn_readfirstlane((firstStage + cc) * BK * (copiesW ? 1 : (int)sizeof(T)));
#pragma unroll
    for (int i = 0; i < IPW; ++i)
      if (i < ipw) {
        const unsigned to = ldsBase + (unsigned)buf * bufBytes + (unsigned)(ci + 4 * i) * 1024u;
        if (copiesW) loadToLds16Stream(rs, (int)voff[i], from, to);
        else loadToLds16(rs, (int)voff[i], from, to);
      }
  };
  // scale and bias of the channels this wave finishes: requested now, used at the end
  float sc[NTP], bv[NTP];
#pragma unroll
  for (int j = 0; j < NTP; ++j) {
    const int lc = (nb * NTP + j) * 16 + r16;
    sc[j] = bv[j] = 0.f;
    if (lc < nCols) {
      sc[j] = loadAs<float>(a.scale, n0 + lc, a.scaleDtype);
      if (a.bias) bv[j] = loadAs<float>(a.bias, n0 + lc, a.biasDtype);
    }
  }
  f32x4 acc[G][NTP];
#pragma unroll
  for (int gi = 0; gi < G; ++gi)
#pragma unroll
    for (int j = 0; j < NTP; ++j) acc[gi][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  // this wave's fragments of 64-column piece p = kq + 4 pp: weights 16-byte piece 4 p + kgrp of row r16 (+ 16 (NTP nb + j)
  // rows): 16 int8, the K slots of two MFMAs; activations pieces 8 p + 2 kgrp + t of row r16 (+ 16 gi rows): the 8
  // elements that meet the t-th half of those int8
  const char* wlane[PPW];
  const char* xlane[PPW][2];
#pragma unroll
  for (int pp = 0; pp < PPW; ++pp) {
    const int p = kq + 4 * pp;
    wlane[pp] = sw + (nb * NTP * 16 + r16) * BK + (((4 * p + kgrp) ^ r16) << 4);
#pragma unroll
    for (int t = 0; t < 2; ++t) xlane[pp][t] = sx + r16 * BK * (int)sizeof(T) + (((8 * p + 2 * kgrp + t) ^ r16) << 4);
  }

  if (copiesW) {
#pragma unroll
    for (int c = 0; c < WST - 1; ++c) copyStage(c, c);
  } else {
#pragma unroll
    for (int c = 0; c < XST - 1; ++c) copyStage(c, c);
  }
  for (int c0 = 0; c0 < nStages; c0 += UNROLL) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u;
      if (c < nStages) {  // workgroup-uniform
        // this wave's copies of stage c have landed (loads return in order; only the stages requested after it are in
        // flight); past the barrier both operands of the stage are in LDS and every wave has left the buffers of stage c - 1
        if (copiesW) {
          constexpr int n = (WST - 2) * WIPW;
          __builtin_amdgcn_s_waitcnt(0x0f70 | (n & 15) | ((n >> 4) << 14));
        } else {
          constexpr int n = (XST - 2) * XIPW;
          __builtin_amdgcn_s_waitcnt(0x0f70 | (n & 15) | ((n >> 4) << 14));
        }
        __builtin_amdgcn_s_barrier();
        if (copiesW) copyStage(c + WST - 1, (u + WST - 1) % WST);
        else copyStage(c + XST - 1, (u + XST - 1) % XST);
#pragma unroll
        for (int pp = 0; pp < PPW; ++pp) {
          Frag x0[G], x1[G];
#pragma unroll
          for (int gi = 0; gi < G; ++gi) {
            x0[gi] = *reinterpret_cast<const Frag*>(xlane[pp][0] + (u % XST) * XBUF + gi * 16 * BK * (int)sizeof(T));
            x1[gi] = *reinterpret_cast<const Frag*>(xlane[pp][1] + (u % XST) * XBUF + gi * 16 * BK * (int)sizeof(T));
          }
#pragma unroll
          for (int j = 0; j < NTP; ++j) {
            const u32x4 w = *reinterpret_cast<const u32x4*>(wlane[pp] + (u % WST) * WBUF + j * 16 * BK);
            const Frag f0 = cvt8<T>(w[0], w[1]), f1 = cvt8<T>(w[2], w[3]);
#pragma unroll
            for (int gi = 0; gi < G; ++gi) {
              acc[gi][j] = W8Mfma<T>::run(x0[gi], f0, acc[gi][j]);
              acc[gi][j] = W8Mfma<T>::run(x1[gi], f1, acc[gi][j]);
            }
          }
        }
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // the repeated copies of the last stage: nothing may land after the workgroup has gone
  __syncthreads();
  // the four shares of a channel tile meet where the stages were; wave (nb, kq) then finishes row group kq
  float* red = reinterpret_cast<float*>(w8smem);  // [8 waves][G][NTP][4][64]
#pragma unroll
  for (int gi = 0; gi < G; ++gi)
#pragma unroll
    for (int j = 0; j < NTP; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[(((wave * G + gi) * NTP + j) * 4 + r) * 64 + lane] = acc[gi][j][r];
  __syncthreads();
  const int gi = kq;
  if (gi < G) {
    T* out = reinterpret_cast<T*>(a.out);
#pragma unroll
    for (int j = 0; j < NTP; ++j) {
      const int lc = (nb * NTP + j) * 16 + r16;
      if (lc >= nCols) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = gi * 16 + kgrp * 4 + r;
        if (row < rows) {
          float v = 0.f;
#pragma unroll
          for (int k2 = 0; k2 < 4; ++k2) v += red[((((nb * 4 + k2) * G + gi) * NTP + j) * 4 + r) * 64 + lane];
          if (a.partial) a.partial[((int64_t)blockIdx.z * a.M + m0 + row) * a.N + n0 + lc] = v;
          else out[(int64_t)(m0 + row) * a.ldo + n0 + lc] = static_cast<T>(v * sc[j] + bv[j]);
        }
      }
    }
  }
}

// out[m, n] = (sum over the K slices of partial[z][m][n]) * scale[n] + bias[n]: four consecutive channels per thread.
template <typename T>
__global__ __launch_bounds__(256) void w8SliceReduceKernel(W8Args a, int slices) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, perRow = a.N / 4;
  if (idx >= (int64_t)a.M * perRow) return;
  const int64_t m = idx / perRow, n = (idx - m * perRow) * 4;
  f32x4 v = *reinterpret_cast<const f32x4*>(a.partial + m * a.N + n);
  for (int z = 1; z < slices; ++z) {
    const f32x4 p = *reinterpret_cast<const f32x4*>(a.partial + ((int64_t)z * a.M + m) * a.N + n);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] += p[e];
  }
  typedef T T4 __attribute__((ext_vector_type(4)));
  T4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float r = v[e] * loadAs<float>(a.scale, n + e, a.scaleDtype);
    if (a.bias) r += loadAs<float>(a.bias, n + e, a.biasDtype);
    o[e] = static_cast<T>(r);
  }
  *reinterpret_cast<T4*>(reinterpret_cast<T*>(a.out) + m * a.ldo + n) = o;
}

template <typename T, int G, int NTP, int BK, int WST, int XST>
static diopiError_t launchW8Lds(hipStream_t stream, const W8Args& a) {
  constexpr int BN = 32 * NTP;
  AMD_CHECK(a.colsPerWg >= 1 && a.colsPerWg <= BN, "int8 linear: %d channels per workgroup do not fit %d", a.colsPerWg, BN);
  const int lds = std::max((WST * BN + XST * G * 16 * (int)sizeof(T)) * BK, 8 * G * NTP * 4 * 64 * (int)sizeof(float));
  AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&w8LinearLdsKernel<T, G, NTP, BK, WST, XST>), lds));
  const int slices = a.partial ? (a.K / BK + a.stagesPerSlice - 1) / a.stagesPerSlice : 1;
  dim3 grid((unsigned)((a.N + a.colsPerWg - 1) / a.colsPerWg), (unsigned)((a.M + 16 * G - 1) / (16 * G)), (unsigned)slices);
  hipLaunchKernelGGL((w8LinearLdsKernel<T, G, NTP, BK, WST, XST>), grid, dim3(512), lds, stream, a);
  AMD_LAUNCH_CHECK();
  if (a.partial) {
    const int64_t items = (int64_t)a.M * (a.N / 4);
    hipLaunchKernelGGL(w8SliceReduceKernel<T>, dim3((unsigned)ceilDiv(items, (int64_t)256)), dim3(256), 0, stream, a, slices);
    AMD_LAUNCH_CHECK();
  }
  return diopiSuccess;
}

template <typename T, int NTW, int G>
static diopiError_t launchW8(hipStream_t stream, const W8Args& a) {
  constexpr int CHUNK = kW8RowsK / (16 * G);
  const size_t staged = (size_t)std::min(16 * G, a.M) * (std::min(a.K, CHUNK) + kW8Pad) * sizeof(T);
  const size_t lds = std::max(staged, (size_t)NTW * kW8KSplit * G * 4 * 64 * sizeof(float));
  // the largest request (16 G rows x one chunk) covers every later one
  AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&w8LinearKernel<T, NTW, G>), 16 * G * (CHUNK + kW8Pad) * (int)sizeof(T)));
  const int tiles = (a.N + 15) / 16;
  dim3 grid((unsigned)((tiles + NTW - 1) / NTW), (unsigned)((a.M + 16 * G - 1) / (16 * G)));
  hipLaunchKernelGGL((w8LinearKernel<T, NTW, G>), grid, dim3(NTW * kW8KSplit * 64), lds, stream, a);
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

template <typename T, int G>
static diopiError_t launchW8ForTiles(hipStream_t stream, const W8Args& a) {
  // 16-channel tiles per workgroup: enough to bring the grid down to about one workgroup per CU
  const int tiles = (a.N + 15) / 16;
  const int ntw = std::min(kW8MaxTiles, std::max(1, (tiles + computeUnits() - 1) / computeUnits()));
  switch (ntw) {
    case 1: return launchW8<T, 1, G>(stream, a);
    case 2: return launchW8<T, 2, G>(stream, a);
    case 3: return launchW8<T, 3, G>(stream, a);
    default: return launchW8<T, 4, G>(stream, a);
  }
}

// K slices for a weight of fewer than 10240 channels at more than 16 rows, or with a long K (0: the call keeps the other
// forms): 64 channels per workgroup and enough slices of whole 256-column stages to give every CU a workgroup, so that a
// workgroup stages only its slice of the activations (with whole K per workgroup the activations, re-read by every
// workgroup, outweigh the weights: 64 x 4096 x 14336 took 68 us against 28 for the same product with 16-bit weights;
// 64 x 8192 x 28672 110 -> 73 us, 16 x 8192 x 8192 23.8 -> 16.9 us).
static int w8SlicesFor(const W8Args& a) {
  if (a.M > 64 || a.N >= 10240 || a.N < 64 || a.N % 4 != 0 || a.K % 256 != 0 || a.K < (a.M <= 16 ? 8192 : 2048)) return 0;
  // (a few rows against a large weight of medium width stream well as they are: 1 x 8192 x 28672 35.6 us, 39.4 in slices)
  if (a.M <= 4 && a.N >= 6144 && (int64_t)a.N * a.K >= ((int64_t)1 << 27)) return 0;
  if ((int64_t)(a.N - 1) * a.ldw + a.K >= ((int64_t)1 << 31) || a.ldo % 4 != 0) return 0;
  const int wgs = (a.N + 63) / 64, stages = a.K / 256;
  const int want = std::max(1, computeUnits() / wgs);
  const int slices = std::min(std::min(want, stages / 2), 16);  // at least two stages per slice
  return slices >= 2 ? slices : 0;
}

template <typename T>
static diopiError_t launchW8ForShape(hipStream_t stream, const W8Args& a0) {
  W8Args a = a0;
  if (a.partial) {  // the caller has asked w8SlicesFor and brought the workspace
    a.colsPerWg = 64;
    if (a.M <= 16) return launchW8Lds<T, 1, 2, 256, 4, 4>(stream, a);
    if (a.M <= 32) return launchW8Lds<T, 2, 2, 256, 4, 3>(stream, a);
    return launchW8Lds<T, 4, 2, 256, 4, 2>(stream, a);
  }
  // Wide weights go through w8LinearLdsKernel, the channels dealt evenly over the CUs. Measured cold against the form
  // below at K = 4096 (us, 1 / 16 / 32 / 64 rows): N = 11008 11.0 -> 10.8, 12.9 -> 11.7, 17.0 -> 14.2, 23.1 -> 21.1;
  // N = 22016 22.0 -> 19.2, 26.8 -> 20.2. Both forms have about 10 us of floor at these sizes, so narrower weights
  // gain only with more than 16 rows (N = 6144: 14.7 -> 13.1 at 32 rows, 9.0 -> 10.4 at one).
  if ((a.N >= 10240 || (a.N >= 6144 && a.M > 16)) && a.K % 256 == 0 && (int64_t)(a.N - 1) * a.ldw + a.K < ((int64_t)1 << 31)) {
    const int cus = computeUnits(), rounds = (a.N + 128 * cus - 1) / (128 * cus);
    a.colsPerWg = (a.N + cus * rounds - 1) / (cus * rounds);
    if (a.colsPerWg > 64) {
      if (a.M <= 16) return launchW8Lds<T, 1, 4, 256, 3, 3>(stream, a);
      if (a.M <= 32) return launchW8Lds<T, 2, 4, 256, 3, 3>(stream, a);
      return launchW8Lds<T, 4, 4, 256, 2, 2>(stream, a);
    }
    if (a.M <= 16) return launchW8Lds<T, 1, 2, 256, 4, 4>(stream, a);
    if (a.M <= 32) return launchW8Lds<T, 2, 2, 256, 4, 3>(stream, a);
    return launchW8Lds<T, 4, 2, 256, 4, 2>(stream, a);
  }
  if (a.M <= 16) return launchW8ForTiles<T, 1>(stream, a);
  if (a.M <= 32) return launchW8ForTiles<T, 2>(stream, a);
  return launchW8ForTiles<T, 4>(stream, a);
}

// Any K / alignment: one lane per output element, fp32 accumulate (correctness path).
template <typename T>
__global__ __launch_bounds__(256) void w8LinearScalarKernel(W8Args a) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)a.M * a.N) return;
  const int m = (int)(idx / a.N), n = (int)(idx % a.N);
  const T* x = reinterpret_cast<const T*>(a.x) + (int64_t)m * a.ldx;
  const int8_t* w = a.w + (int64_t)n * a.ldw;
  float acc = 0.f;
  for (int k = 0; k < a.K; ++k) acc += static_cast<float>(x[k]) * static_cast<float>(w[k]);
  float v = acc * loadAs<float>(a.scale, n, a.scaleDtype);
  if (a.bias) v += loadAs<float>(a.bias, n, a.biasDtype);
  reinterpret_cast<T*>(a.out)[(int64_t)m * a.ldo + n] = static_cast<T>(v);
}

// Many rows (prefill with int8 weights): the streaming kernels above read the weights once per 64 rows, which at 8192
// rows is 128 times. From 129 rows on the weights are expanded once to the activation type (exact: an int8 fits its
// mantissa), the dense GEMM multiplies with alpha = 1 / 128 (so that the unscaled sums stay far inside the range of
// fp16), and one pass over the result applies the channel scale: 8192 x 11008 x 4096 2387 -> about 600 us. Where the
// product goes to the large-tile kernel, that kernel's epilogue multiplies the fp32 sums by the channel scale instead
// (alpha = 1, one rounding, no pass over the result).
// The scale is applied to the sum, not folded into the weights: a weight rounded with its scale puts noise of
// the size of the largest terms on every output, which the small outputs of a long sum do not survive. For the same
// reason a call with a bias takes this route only where the epilogue adds it to the fp32 sum, and stays with the
// streaming kernels otherwise: added after the sum has been rounded, a bias that nearly cancels it leaves the
// rounding error of the sum on a result many times smaller.
template <typename T>
__global__ __launch_bounds__(256) void w8ExpandKernel(T* __restrict__ dst, const int8_t* __restrict__ w, int64_t n, int64_t k,
                                                       int64_t ldw) {
  typedef T T8 __attribute__((ext_vector_type(8)));
  const int64_t perRow = k / 16;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n * perRow) return;
  const int64_t row = idx / perRow, piece = idx - row * perRow;
  const u32x4 q = *reinterpret_cast<const u32x4*>(w + row * ldw + piece * 16);
  T8 lo, hi;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    lo[e] = static_cast<T>(static_cast<float>((int8_t)(q[e >> 2] >> (8 * (e & 3)))));
    hi[e] = static_cast<T>(static_cast<float>((int8_t)(q[2 + (e >> 2)] >> (8 * (e & 3)))));
  }
  T8* o = reinterpret_cast<T8*>(dst + row * k + piece * 16);
  o[0] = lo, o[1] = hi;
}

constexpr float kW8SumScale = 1.f / 128.f;

// out[m, n] = out[m, n] / kW8SumScale * scale[n], in place; a lane takes PER consecutive columns (8 when rows and base
// are 16-byte aligned, else 1) and walks rows blockIdx.y, blockIdx.y + gridDim.y, ...
template <typename T, int PER>
__global__ __launch_bounds__(256) void w8ScaleKernel(T* __restrict__ out, const void* scale, int scaleDtype, int64_t m, int64_t n) {
  typedef T TV __attribute__((ext_vector_type(PER)));
  const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * PER;
  if (col >= n) return;
  float sc[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) sc[e] = loadAs<float>(scale, col + e, scaleDtype) * (1.f / kW8SumScale);
  for (int64_t row = blockIdx.y; row < m; row += gridDim.y) {
    TV* o = reinterpret_cast<TV*>(out + row * n + col);
    TV v = *o;
#pragma unroll
    for (int e = 0; e < PER; ++e) v[e] = static_cast<T>(static_cast<float>(v[e]) * sc[e]);
    *o = v;
  }
}

constexpr int64_t kW8ExpandFromRows = 129;

}  // namespace amd

using namespace amd;

extern "C" __attribute__((visibility("default"))) diopiError_t diopiWeightOnlyInt8Linear(
    diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t inH, diopiConstTensorHandle_t wH,
    diopiConstTensorHandle_t scaleH, diopiConstTensorHandle_t biasH) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, in, w, sc, bias;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(inH, &in, "input"));
  AMD_TRY(getView(wH, &w, "weight"));
  AMD_TRY(getView(scaleH, &sc, "scale"));
  AMD_TRY(getView(biasH, &bias, "bias"));
  AMD_CHECK(out.defined() && in.defined() && w.defined() && sc.defined(), "diopiWeightOnlyInt8Linear: null tensor");
  AMD_CHECK(w.dtype == diopi_dtype_int8 && w.ndim == 2, "diopiWeightOnlyInt8Linear: weight must be int8 [N, K]");
  AMD_CHECK(in.dtype == diopi_dtype_bfloat16 || in.dtype == diopi_dtype_float16,
            "diopiWeightOnlyInt8Linear: input must be bfloat16 or float16, got %s", dtypeName(in.dtype));
  AMD_CHECK(out.dtype == in.dtype, "diopiWeightOnlyInt8Linear: out dtype differs from input dtype");
  AMD_CHECK(in.ndim >= 1 && out.ndim == in.ndim, "diopiWeightOnlyInt8Linear: out must be shaped like input");
  const int64_t N = w.shape[0], K = w.shape[1];
  AMD_CHECK(in.shape[in.ndim - 1] == K, "diopiWeightOnlyInt8Linear: input last dim %ld differs from K=%ld",
            (long)in.shape[in.ndim - 1], (long)K);
  AMD_CHECK(out.shape[out.ndim - 1] == N, "diopiWeightOnlyInt8Linear: out last dim %ld differs from N=%ld",
            (long)out.shape[out.ndim - 1], (long)N);
  AMD_CHECK(sc.numel == N && isFloatDtype(sc.dtype) && sc.dtype != diopi_dtype_float64,
            "diopiWeightOnlyInt8Linear: scale must hold N fp16/bf16/fp32 values");
  if (bias.defined())
    AMD_CHECK(bias.numel == N && isFloatDtype(bias.dtype) && bias.dtype != diopi_dtype_float64,
              "diopiWeightOnlyInt8Linear: bias must hold N fp16/bf16/fp32 values");
  const int64_t M = K > 0 ? in.numel / K : 0;
  AMD_CHECK(out.numel == M * N, "diopiWeightOnlyInt8Linear: out has %ld elements, expected %ld", (long)out.numel, (long)(M * N));
  if (M == 0 || N == 0) return diopiSuccess;
  TensorView cin, cw, csc, cb;
  AMD_TRY(makeContiguous(ctx, stream, in, &cin));
  AMD_TRY(makeContiguous(ctx, stream, sc, &csc));
  if (bias.defined()) AMD_TRY(makeContiguous(ctx, stream, bias, &cb));
  cw = w;
  if (!(w.stride[1] == 1 || K == 1)) AMD_TRY(makeContiguous(ctx, stream, w, &cw));
  TensorView cout = out;
  bool outTemp = !out.isContiguous();
  if (outTemp) {
    diopiTensorHandle_t th;
    AMD_TRY(requireTensor(ctx, out.shape, out.ndim, out.dtype, &th, &cout));
  }
  GemmProblem p;
  p.dtype = in.dtype, p.batch = 1, p.M = M, p.N = N, p.K = K;
  p.A = cin.data, p.sAm = K, p.sAk = 1;
  p.B = cw.data, p.sBn = K, p.sBk = 1;  // (stands in for the expanded copy, which is aligned at least as well)
  p.out = cout.data, p.sOm = N;
  // where the product goes to the kernel that can scale every column in its epilogue, the channel scale (and a bias)
  // meet the fp32 sum there: 8192 x 11008 x 4096 594 -> 544 us, 2048 rows 204 -> 183 us (the same products with 16-bit
  // weights: 499 and 151 us; what remains above them is the expansion)
  const bool manyRows = M >= kW8ExpandFromRows && K % 16 == 0 && cw.aligned16() && (N == 1 || cw.stride[0] % 16 == 0);
  const bool scaleInEpilogue = manyRows && gemmAppliesColumnScale(p);
  if (manyRows && (scaleInEpilogue || !bias.defined())) {
    void* expanded = nullptr;
    AMD_TRY(requireWorkspace(ctx, N * K * in.itemsize, &expanded));
    const int64_t pieces = N * (K / 16), ldw = N > 1 ? cw.stride[0] : K;
    AMD_CHECK(ceilDiv(pieces, (int64_t)256) <= 0x7fffffff, "diopiWeightOnlyInt8Linear: weight of %ld x %ld is too large", (long)N, (long)K);
    const dim3 egrid((unsigned)ceilDiv(pieces, (int64_t)256));
    const int per = N % 8 == 0 && cout.aligned16() ? 8 : 1;
    const dim3 sgrid((unsigned)ceilDiv(N / per, (int64_t)256), (unsigned)std::min<int64_t>(M, 2048));
    p.B = expanded;
    p.alpha = kW8SumScale;
    if (scaleInEpilogue) {
      p.alpha = 1.f, p.colScale = csc.data, p.colScaleDtype = csc.dtype;
      if (bias.defined()) p.colBias = cb.data, p.colBiasDtype = cb.dtype;
    }
#define W8_MANY_ROWS(T)                                                                                                          \
  do {                                                                                                                           \
    hipLaunchKernelGGL(w8ExpandKernel<T>, egrid, dim3(256), 0, stream, static_cast<T*>(expanded), cw.ptr<int8_t>(), N, K, ldw);   \
    AMD_LAUNCH_CHECK();                                                                                                          \
    AMD_TRY(runGemm(ctx, stream, p));                                                                                            \
    if (scaleInEpilogue) break;                                                                                                  \
    if (per == 8) hipLaunchKernelGGL((w8ScaleKernel<T, 8>), sgrid, dim3(256), 0, stream, cout.ptr<T>(), csc.data, (int)csc.dtype, M, N); \
    else hipLaunchKernelGGL((w8ScaleKernel<T, 1>), sgrid, dim3(256), 0, stream, cout.ptr<T>(), csc.data, (int)csc.dtype, M, N);   \
  } while (0)
    if (in.dtype == diopi_dtype_bfloat16) W8_MANY_ROWS(bf16_t);
    else W8_MANY_ROWS(half_t);
#undef W8_MANY_ROWS
    AMD_LAUNCH_CHECK();
    if (outTemp) AMD_TRY(stridedCopy(stream, cout, out));
    return diopiSuccess;
  }
  W8Args a;
  a.x = cin.data, a.w = cw.ptr<int8_t>(), a.scale = csc.data, a.bias = bias.defined() ? cb.data : nullptr, a.out = cout.data;
  a.ldx = K, a.ldw = N > 1 ? cw.stride[0] : K, a.ldo = N;
  a.M = (int)M, a.N = (int)N, a.K = (int)K;
  a.scaleDtype = csc.dtype, a.biasDtype = bias.defined() ? cb.dtype : diopi_dtype_float32;
  if (const int slices = w8SlicesFor(a); slices > 0 && cin.aligned16() && cw.aligned16() && a.ldw % 16 == 0 && cout.aligned16() &&
                                           (std::min<int64_t>(M, 64) * K + K) * 2 < (int64_t(1) << 31)) {
    const int stages = (int)(K / 256);
    a.stagesPerSlice = (stages + slices - 1) / slices;
    const int used = (stages + a.stagesPerSlice - 1) / a.stagesPerSlice;  // every slice holds at least one stage
    void* ws = nullptr;
    AMD_TRY(requireWorkspace(ctx, (int64_t)used * M * N * (int64_t)sizeof(float), &ws));
    a.partial = static_cast<float*>(ws);
  }
  const bool fast = K % kW8Block == 0 && cin.aligned16() && cw.aligned16() && a.ldw % 16 == 0 && ceilDiv(M, 64) <= 65535 &&
                    (std::min<int64_t>(M, 64) * K + K) * 2 < (int64_t(1) << 31);
  if (fast) {
    if (in.dtype == diopi_dtype_bfloat16) AMD_TRY(launchW8ForShape<bf16_t>(stream, a));
    else AMD_TRY(launchW8ForShape<half_t>(stream, a));
  } else {
    dim3 grid((unsigned)ceilDiv(M * N, 256));
    if (in.dtype == diopi_dtype_bfloat16) hipLaunchKernelGGL(w8LinearScalarKernel<bf16_t>, grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(w8LinearScalarKernel<half_t>, grid, dim3(256), 0, stream, a);
  }
  AMD_LAUNCH_CHECK();
  if (outTemp) AMD_TRY(stridedCopy(stream, cout, out));
  return diopiSuccess;
}
