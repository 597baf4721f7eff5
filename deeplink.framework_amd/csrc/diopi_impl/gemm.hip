// Dense contractions for gfx950: diopiMm, diopiBmm, diopiMatmul, diopiAddmm, diopiBaddbmm,
// diopiLinear (dipu/scripts/autogen_diopi_wrapper/diopi_functions.yaml:594-597,902-909,
// 1534-1548,1755-1765,1829-1837,1852-1893).
//
// MFMA engine (bf16 / fp16 inputs, fp32 accumulate) -- C[M,N] = A[M,K] . B[N,K]^T with both
// operands K-contiguous, which is exactly what the MFMA instructions want: every lane feeds 8
// consecutive K elements (one 16-byte LDS read) of one row.
//   * large problems with an even number of 64-wide K tiles: 256x256x64 macro tile, workgroup = 256 threads =
//     4 waves in a 2x2 arrangement (wave tile 128x128 = 8x8 tiles of v_mfma_f32_16x16x32, 256 fp32 accumulators
//     per lane in the accumulation registers), one persistent workgroup per CU, K loop placed instruction by
//     instruction (gemm_loop_4wave.inc, generated); its counters match the vendor library's kernel;
//   * large problems otherwise (K a multiple of 64): the same macro tile with 512 threads = 8 waves
//     in a 2x4 arrangement (wave tile 128x64 = 8x4 tiles of v_mfma_f32_16x16x32, 128 fp32
//     accumulators per lane, two waves per SIMD so one wave's LDS traffic hides behind the other's
//     MFMAs). The 16x16x32 shape draws less power per flop than 32x32x16 (an MFMA-only loop holds
//     ~2.02 GHz against ~1.86 GHz on random operands), and these kernels run at the power limit;
//   * operand tiles go from memory straight into a two-stage LDS ring (buffer_load ... lds, no
//     registers and no ds_write in between): tile k+1 lands in the other stage while tile k is
//     being multiplied, and the loads of tile k+2 start as soon as every wave is past the one
//     barrier per K tile. Operand rows are addressed through buffer descriptors (32-bit lane offset
//     + scalar K offset);
//   * fragments are double-buffered (A) or refilled in place (B) in registers and the order of
//     MFMAs, fragment reads and tile loads is pinned in groups of four MFMAs;
//   * LDS rows are 128 bytes (64 elements) with the 16-byte chunk index XOR-swizzled by
//     ((row >> 1) & 7): the 1 KiB blocks written by the tile loads and the ds_read_b128 operand
//     fetches (16 consecutive rows, 4 consecutive logical chunks) are bank-conflict free;
//   * workgroup ids are remapped so that each of the 8 XCDs (own L2 each) works on a
//     contiguous band of tiles, walked in groups of 8 tile-rows to reuse A and B from L2;
//   * epilogue: alpha * acc + beta * C + bias straight from the accumulators: the weight fragment is
//     the first MFMA operand, so a lane holds consecutive columns of one output row, and one lane
//     swap per register turns that into 16-byte pieces of C and of the addend; the stream never
//     waits for a store (code that may load an addend otherwise waits for the store before it);
//   * small or ragged problems: 128x128 (or 256x256) tiles with 4 waves of v_mfma_f32_32x32x16,
//     staged through registers, any K that is a multiple of 8, stores straight from the
//     accumulator layout;
//   * more than 64 rows but too few 256x256 tiles to fill the chip: the large-tile kernel with K split over
//     grid.y, fp32 partial products in workspace, and a reduction pass that applies the epilogue;
//   * at most 32 rows (64 while N is small), the decode shape: a weight-streaming kernel with 16-column tiles
//     whose waves split K and stage the activation rows in LDS.
// Operands that are not K-contiguous (mm with a row-major mat2, bmm's second operand) are
// transposed once into workspace by a tiled LDS transpose, then use the same engine.
//
// FMA engine: fp32 (and any shape/stride/alignment the MFMA engine rejects): 64x64 LDS
// tiles, 4x4 outputs per lane, fp32 accumulate.
#include <algorithm>
#include <type_traits>
#include <utility>

#include "gemm.hpp"

namespace amd {

// ------------------------------------------------------------- MFMA engine ---
template <typename T>
struct MfmaOp;
template <>
struct MfmaOp<bf16_t> {
  typedef bf16x8 Frag;
  typedef bf16x4 Half;
  static __device__ __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct MfmaOp<half_t> {
  typedef f16x8 Frag;
  typedef f16x4 Half;
  static __device__ __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

struct MfmaArgs {
  const void* A;
  const void* B;
  void* out;
  const void* Cin;
  const void* bias;
  int64_t sAb, lda, sBb, ldb, sOb, ldo, sCb, sCm, sCn;
  int M, N, K;
  int tilesM, tilesN;
  float alpha, beta;
  bool vecEpilogue;  // out / addend / bias allow 16-byte row segments
  float* partial = nullptr;  // split-K: fp32 partial products [gridDim.y][M][N]
  int kTilesPerSplit = 0;
  // rotary epilogue: adjacent column pairs (2i, 2i + 1) of every head of rotHeadDim columns below rotCols are
  // rotated by the angle whose cosine / sine sit at table[(row % rotTableRows) * rotHeadDim / 2 + i]
  const void* rotCos = nullptr;
  const void* rotSin = nullptr;
  int rotCols = 0, rotHeadDim = 0, rotTableRows = 1;
  bool rotTableF32 = false;
  float rotSinSign = 1.f;
  const void* colScale = nullptr;  // kEpiColScale: N values of dtype colScaleDtype, and optionally N of colBiasDtype to add
  int colScaleDtype = 0;
  const void* colBias = nullptr;
  int colBiasDtype = 0;
};

constexpr int kBK = 64;  // K elements per LDS tile (128-byte rows)

template <typename T, int BM, int BN>
__global__ __launch_bounds__(256) void gemmMfmaKernel(MfmaArgs g) {
  using Frag = typename MfmaOp<T>::Frag;
  constexpr int WM = BM / 2, WN = BN / 2;      // per-wave tile
  constexpr int TM = WM / 32, TN = WN / 32;    // MFMA tiles per wave
  constexpr int A_CH = BM * 8 / 256, B_CH = BN * 8 / 256;  // 16-byte chunks per thread per K tile
  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* sA = reinterpret_cast<T*>(smem);                  // [2][BM][64]
  T* sB = sA + 2 * BM * kBK;                           // [2][BN][64]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // ---- tile id: XCD band, then groups of 8 tile-rows
  int tm, tn;
  {
    const int total = g.tilesM * g.tilesN;
    const int pid = blockIdx.x;
    const int xcd = pid & 7, idx = pid >> 3;
    const int q = total >> 3, r = total & 7;
    const int logical = xcd * q + min(xcd, r) + idx;
    constexpr int GROUP = 8;
    const int width = GROUP * g.tilesN;
    const int group = logical / width;
    const int first = group * GROUP;
    const int gsize = min(g.tilesM - first, GROUP);
    const int in = logical - group * width;
    tm = first + in % gsize;
    tn = in / gsize;
  }
  const int batch = blockIdx.z;
  const T* A = reinterpret_cast<const T*>(g.A) + (int64_t)batch * g.sAb;
  const T* B = reinterpret_cast<const T*>(g.B) + (int64_t)batch * g.sBb;

  // ---- staging assignment: chunk id = tid + 256*i -> (row, 16-byte chunk)
  const T* aPtr[A_CH];
  const T* bPtr[B_CH];
  int aOff[A_CH], bOff[B_CH];
  const int c8 = (tid & 7) * 8;  // K offset of this thread's chunk inside a tile
#pragma unroll
  for (int i = 0; i < A_CH; ++i) {
    int row = (tid >> 3) + 32 * i;
    int grow = min(tm * BM + row, g.M - 1);
    aPtr[i] = A + (int64_t)grow * g.lda + c8;
    aOff[i] = row * kBK + (((tid & 7) ^ ((row >> 1) & 7)) << 3);
  }
#pragma unroll
  for (int i = 0; i < B_CH; ++i) {
    int row = (tid >> 3) + 32 * i;
    int grow = min(tn * BN + row, g.N - 1);
    bPtr[i] = B + (int64_t)grow * g.ldb + c8;
    bOff[i] = row * kBK + (((tid & 7) ^ ((row >> 1) & 7)) << 3);
  }
  Frag ra[A_CH], rb[B_CH];
  const int nK = (g.K + kBK - 1) / kBK;

  auto gload = [&](int kt) {
    const int k0 = kt * kBK;
    const bool inK = k0 + c8 < g.K;  // K is a multiple of 8: a chunk is entirely in or out
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    const Frag z = __builtin_bit_cast(Frag, zero4);
#pragma unroll
    for (int i = 0; i < A_CH; ++i) ra[i] = inK ? *reinterpret_cast<const Frag*>(aPtr[i] + k0) : z;
#pragma unroll
    for (int i = 0; i < B_CH; ++i) rb[i] = inK ? *reinterpret_cast<const Frag*>(bPtr[i] + k0) : z;
  };
  auto swrite = [&](int stage) {
    T* a = sA + stage * BM * kBK;
    T* b = sB + stage * BN * kBK;
#pragma unroll
    for (int i = 0; i < A_CH; ++i) *reinterpret_cast<Frag*>(a + aOff[i]) = ra[i];
#pragma unroll
    for (int i = 0; i < B_CH; ++i) *reinterpret_cast<Frag*>(b + bOff[i]) = rb[i];
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // operand fetch offsets: row = lane&31 inside an MFMA tile, chunk = 2*ks + (lane>>5)
  const int frow = lane & 31, fhalf = lane >> 5;

  gload(0);
  swrite(0);
  if (nK > 1) gload(1);
  __syncthreads();

  for (int kt = 0; kt < nK; ++kt) {
    const int cur = kt & 1;
    const T* a = sA + cur * BM * kBK + (wm * WM) * kBK;
    const T* b = sB + cur * BN * kBK + (wn * WN) * kBK;
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      Frag fa[TM], fb[TN];
      const int chunk = 2 * ks + fhalf;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        int row = i * 32 + frow;
        fa[i] = *reinterpret_cast<const Frag*>(a + row * kBK + ((chunk ^ ((row >> 1) & 7)) << 3));
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        int row = j * 32 + frow;
        fb[j] = *reinterpret_cast<const Frag*>(b + row * kBK + ((chunk ^ ((row >> 1) & 7)) << 3));
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = MfmaOp<T>::run(fa[i], fb[j], acc[i][j]);
    }
    if (kt + 1 < nK) {
      swrite(cur ^ 1);                 // tile kt+1 (loaded during the previous iteration)
      if (kt + 2 < nK) gload(kt + 2);  // in flight across the next iteration's math
    }
    __syncthreads();
  }

  // ---- epilogue
  T* out = reinterpret_cast<T*>(g.out) + (int64_t)batch * g.sOb;
  const T* cin = g.Cin ? reinterpret_cast<const T*>(g.Cin) + (int64_t)batch * g.sCb : nullptr;
  const T* bias = reinterpret_cast<const T*>(g.bias);
  // Two instruction streams: loads and stores share one in-order counter, so the addend of a whole
  // 32 x 32 block is requested before its first store (one wait per block instead of one per element,
  // each of which would also wait for the store before it), and without an addend nothing is loaded.
  auto store = [&](auto withAddend) {
    constexpr bool kAddend = decltype(withAddend)::value;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = tn * BN + wn * WN + j * 32 + frow;
      if (col >= g.N) continue;
      const float bv = bias ? static_cast<float>(bias[col]) : 0.f;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int rbase = tm * BM + wm * WM + i * 32 + fhalf * 4;
        float c[16];
        if constexpr (kAddend) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int row = min(rbase + (r >> 2) * 8 + (r & 3), g.M - 1);
            c[r] = static_cast<float>(cin[(int64_t)row * g.sCm + (int64_t)col * g.sCn]);
          }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = rbase + (r >> 2) * 8 + (r & 3);
          if (row < g.M) {
            float v = acc[i][j][r] * g.alpha + bv;
            if constexpr (kAddend) v += g.beta * c[r];
            out[(int64_t)row * g.ldo + col] = static_cast<T>(v);
          }
        }
      }
    }
  };
  if (cin)
    store(std::true_type{});
  else
    store(std::false_type{});
}

// ------------------------------------------------- software-pipelined 256x256 ---
// For K a multiple of 64 with at least two K tiles. Same LDS layout as gemmMfmaKernel<T,256,256>;
// the instruction stream of every wave is arranged by hand in four phases of 16 MFMAs per K tile
// so that it does not wait on LDS or HBM inside the K loop:
//   phase 0: k-step 0, rows 0-63   | A fragments of phase 1 | direct-to-LDS loads: B half of the next tile
//   phase 1: k-step 0, rows 64-127 | A fragments of phase 2, B fragments of k-step 1
//   phase 2: k-step 1, rows 0-63   | A fragments of phase 3
//   wait for this wave's tile loads, barrier: the next tile is published, this stage is free
//   phase 3: k-step 1, rows 64-127 | A and B fragments of phase 0 of the next tile |
//            direct-to-LDS loads: A half of the tile after next into the stage just freed
__device__ __forceinline__ void ldsBarrier() {
  // wait for this wave's LDS traffic only (lgkmcnt(0)); outstanding global loads keep flying
  __builtin_amdgcn_s_waitcnt(0xc07f);
  __builtin_amdgcn_s_barrier();
}


// 8 waves (2 x 4, wave tile 128 x 64): two waves per SIMD, so one wave's LDS / VMEM issue
// overlaps the other's MFMAs; measured faster than 4 waves of 128 x 128 and 16 of 64 x 64.
constexpr int kPipeWavesM = 2, kPipeWavesN = 4, kPipeThreads = kPipeWavesM * kPipeWavesN * 64;

// v_mfma_f32_16x16x32: lane l feeds row (l & 15), K elements [8 * (l >> 4), +8) of both operands and
// receives D[4 * (l >> 4) + r][l & 15], r = 0..3. The large-tile kernel passes the weight fragment
// first, so D is the transposed block and a lane holds four consecutive columns of output row (l & 15).
template <typename T>
struct MfmaOp16;
template <>
struct MfmaOp16<bf16_t> {
  static __device__ __forceinline__ f32x4 run(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct MfmaOp16<half_t> {
  static __device__ __forceinline__ f32x4 run(f16x8 a, f16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

// EPI selects the epilogue: kEpiLinear is alpha * acc + beta * C + bias; kEpiSiluMul treats every 64 consecutive
// output columns as 32 gate columns followed by the 32 up columns of the same channels and stores
// silu(gate) * up, half as wide (out has N / 2 columns); kEpiPartial is the split-K form: workgroup (tile, s)
// multiplies K tiles [s * kTilesPerSplit, ...) and stores its fp32 accumulators to partial[s], to be summed and
// given the linear epilogue by splitKReduceKernel; kEpiRotary is acc + bias followed by the interleaved rotary
// embedding on the leading rotCols columns (the q and k heads of a stacked QKV projection).
// kEpiRotaryUniform is kEpiRotary for the usual case, no bias and a rotated width that is a multiple of 32 columns:
// whether a lane's 32-column piece is rotated is then the same for the whole wave. It is an instantiation of its own
// because the one-wave-per-SIMD kernel has no register to spare for a second path next to the general one.
// kEpiRotaryLds (4-wave kernel only) is kEpiRotaryUniform for 16-bit tables and heads of 128 columns with the table
// entries of an output tile's first four fragment rows waiting in LDS when the epilogue starts (see rotaryTablesToLds).
// kEpiColScale (4-wave kernel only): out = alpha * sum * colScale[column] (+ colBias[column]), no addend (int8 weights
// expanded to the activation type, the channel scale and the bias applied to the fp32 sum).
// kEpiAddendLds (4-wave kernel only) is kEpiLinear with an addend whose pieces for an output tile's first two fragment
// rows wait in LDS when the epilogue starts (see addendToLds).
enum PipeEpilogue { kEpiLinear = 0, kEpiSiluMul = 1, kEpiPartial = 2, kEpiRotary = 3, kEpiRotaryUniform = 4, kEpiRotaryLds = 5, kEpiAddendLds = 6, kEpiColScale = 7 };
constexpr int kAddendLdsBytes = 32768;  // behind the two K-tile stages of the 4-wave kernel: 4 waves x 32 rows x 128 columns x 2 bytes
constexpr int kRotaryLdsBytes = 32768;  // behind the two K-tile stages of the 4-wave kernel: 128 rows x (64 cos | 64 sin) x 2 bytes

// The vector epilogue of the 256 x 256 kernels: a wave's TM x TN fragments of 16 x 16 (v_mfma_f32_16x16x32 with the
// weight fragment first, so lane (frow = l & 15, kq = l >> 4) holds columns 4 kq .. 4 kq + 3 of row frow of every
// fragment) whose first row is row0 and first column colBase; accRow(ic, row) hands over the TN accumulators of
// fragment row ic (a std::integral_constant), one fragment row at a time, so the accumulators may live anywhere.
//
// Straight from the accumulators: v_permlane16_swap between the two fragments of a 32-column pair leaves a lane
// with 8 consecutive columns (lane group q gets the columns starting at 16 * (q & 1) + 8 * (q >> 1)),
// so the addend is read and the result written as 16-byte pieces, 64 contiguous bytes per row and
// instruction, without a trip through LDS. alpha / beta / bias are applied in fp32 after the swap.
// Output and addend go through buffer descriptors (the host guarantees both span less than 2 GiB):
// a piece outside the matrix gets an offset past the end, which the hardware drops (stores) or
// answers with zeros (loads), so the instruction stream has no branches and the compiler can count
// outstanding accesses exactly. Loads and stores share one in-order counter: a wait for an addend
// piece also waits for every store before it, so the pieces of four fragment rows are requested
// together before the first store of the four (one exposed round trip per four rows instead of one per
// row), and without an addend there is no load (and no wait) in the stream.
// The rotary epilogue's table entries are what it waits for: with the loads answered by constants the launch is as
// long as a plain linear's, with them it was 26 - 37 us longer (8192 x 4096 x 12288; 15 - 21 us now), because a wave that asks for a
// batch of entries has nothing else to do until L2 answers, and with one wave per SIMD nobody else has either. So the
// workgroup copies the cosines and sines of the first four fragment rows of both row halves of its output tile
// (2 x 64 rows of 64 entries each, 16 KiB + 16 KiB) straight into LDS before the last K tiles run: the copies are
// over when the epilogue starts, and the entries of the other four rows are requested from memory at that point and
// arrive while the first four are worked through. Wave w copies table rows 32 w .. 32 w + 31 of that region (row
// r: row half r / 64, fragment row (r % 64) / 16, row in fragment r % 16): four copy instructions of 8 rows x 128
// bytes for the cosines and four for the sines. The caller waits for its own copies and meets the other waves at a
// barrier before the epilogue reads.
template <typename T>
__device__ __forceinline__ void rotaryTablesToLds(const MfmaArgs& g, int tileRow0, int wave, int lane, unsigned ldsTab) {
  int tableRows = g.rotTableRows;
  asm volatile("" : "+s"(tableRows));  // (a division by a run-time value: its set-up is not to be kept across the K loop)
  const int64_t bytes = (int64_t)tableRows * 64 * (int64_t)sizeof(T);
  auto descriptor = [&](const void* base) {
    uint64_t p = reinterpret_cast<uint64_t>(base);
    asm volatile("" : "+s"(p));  // built here, per call: eight scalar registers that must not stay live across the K loop
    u32x4 d = {(uint32_t)p, (uint32_t)(p >> 32) & 0xffffu, (uint32_t)bytes, 0x00020000u};
    return d;
  };
  const u32x4 rsCos = descriptor(g.rotCos), rsSin = descriptor(g.rotSin);
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int r = wave * 32 + q * 8 + (lane >> 3);
    const int row = tileRow0 + (r >> 6) * 128 + ((r >> 4) & 3) * 16 + (r & 15);
    const int voff = row < g.M ? ((row % tableRows) * 64 + (lane & 7) * 8) * (int)sizeof(T) : (int)0x80000000u;
    const unsigned to = ldsTab + (unsigned)(wave * 32 + q * 8) * 128u;
    loadToLds16(rsCos, voff, 0, to);
    loadToLds16(rsSin, voff, 0, to + 16384u);
  }
}

// The addend of the linear epilogue is waited for in the same way: a wave that asks for the pieces of four fragment
// rows has nothing to do until they arrive, twice per output tile. The 32 KiB behind the K-tile stages hold a quarter
// of a tile's addend, so every wave copies the addend of its own first two fragment rows (32 rows of 128 columns,
// 8 KiB) there before the last K tiles run, asks for the other six rows' pieces when the epilogue starts and works
// through the two rows in LDS while those are on their way: one shortened wait per tile instead of two whole ones.
// A copy instruction takes 4 rows of 256 bytes; the 16-byte piece p of local row r lies in slot p ^ (r & 15) of its
// row (the swizzle is applied to the global address), so that the 16 lanes which read one piece index of 16
// consecutive rows touch every bank once. A wave reads only what it copied itself: it waits for its own copies, and
// no barrier is needed.
template <typename T>
__device__ __forceinline__ void addendToLds(const MfmaArgs& g, const T* cin, int waveRow0, int waveCol0, int lane, unsigned ldsDst) {
  uint64_t p = reinterpret_cast<uint64_t>(cin);
  asm volatile("" : "+s"(p));  // the descriptor is built here, per call: its registers must not stay live across the K loop
  const u32x4 rsC = {(uint32_t)p, (uint32_t)(p >> 32) & 0xffffu, (uint32_t)(((int64_t)(g.M - 1) * g.sCm + g.N) * (int64_t)sizeof(T)), 0x00020000u};
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const int r = q * 4 + (lane >> 4);
    const int row = waveRow0 + r, col = waveCol0 + (((lane & 15) ^ (r & 15)) << 3);
    const int voff = row < g.M && col < g.N ? (int)(((int64_t)row * g.sCm + col) * (int64_t)sizeof(T)) : (int)0x80000000u;
    loadToLds16(rsC, voff, 0, ldsDst + (unsigned)q * 1024u);
  }
}

template <typename T, int EPI, int TM, int TN, typename AccRow>
__device__ __forceinline__ void vectorEpilogue(const MfmaArgs& g, T* out, const T* cin, const T* bias, int row0, int colBase,
                                               int frow, int kq, AccRow&& accRow, unsigned ldsTab = 0) {
  using Frag = typename MfmaOp<T>::Frag;
  static_assert(TM % 4 == 0 && TN % 4 == 0, "rows are handled four at a time, columns in pairs of fragments");
  const int cperm = (kq & 1) * 16 + (kq >> 1) * 8;
  auto swapPair = [](f32x4& x0, f32x4& x1) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(x0[r]), __float_as_uint(x1[r]), false, false);
      x0[r] = __uint_as_float(sw[0]);
      x1[r] = __uint_as_float(sw[1]);
    }
  };
  constexpr int kOutside = (int)0x80000000u;
  constexpr int OW = EPI == kEpiSiluMul ? 2 : 1;  // input columns per output column
  const int outCols = g.N / OW;
  const __amdgpu_buffer_rsrc_t rsOut =
      __builtin_amdgcn_make_buffer_rsrc(out, 0, (int)(((int64_t)(g.M - 1) * g.ldo + outCols) * sizeof(T)), 0x00020000);
  const int col0 = colBase / OW + cperm;  // this lane's first output column
  auto offsetOf = [&](int i, int jp, int64_t pitch) {
    const int row = row0 + i * 16 + frow, col = col0 + jp * 32;
    return row < g.M && col < outCols ? (int)(((int64_t)row * pitch + col) * sizeof(T)) : kOutside;
  };
  auto put = [&](int i, int jp, const Frag& o) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, o), rsOut, offsetOf(i, jp, g.ldo), 0, 0);
  };
  if constexpr (EPI == kEpiSiluMul) {
    // every 64 columns of a wave are one block: fragments 0, 1 are gate, 2, 3 the up values of the same 32 channels
    staticFor<TM>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      f32x4 a[TN];
      accRow(ic, a);
#pragma unroll
      for (int hb = 0; hb < TN / 4; ++hb) {
        f32x4 x0, x1;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float g0 = a[4 * hb][r], g1 = a[4 * hb + 1][r];
          x0[r] = g0 * __builtin_amdgcn_rcpf(1.f + __expf(-g0)) * a[4 * hb + 2][r];  // hardware reciprocal: an IEEE division is ten
          // instructions, 128 of them per lane and tile in a wave that nothing overlaps
          x1[r] = g1 * __builtin_amdgcn_rcpf(1.f + __expf(-g1)) * a[4 * hb + 3][r];
        }
        swapPair(x0, x1);
        Frag o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = static_cast<T>(x0[e]), o[4 + e] = static_cast<T>(x1[e]);
        put(i, hb, o);
      }
    });
  } else if constexpr (EPI == kEpiRotary || EPI == kEpiRotaryUniform || EPI == kEpiRotaryLds) {
    // A lane's 8 consecutive columns are 4 adjacent pairs of one head; their angles are 4 consecutive table
    // entries of the lane's row. Pieces at or past rotCols (the v heads) pass through with cos = 1, sin = 0.
    // the two divisors are made opaque so that the set-up of the divisions by them is done here, per call, and not
    // once per kernel with its results kept in registers across the K loop of a persistent caller
    int headDim = g.rotHeadDim, tableRows = g.rotTableRows;
    asm volatile("" : "+s"(headDim), "+s"(tableRows));
    float zero = 0.f;  // produced here for the same reason: a zero kept from before the K loop came back from scratch
    asm volatile("" : "+v"(zero));
    float bv[TN / 2][8];
    int pair0[TN / 2];
    bool rot[TN / 2];
#pragma unroll
    for (int jp = 0; jp < TN / 2; ++jp) {
      const int col = min(col0 + jp * 32, g.N - 8);
      Frag b8;
      if (bias) b8 = *reinterpret_cast<const Frag*>(bias + col);
#pragma unroll
      for (int e = 0; e < 8; ++e) bv[jp][e] = bias ? static_cast<float>(b8[e]) : zero;
      rot[jp] = col < g.rotCols;
      pair0[jp] = (col % headDim) >> 1;
    }
    const int half = headDim >> 1;
    const int tsz = g.rotTableF32 ? 4 : (int)sizeof(T);
    const __amdgpu_buffer_rsrc_t rsCos = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<void*>(g.rotCos), 0, (int)((int64_t)tableRows * half * tsz), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsSin = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<void*>(g.rotSin), 0, (int)((int64_t)tableRows * half * tsz), 0x00020000);
    // Table entries are requested four fragment rows at a time, before any store of the batch: loads and stores share
    // one in-order counter, so a request one row ahead would expose the L2 round trip once per row. (Measured on the
    // stacked QKV projection, 8192 x 4096 x 12288, same box: a ring of three rows requested two rows ahead 593.8 us,
    // this form 588.7; the same ring for the addend of the linear form is 3 us slower than its batches of four.)
    float cs[4][TN / 2][4], sn[4][TN / 2][4];
    // a wave whose columns all lie at or past rotCols (v heads) asks for no table entries at all
    const bool anyRot = __builtin_amdgcn_readfirstlane(colBase) < g.rotCols;
    if constexpr (EPI == kEpiRotaryLds) {
      // Fragment rows 0 - 3 find their entries in LDS (rotaryTablesToLds); those of rows 4 - 7 are requested now, before
      // anything is stored, and land while rows 0 - 3 are rotated and stored.
      static_assert(TM == 8, "four fragment rows from LDS, four from memory");
      bool rotU[TN / 2];
#pragma unroll
      for (int jp = 0; jp < TN / 2; ++jp) rotU[jp] = __builtin_amdgcn_readfirstlane(colBase) + jp * 32 < g.rotCols;
      const float sign = g.rotSinSign;
      u32x2 craw[4][TN / 2], sraw[4][TN / 2];
      if (anyRot) {
#pragma unroll
        for (int i = 4; i < 8; ++i) {
          const int row = row0 + i * 16 + frow;
#pragma unroll
          for (int jp = 0; jp < TN / 2; ++jp) {
            if (!rotU[jp]) continue;
            const int off = row < g.M ? ((row % tableRows) * half + pair0[jp]) * tsz : kOutside;
            craw[i - 4][jp] = __builtin_amdgcn_raw_buffer_load_b64(rsCos, off, 0, 0);
            sraw[i - 4][jp] = __builtin_amdgcn_raw_buffer_load_b64(rsSin, off, 0, 0);
          }
        }
      }
      typedef __attribute__((address_space(3))) const u32x2* LdsPair;
      const unsigned tabRow = ldsTab + (unsigned)((((row0 >> 7) & 1) * 64 + frow) * 128);
      staticFor<TM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        f32x4 a[TN];
        accRow(ic, a);
#pragma unroll
        for (int jp = 0; jp < TN / 2; ++jp) {
          f32x4 x0 = a[2 * jp], x1 = a[2 * jp + 1];
          swapPair(x0, x1);
          const float v[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
          Frag o;
          if (rotU[jp]) {
            u32x2 cr, sr;
            if constexpr (i < 4) {
              const unsigned at = tabRow + (unsigned)(i * 16 * 128 + pair0[jp] * 2);
              cr = *(LdsPair)(uintptr_t)at;
              sr = *(LdsPair)(uintptr_t)(at + 16384u);
            } else {
              cr = craw[i - 4][jp], sr = sraw[i - 4][jp];
            }
            typedef T T4 __attribute__((ext_vector_type(4)));
            const T4 c4 = __builtin_bit_cast(T4, cr), s4 = __builtin_bit_cast(T4, sr);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float c = static_cast<float>(c4[e]), sv = static_cast<float>(s4[e]) * sign;
              o[2 * e] = static_cast<T>(v[2 * e] * c - v[2 * e + 1] * sv);
              o[2 * e + 1] = static_cast<T>(v[2 * e] * sv + v[2 * e + 1] * c);
            }
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = static_cast<T>(v[e]);
          }
          put(i, jp, o);
        }
      });
    } else if constexpr (EPI == kEpiRotaryUniform) {
      // The choice per 32-column piece is a branch instead of selects in every lane, the pieces of the v heads are
      // converted and stored like a plain linear's, no zero bias is added, and the sine's sign is applied once, where the
      // table entries are converted: 52 vector instructions per 8 outputs become 36 for rotated pieces and 8 for the
      // others. (No faster for that: what the rotary epilogue waits for is its table entries, see rotaryTablesToLds.)
      bool rotU[TN / 2];
#pragma unroll
      for (int jp = 0; jp < TN / 2; ++jp) rotU[jp] = __builtin_amdgcn_readfirstlane(colBase) + jp * 32 < g.rotCols;
      const float sign = g.rotSinSign;
      auto fetchU = [&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if (!anyRot) return;
        const int row = row0 + i * 16 + frow;
#pragma unroll
        for (int jp = 0; jp < TN / 2; ++jp) {
          if (!rotU[jp]) continue;
          const int off = row < g.M ? ((row % tableRows) * half + pair0[jp]) * tsz : kOutside;
          if (g.rotTableF32) {
            const u32x4 c4 = __builtin_amdgcn_raw_buffer_load_b128(rsCos, off, 0, 0);
            const u32x4 s4 = __builtin_amdgcn_raw_buffer_load_b128(rsSin, off, 0, 0);
#pragma unroll
            for (int e = 0; e < 4; ++e) cs[i % 4][jp][e] = __uint_as_float(c4[e]), sn[i % 4][jp][e] = __uint_as_float(s4[e]) * sign;
          } else {
            typedef T T4 __attribute__((ext_vector_type(4)));
            const T4 c4 = __builtin_bit_cast(T4, __builtin_amdgcn_raw_buffer_load_b64(rsCos, off, 0, 0));
            const T4 s4 = __builtin_bit_cast(T4, __builtin_amdgcn_raw_buffer_load_b64(rsSin, off, 0, 0));
#pragma unroll
            for (int e = 0; e < 4; ++e) cs[i % 4][jp][e] = static_cast<float>(c4[e]), sn[i % 4][jp][e] = static_cast<float>(s4[e]) * sign;
          }
        }
      };
      staticFor<TM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (i % 4 == 0) {
          fetchU(std::integral_constant<int, i>{});
          fetchU(std::integral_constant<int, i + 1>{});
          fetchU(std::integral_constant<int, i + 2>{});
          fetchU(std::integral_constant<int, i + 3>{});
        }
        f32x4 a[TN];
        accRow(ic, a);
#pragma unroll
        for (int jp = 0; jp < TN / 2; ++jp) {
          f32x4 x0 = a[2 * jp], x1 = a[2 * jp + 1];
          swapPair(x0, x1);
          const float v[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
          Frag o;
          if (rotU[jp]) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float c = cs[i % 4][jp][e], sv = sn[i % 4][jp][e];
              o[2 * e] = static_cast<T>(v[2 * e] * c - v[2 * e + 1] * sv);
              o[2 * e + 1] = static_cast<T>(v[2 * e] * sv + v[2 * e + 1] * c);
            }
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = static_cast<T>(v[e]);
          }
          put(i, jp, o);
        }
      });
    } else {
    auto fetch = [&](auto ic) {
      constexpr int i = decltype(ic)::value;
      if (!anyRot) return;
      const int row = row0 + i * 16 + frow;
#pragma unroll
      for (int jp = 0; jp < TN / 2; ++jp) {
        const int off = row < g.M ? ((row % tableRows) * half + pair0[jp]) * tsz : kOutside;
        if (g.rotTableF32) {
          const u32x4 c4 = __builtin_amdgcn_raw_buffer_load_b128(rsCos, off, 0, 0);
          const u32x4 s4 = __builtin_amdgcn_raw_buffer_load_b128(rsSin, off, 0, 0);
#pragma unroll
          for (int e = 0; e < 4; ++e) cs[i % 4][jp][e] = __uint_as_float(c4[e]), sn[i % 4][jp][e] = __uint_as_float(s4[e]);
        } else {
          typedef T T4 __attribute__((ext_vector_type(4)));
          const T4 c4 = __builtin_bit_cast(T4, __builtin_amdgcn_raw_buffer_load_b64(rsCos, off, 0, 0));
          const T4 s4 = __builtin_bit_cast(T4, __builtin_amdgcn_raw_buffer_load_b64(rsSin, off, 0, 0));
#pragma unroll
          for (int e = 0; e < 4; ++e) cs[i % 4][jp][e] = static_cast<float>(c4[e]), sn[i % 4][jp][e] = static_cast<float>(s4[e]);
        }
      }
    };
    staticFor<TM>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      if constexpr (i % 4 == 0) {
        fetch(std::integral_constant<int, i>{});
        fetch(std::integral_constant<int, i + 1>{});
        fetch(std::integral_constant<int, i + 2>{});
        fetch(std::integral_constant<int, i + 3>{});
      }
      f32x4 a[TN];
      accRow(ic, a);
#pragma unroll
      for (int jp = 0; jp < TN / 2; ++jp) {
        f32x4 x0 = a[2 * jp], x1 = a[2 * jp + 1];
        swapPair(x0, x1);
        const float v[8] = {x0[0] + bv[jp][0], x0[1] + bv[jp][1], x0[2] + bv[jp][2], x0[3] + bv[jp][3],
                            x1[0] + bv[jp][4], x1[1] + bv[jp][5], x1[2] + bv[jp][6], x1[3] + bv[jp][7]};
        Frag o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float c = rot[jp] ? cs[i % 4][jp][e] : 1.f;
          const float sv = rot[jp] ? sn[i % 4][jp][e] * g.rotSinSign : 0.f;
          o[2 * e] = static_cast<T>(v[2 * e] * c - v[2 * e + 1] * sv);
          o[2 * e + 1] = static_cast<T>(v[2 * e] * sv + v[2 * e + 1] * c);
        }
        put(i, jp, o);
      }
    });
    }
  } else if constexpr (EPI == kEpiColScale) {
    float sv[TN / 2][8], bv[TN / 2][8];
#pragma unroll
    for (int jp = 0; jp < TN / 2; ++jp) {
      const int col = min(col0 + jp * 32, g.N - 8);  // N % 8 == 0 here; a clamped piece is never stored
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        sv[jp][e] = loadAs<float>(g.colScale, col + e, g.colScaleDtype) * g.alpha;
        bv[jp][e] = g.colBias ? loadAs<float>(g.colBias, col + e, g.colBiasDtype) : 0.f;
      }
    }
    staticFor<TM>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      f32x4 a[TN];
      accRow(ic, a);
#pragma unroll
      for (int jp = 0; jp < TN / 2; ++jp) {
        f32x4 x0 = a[2 * jp], x1 = a[2 * jp + 1];
        swapPair(x0, x1);
        const float v[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        Frag o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = static_cast<T>(v[e] * sv[jp][e] + bv[jp][e]);
        put(i, jp, o);
      }
    });
  } else if constexpr (EPI == kEpiAddendLds) {
    // ldsTab is this wave's own 8 KiB: the addend of fragment rows 0 and 1 (addendToLds). The pieces of rows 2 - 7 are
    // requested now, before anything is stored, and land while rows 0 and 1 are worked through.
    static_assert(TM == 8 && TN == 8, "two fragment rows from LDS, six from memory, 128 columns per wave");
    float zero = 0.f;  // (produced here: a zero kept from before the K loop would occupy a register across it)
    asm volatile("" : "+v"(zero));
    float bv[TN / 2][8];
#pragma unroll
    for (int jp = 0; jp < TN / 2; ++jp) {
      const int col = min(col0 + jp * 32, g.N - 8);
      Frag b8;
      if (bias) b8 = *reinterpret_cast<const Frag*>(bias + col);
#pragma unroll
      for (int e = 0; e < 8; ++e) bv[jp][e] = bias ? static_cast<float>(b8[e]) : zero;
    }
    const __amdgpu_buffer_rsrc_t rsC = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T*>(cin), 0, (int)(((int64_t)(g.M - 1) * g.sCm + g.N) * sizeof(T)), 0x00020000);
    u32x4 cv[TM - 2][TN / 2];
#pragma unroll
    for (int i = 2; i < TM; ++i) {
#pragma unroll
      for (int jp = 0; jp < TN / 2; ++jp) cv[i - 2][jp] = __builtin_amdgcn_raw_buffer_load_b128(rsC, offsetOf(i, jp, g.sCm), 0, 0);
    }
    typedef __attribute__((address_space(3))) const u32x4* LdsQuad;
    const unsigned ldsRow = ldsTab + (unsigned)frow * 256u;
    const int piece0 = (kq & 1) * 2 + (kq >> 1);  // this lane's 8 columns of a 32-column pair, as a piece index
    staticFor<TM>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      f32x4 a[TN];
      accRow(ic, a);
#pragma unroll
      for (int jp = 0; jp < TN / 2; ++jp) {
        f32x4 x0 = a[2 * jp], x1 = a[2 * jp + 1];
        swapPair(x0, x1);
        const float v[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        u32x4 craw;
        if constexpr (i < 2)
          craw = *(LdsQuad)(uintptr_t)(ldsRow + (unsigned)(i * 16 * 256) + (unsigned)(((piece0 + 4 * jp) ^ frow) << 4));
        else
          craw = cv[i - 2][jp];
        const Frag c8 = __builtin_bit_cast(Frag, craw);
        Frag o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float x = v[e] * g.alpha + bv[jp][e];
          x += g.beta * static_cast<float>(c8[e]);
          o[e] = static_cast<T>(x);
        }
        put(i, jp, o);
      }
    });
  } else {
    float bv[TN / 2][8];
#pragma unroll
    for (int jp = 0; jp < TN / 2; ++jp) {
      const int col = min(col0 + jp * 32, g.N - 8);  // N % 8 == 0 here; a clamped piece is never stored
      Frag b8;
      if (bias) b8 = *reinterpret_cast<const Frag*>(bias + col);
#pragma unroll
      for (int e = 0; e < 8; ++e) bv[jp][e] = bias ? static_cast<float>(b8[e]) : 0.f;
    }
    auto store = [&](auto withAddend) {
      constexpr bool kAddend = decltype(withAddend)::value;
      const __amdgpu_buffer_rsrc_t rsC = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<T*>(kAddend ? cin : out), 0, (int)(((int64_t)(g.M - 1) * g.sCm + g.N) * sizeof(T)), 0x00020000);
      u32x4 cv[4][TN / 2];
      auto fetch = [&](int i) {
#pragma unroll
        for (int jp = 0; jp < TN / 2; ++jp) cv[i & 3][jp] = __builtin_amdgcn_raw_buffer_load_b128(rsC, offsetOf(i, jp, g.sCm), 0, 0);
      };
      staticFor<TM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (kAddend && i % 4 == 0) {
#pragma unroll
          for (int ii = i; ii < i + 4; ++ii) fetch(ii);
        }
        f32x4 a[TN];
        accRow(ic, a);
#pragma unroll
        for (int jp = 0; jp < TN / 2; ++jp) {
          f32x4 x0 = a[2 * jp], x1 = a[2 * jp + 1];
          swapPair(x0, x1);
          const float v[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
          Frag o, c8;
          if constexpr (kAddend) c8 = __builtin_bit_cast(Frag, cv[i & 3][jp]);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            float x = v[e] * g.alpha + bv[jp][e];
            if constexpr (kAddend) x += g.beta * static_cast<float>(c8[e]);
            o[e] = static_cast<T>(x);
          }
          put(i, jp, o);
        }
      });
    };
    if (cin)
      store(std::true_type{});
    else
      store(std::false_type{});
  }
}


// TILE is the edge of the square macro tile: 256 (8 waves, 2 x 4, wave tile 128 x 64) or 128 (4 waves, 2 x 2, wave
// tile 64 x 64, 64 KiB of LDS, two workgroups per CU) for problems with too few 256 x 256 tiles to fill the chip:
// the same pipeline with half as many A fragments per phase.
//
// BT: the second operand lies in memory as [K, N] with N contiguous (the right-hand side of mm / bmm / matmul as the
// caller holds it) and is used in place. Its tile is copied as it lies, 64 rows of TILE columns, and the fragment a
// lane needs (8 consecutive k of one column) comes out of two transposing LDS reads (ds_read_b64_tr_b16: the 16 lanes
// of a group each point at 4 consecutive columns of one of 4 consecutive k rows, and lane i receives those 4 rows'
// values of column i). The 32-byte pieces of row k are XOR-swizzled with (k & 3) | 4 (k >> 3 & 1), which puts the 8
// row pieces one half-wave touches (k .. k + 3 and k + 8 .. k + 11) on 8 different bank groups. g.ldb is then the
// stride between k rows.
template <typename T, int EPI, int TILE = 256, bool BT = false>
__global__ __launch_bounds__(TILE == 256 ? kPipeThreads : 256, TILE == 256 ? 1 : 2) void gemmMfmaPipelinedKernel(MfmaArgs g) {
  using Frag = typename MfmaOp<T>::Frag;
  constexpr int kWavesN = TILE == 256 ? kPipeWavesN : 2, kThreads = TILE == 256 ? kPipeThreads : 256;
  constexpr int BM = TILE, BN = TILE, WM = BM / kPipeWavesM, WN = BN / kWavesN, TM = WM / 16, TN = WN / 16;
  constexpr int HM = TM / 2;                 // A fragments of one phase (half of the wave's rows)
  constexpr int CH = BM * 8 / kThreads;      // 16-byte chunks per thread per operand tile
  constexpr int RS = kThreads / 8;           // rows covered by one pass of the workgroup
  static_assert((HM == 4 || HM == 2) && TN == 4 && CH == 4, "the phase schedule below is written for 4 (or 2) x 4 fragments");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* sA = reinterpret_cast<T*>(smem);  // [2][BM][64]
  T* sB = sA + 2 * BM * kBK;           // [2][BN][64]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / kWavesN, wn = wave % kWavesN;
  int tm, tn;
  {
    const int total = g.tilesM * g.tilesN;
    const int pid = blockIdx.x;
    const int xcd = pid & 7, idx = pid >> 3;
    const int q = total >> 3, r = total & 7;
    const int logical = xcd * q + min(xcd, r) + idx;
    constexpr int GROUP = 8;
    const int width = GROUP * g.tilesN;
    const int group = logical / width;
    const int first = group * GROUP;
    const int gsize = min(g.tilesM - first, GROUP);
    const int in = logical - group * width;
    tm = first + in % gsize;
    tn = in / gsize;
  }
  const int batch = blockIdx.z;
  // split-K: this workgroup's K range starts kFirst tiles in (0 otherwise); the operands are simply entered there
  const int kFirst = EPI == kEpiPartial ? (int)blockIdx.y * g.kTilesPerSplit : 0;
  const T* A = reinterpret_cast<const T*>(g.A) + (int64_t)batch * g.sAb + kFirst * kBK;
  const T* B = reinterpret_cast<const T*>(g.B) + (int64_t)batch * g.sBb + (BT ? (int64_t)kFirst * kBK * g.ldb : (int64_t)kFirst * kBK);
  // Operand tiles go from memory straight into LDS: lane l of a wave fills the l-th 16-byte slot of a
  // 1 KiB block (8 rows of 128 bytes), so the chunk swizzle is applied on the global side: the lane
  // that owns physical slot (row, c) fetches logical chunk c ^ ((row >> 1) & 7). A 32-bit per-lane
  // byte offset is fixed for the whole K loop and a scalar K offset moves per tile; rows past M / N
  // are clamped to the last row (their products are never stored).
  // (The host guarantees both operands span less than 2 GiB.)
  auto descriptor = [](const T* base, int64_t bytes) {
    const uint64_t p = reinterpret_cast<uint64_t>(base);
    u32x4 d = {(uint32_t)p, (uint32_t)(p >> 32) & 0xffffu, (uint32_t)bytes, 0x00020000u};
    return d;
  };
  const u32x4 rsA = descriptor(A, ((int64_t)(g.M - 1) * g.lda + g.K - kFirst * kBK) * 2);
  const u32x4 rsB = BT ? descriptor(B, ((int64_t)(g.K - kFirst * kBK - 1) * g.ldb + g.N) * 2)
                       : descriptor(B, ((int64_t)(g.N - 1) * g.ldb + g.K - kFirst * kBK) * 2);
  int aOffG[CH], bOffG[CH];
  const int srow = tid >> 3;  // staging row of chunk 0; chunk i is RS rows further (same swizzle)
  const int c8 = ((tid & 7) ^ ((srow >> 1) & 7)) * 8;
  constexpr int CPRT = BN / 8;         // [K, N] layout: 16-byte chunks per k row of the tile
  constexpr int RST = kThreads / CPRT;  // and k rows covered by one pass of the workgroup
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    aOffG[i] = (int)(((int64_t)min(tm * BM + srow + RS * i, g.M - 1) * g.lda + c8) * 2);
    if constexpr (BT) {
      // the thread owns physical slot (k row, chunk) of the tile as it lies and fetches the logical chunk the swizzle
      // puts there; columns past N read the next row or zeros and only reach output columns that are never stored
      const int krow = tid / CPRT + RST * i, chunk = (tid % CPRT) ^ (2 * ((krow & 3) | (((krow >> 3) & 1) << 2)));
      bOffG[i] = (int)(((int64_t)krow * g.ldb + tn * BN + chunk * 8) * 2);
    } else {
      bOffG[i] = (int)(((int64_t)min(tn * BN + srow + RS * i, g.N - 1) * g.ldb + c8) * 2);
    }
  }
  // LDS byte address of this wave's 1 KiB block in stage 0 of A; stage 1 is kStageBytes further, B 2 * kStageBytes
  constexpr unsigned kStageBytes = BM * kBK * sizeof(T), kPassBytes = RS * kBK * sizeof(T);
  const unsigned ldsWave = (unsigned)(size_t)(__attribute__((address_space(3))) char*)smem +
                           __builtin_amdgcn_readfirstlane(wave) * 1024u;
  const int nK = EPI == kEpiPartial ? min(g.kTilesPerSplit, g.K / kBK - kFirst) : g.K / kBK;

  const int frow = lane & 15, kq = lane >> 4;
  const int swz = (frow >> 1) & 7;  // fragment rows are 16 apart: they all share this lane's swizzle
  int kx[2];                        // swizzled element offset of this lane's chunk for each 32-wide k-step
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) kx[ks] = ((4 * ks + kq) ^ swz) << 3;
  const int aBase = (wm * WM + frow) * kBK, bBase = (wn * WN + frow) * kBK;

  Frag fa[2][HM], fb[TN];
  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

  auto dmaA = [&](int stage, int kt, int i) {
    loadToLds16(rsA, aOffG[i], kt * kBK * (int)sizeof(T), ldsWave + stage * kStageBytes + i * kPassBytes);
  };
  const int bTileStep = BT ? kBK * (int)g.ldb * (int)sizeof(T) : kBK * (int)sizeof(T);  // bytes from one K tile to the next
  auto dmaB = [&](int stage, int kt, int i) {
    loadToLds16(rsB, bOffG[i], kt * bTileStep, ldsWave + (2 + stage) * kStageBytes + i * kPassBytes);
  };
  auto loadA = [&](int stage, int ks, int half, int buf, int i) {
    fa[buf][i] = *reinterpret_cast<const Frag*>(sA + stage * BM * kBK + aBase + kx[ks] + (half * HM + i) * 16 * kBK);
  };
  // [K, N] layout: byte offset of this lane's piece for fragment j within a k row, swizzle applied (the swizzle
  // depends on k & 3 and k >> 3 & 1, which the lane fixes: k = 32 ks + 8 kq + 4 r + (lane & 15) / 4)
  int btCol[TN];
  const int btRow = kq * 8 + (frow >> 2);
  if constexpr (BT) {
    const int sw2 = 2 * ((frow >> 2) | ((kq & 1) << 2));
#pragma unroll
    for (int j = 0; j < TN; ++j) btCol[j] = ((((wn * WN + j * 16) >> 3) + ((lane & 3) >> 1)) ^ sw2) * 16 + (lane & 1) * 8;
  }
  auto loadB = [&](int stage, int ks, int j) {
    if constexpr (BT) {
      typedef typename MfmaOp<T>::Half HalfFrag;
      typedef __attribute__((address_space(3))) s16x4* LdsTr;
      const unsigned at = (unsigned)(size_t)(__attribute__((address_space(3))) char*)smem + (2 + stage) * kStageBytes +
                          (unsigned)((ks * 32 + btRow) * BN * (int)sizeof(T) + btCol[j]);
      const HalfFrag lo = __builtin_bit_cast(HalfFrag, __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsTr)(uintptr_t)at));
      const HalfFrag hi = __builtin_bit_cast(HalfFrag, __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsTr)(uintptr_t)(at + 4 * BN * (unsigned)sizeof(T))));
      Frag f;
      f[0] = lo[0], f[1] = lo[1], f[2] = lo[2], f[3] = lo[3], f[4] = hi[0], f[5] = hi[1], f[6] = hi[2], f[7] = hi[3];
      fb[j] = f;
    } else {
      fb[j] = *reinterpret_cast<const Frag*>(sB + stage * BN * kBK + bBase + kx[ks] + j * 16 * kBK);
    }
  };
  // One phase = 16 MFMAs: half of the wave's rows (4 A fragments) against its 4 B fragments for
  // one 32-wide k-step, B-major in four groups of four. B fragment j is dead after group j and is
  // refilled in place for the next k-step; the A fragments of the next phase arrive in the other
  // register buffer during the first two groups. Every group is fenced so the order holds.
  auto phase = [&](int half, int buf, auto&& before, auto&& after) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      before(j);
#pragma unroll
      for (int i = 0; i < HM; ++i)
        acc[half * HM + i][j] = MfmaOp16<T>::run(fb[j], fa[buf][i], acc[half * HM + i][j]);
      after(j);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // Publishes a stage: this wave's loads into it have landed (vmcnt) and its fragment reads of the
  // stage about to be refilled are done (lgkmcnt), then all waves meet.
  auto publish = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0070);
    __builtin_amdgcn_s_barrier();
  };

#pragma unroll
  for (int i = 0; i < CH; ++i) dmaA(0, 0, i);
#pragma unroll
  for (int i = 0; i < CH; ++i) dmaB(0, 0, i);
  publish();
#pragma unroll
  for (int i = 0; i < CH; ++i) dmaA(1, 1, i);  // the B half of tile 1 goes out in phase 0 below
#pragma unroll
  for (int j = 0; j < TN; ++j) loadB(0, 0, j);
#pragma unroll
  for (int i = 0; i < HM; ++i) loadA(0, 0, 0, 0, i);

  // Iteration kt multiplies tile kt out of stage kt & 1 while tile kt + 1 lands in the other stage. Once
  // every wave has passed the barrier before phase 3 nobody reads this stage any more, so the A half of
  // tile kt + 2 is loaded into it right there and the B half in phase 0 of the next iteration: one load
  // per group of four MFMAs (all eight in one phase measured 1-4 % slower, all in phases 0-1 up to 7 %).
  auto iter = [&](auto hasNext, auto hasNext2, int kt) {
    constexpr bool kNext = decltype(hasNext)::value, kNext2 = decltype(hasNext2)::value;
    const int cur = kt & 1;
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase 0: k-step 0, rows 0-63 | A fragments of phase 1 | B half of the next tile
    phase(0, 0,
          [&](int j) {
            if (j < HM / 2) {
              loadA(cur, 0, 1, 1, 2 * j);
              loadA(cur, 0, 1, 1, 2 * j + 1);
            }
          },
          [&](int j) {
            if constexpr (kNext) dmaB(cur ^ 1, kt + 1, j);
          });
    // ---- phase 1: k-step 0, rows 64-127 | A of phase 2, B of k-step 1
    phase(1, 1,
          [&](int j) {
            if (j < HM / 2) {
              loadA(cur, 1, 0, 0, 2 * j);
              loadA(cur, 1, 0, 0, 2 * j + 1);
            }
          },
          [&](int j) { loadB(cur, 1, j); });
    // ---- phase 2: k-step 1, rows 0-63 | A of phase 3
    phase(0, 0,
          [&](int j) {
            if (j < HM / 2) {
              loadA(cur, 1, 1, 1, 2 * j);
              loadA(cur, 1, 1, 1, 2 * j + 1);
            }
          },
          [&](int) {});
    if constexpr (kNext) publish();
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase 3: k-step 1, rows 64-127 | A and B of phase 0 of the next tile | A half of tile kt + 2
    phase(1, 1,
          [&](int j) {
            if constexpr (kNext2) dmaA(cur, kt + 2, j);
            if constexpr (kNext) {
              if (j < HM / 2) {
                loadA(cur ^ 1, 0, 0, 0, 2 * j);
                loadA(cur ^ 1, 0, 0, 0, 2 * j + 1);
              }
            }
          },
          [&](int j) {
            if constexpr (kNext) loadB(cur ^ 1, 0, j);
          });
  };
  using std::false_type;
  using std::true_type;
  for (int kt = 0; kt < nK - 2; ++kt) iter(true_type{}, true_type{}, kt);
  iter(true_type{}, false_type{}, nK - 2);
  iter(false_type{}, false_type{}, nK - 1);

  // ---- epilogue
  if constexpr (EPI == kEpiPartial) {
    // the accumulators as they are: a lane holds 4 consecutive fp32 columns of one row per fragment, one 16-byte
    // store each; pieces outside the matrix get an offset past the end of the buffer and are dropped
    float* part = g.partial + (int64_t)blockIdx.y * g.M * g.N;
    const __amdgpu_buffer_rsrc_t rsP = __builtin_amdgcn_make_buffer_rsrc(part, 0, (int)((int64_t)g.M * g.N * 4), 0x00020000);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = tm * BM + wm * WM + i * 16 + frow;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = tn * BN + wn * WN + j * 16 + kq * 4;
        const int off = row < g.M && col < g.N ? (int)(((int64_t)row * g.N + col) * 4) : (int)0x80000000u;
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[i][j]), rsP, off, 0, 0);
      }
    }
    return;
  }
  T* out = reinterpret_cast<T*>(g.out) + (int64_t)batch * g.sOb;
  const T* cin = g.Cin ? reinterpret_cast<const T*>(g.Cin) + (int64_t)batch * g.sCb : nullptr;
  const T* bias = reinterpret_cast<const T*>(g.bias);
  if (g.vecEpilogue) {
    // The lane's position is made opaque here: otherwise every lane-dependent value of the epilogue that does not depend
    // on the tile is hoisted out of the persistent loop, has to stay live across the K loop, whose text owns v120-v247,
    // and is spilled (13 registers in the rotary form, reloaded behind the K loop's tile loads).
    int efrow = frow, ekq = kq;
    asm volatile("" : "+v"(efrow), "+v"(ekq));
    vectorEpilogue<T, EPI, TM, TN>(g, out, cin, bias, tm * BM + wm * WM, tn * BN + wn * WN, efrow, ekq, [&](auto ic, f32x4(&row)[TN]) {
#pragma unroll
      for (int j = 0; j < TN; ++j) row[j] = acc[decltype(ic)::value][j];
    });
    return;
  }
  // element-wise stores for outputs that do not allow 16-byte pieces; the addend of a fragment row is
  // requested before the row's first store, for the reason given above
  auto storeScalar = [&](auto withAddend) {
    constexpr bool kAddend = decltype(withAddend)::value;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = tm * BM + wm * WM + i * 16 + frow;
      if (row >= g.M) continue;
      float c[TN][4];
      if constexpr (kAddend) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int col = min(tn * BN + wn * WN + j * 16 + kq * 4 + r, g.N - 1);
            c[j][r] = static_cast<float>(cin[(int64_t)row * g.sCm + (int64_t)col * g.sCn]);
          }
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int col = tn * BN + wn * WN + j * 16 + kq * 4 + r;
          if (col < g.N) {
            float v = acc[i][j][r] * g.alpha + (bias ? static_cast<float>(bias[col]) : 0.f);
            if constexpr (kAddend) v += g.beta * c[j][r];
            out[(int64_t)row * g.ldo + col] = static_cast<T>(v);
          }
        }
      }
    }
  };
  if (cin)
    storeScalar(std::true_type{});
  else
    storeScalar(std::false_type{});
}


// ------------------------------------------------------- 4 waves, hand-placed K loop ---
// The same 256 x 256 x 64 macro tile with 4 waves (2 x 2, wave tile 128 x 128 = 8 x 8 tiles of
// v_mfma_f32_16x16x32, 256 accumulators per lane in the accumulation registers): a third fewer LDS fragment reads per
// MFMA than the 8-wave form (16 per 64 instead of 12 per 32), which is what the kernel pays for in clock at the power
// limit. One wave per SIMD means that nothing hides a stall, so the K loop is generated text (gemm_loop_4wave.inc,
// written by gen_gemm_loop_4wave.py, which documents the schedule): tile loads straight into a two-stage LDS ring,
// fragment reads one k-step ahead into fixed registers, one barrier per K tile. Needs an even number of K tiles and
// the vector epilogue; everything else stays with the 8-wave kernel.
//
// Invariant the compiler does not check: between the PROLOGUE, BODY and TAIL statements, and from the TAIL to the last
// accRegisters16 read of the epilogue, a0-a255 (the accumulators) and v120-v247 (operand fragments read ahead) are
// live, but to the compiler they are only clobbers of each statement. The code in between (tile arithmetic, lane
// offsets, the epilogue's conversions and address arithmetic) must therefore fit the other 128 ordinary registers
// and touch no accumulation register, and nothing may spill: a reload would also stall behind the tile loads in
// flight. build.py compiles this file with the resource-usage remark and fails when any instantiation reports
// scratch or spilled vector registers; tests/test_gpu_attention_gemm.py runs every instantiation by name on exact inputs.
#include "gemm_loop_4wave.inc"

// Sixteen consecutive accumulation registers a[R .. R + 15] as four fragments, in one statement: the reads issue back
// to back, and what follows is ordinary code the compiler may schedule freely (one statement per register would pin
// every read between its neighbours' dependent arithmetic, which a lone wave per SIMD cannot hide).
template <int R>
__device__ __forceinline__ void accRegisters16(f32x4 (&f)[4]) {
  float v[16];
  asm volatile(
      "v_accvgpr_read_b32 %0, a[%16:%16]\n\tv_accvgpr_read_b32 %1, a[%17:%17]\n\tv_accvgpr_read_b32 %2, a[%18:%18]\n\t"
      "v_accvgpr_read_b32 %3, a[%19:%19]\n\tv_accvgpr_read_b32 %4, a[%20:%20]\n\tv_accvgpr_read_b32 %5, a[%21:%21]\n\t"
      "v_accvgpr_read_b32 %6, a[%22:%22]\n\tv_accvgpr_read_b32 %7, a[%23:%23]\n\tv_accvgpr_read_b32 %8, a[%24:%24]\n\t"
      "v_accvgpr_read_b32 %9, a[%25:%25]\n\tv_accvgpr_read_b32 %10, a[%26:%26]\n\tv_accvgpr_read_b32 %11, a[%27:%27]\n\t"
      "v_accvgpr_read_b32 %12, a[%28:%28]\n\tv_accvgpr_read_b32 %13, a[%29:%29]\n\tv_accvgpr_read_b32 %14, a[%30:%30]\n\t"
      "v_accvgpr_read_b32 %15, a[%31:%31]"
      : "=v"(v[0]), "=v"(v[1]), "=v"(v[2]), "=v"(v[3]), "=v"(v[4]), "=v"(v[5]), "=v"(v[6]), "=v"(v[7]), "=v"(v[8]), "=v"(v[9]),
        "=v"(v[10]), "=v"(v[11]), "=v"(v[12]), "=v"(v[13]), "=v"(v[14]), "=v"(v[15])
      : "n"(R), "n"(R + 1), "n"(R + 2), "n"(R + 3), "n"(R + 4), "n"(R + 5), "n"(R + 6), "n"(R + 7), "n"(R + 8), "n"(R + 9),
        "n"(R + 10), "n"(R + 11), "n"(R + 12), "n"(R + 13), "n"(R + 14), "n"(R + 15));
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int r = 0; r < 4; ++r) f[q][r] = v[4 * q + r];
}

template <typename T, int EPI>
__global__ __launch_bounds__(256) void gemmMfma4WaveKernel(MfmaArgs g) {
  constexpr int BM = 256, BN = 256, WM = 128, WN = 128, TM = 8, TN = 8;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int total = g.tilesM * g.tilesN;
  // Persistent: the workgroup takes output tiles blockIdx.x, blockIdx.x + gridDim.x, ... (the grid is a multiple of
  // 8 or covers every tile, so a workgroup's tiles all belong to the XCD it runs on, as in the one-tile-per-workgroup
  // order). XCD x works on a contiguous band of tiles, walked in groups of 8 tile rows.
  auto tileOf = [&](int pid, int& tm, int& tn) {
    const int xcd = pid & 7, idx = pid >> 3;
    const int q = total >> 3, r = total & 7;
    const int logical = xcd * q + min(xcd, r) + idx;
    constexpr int GROUP = 8;
    const int width = GROUP * g.tilesN;
    const int group = logical / width;
    const int first = group * GROUP;
    const int gsize = min(g.tilesM - first, GROUP);
    const int in = logical - group * width;
    tm = first + in % gsize;
    tn = in / gsize;
  };
  const int batch = blockIdx.z;
  const T* A = reinterpret_cast<const T*>(g.A) + (int64_t)batch * g.sAb;
  const T* B = reinterpret_cast<const T*>(g.B) + (int64_t)batch * g.sBb;
  // Rows past M / N and columns past K lie beyond the descriptors' extent and read as zeros.
  auto descriptor = [](const T* base, int64_t bytes) {
    const uint64_t p = reinterpret_cast<uint64_t>(base);
    u32x4 d = {(uint32_t)p, (uint32_t)(p >> 32) & 0xffffu, (uint32_t)bytes, 0x00020000u};
    return d;
  };
  const u32x4 rsA = descriptor(A, ((int64_t)(g.M - 1) * g.lda + g.K) * 2);
  const u32x4 rsB = descriptor(B, ((int64_t)(g.N - 1) * g.ldb + g.K) * 2);
  // lane l of a wave fills the l-th 16-byte slot of a 1 KiB block (8 rows of 128 bytes); the chunk swizzle
  // c ^ ((row >> 1) & 7) is applied to the global address. A pass of the workgroup covers 32 rows.
  constexpr unsigned kFar = 0x80000000u;  // beyond every extent: the load returns zeros
  const int waveS = __builtin_amdgcn_readfirstlane(wave);
  // this lane's number within the wave, asked of the hardware each time (volatile: neither hoisted nor shared)
  auto laneNow = []() {
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
  };
  unsigned voA[8], voB[8];
  auto laneOffsets = [&](int tm, int tn) {
    // recomputed on every call from the lane number the hardware hands out: the eight row numbers and the chunk
    // offset (or the thread index they come from) would otherwise be kept live across the K loop, whose text owns
    // v120-v247, and spilled; a reload between two pieces of that text waits for every tile load in flight (loads
    // return in order)
    const int t = waveS * 64 + laneNow();
    const int srow = t >> 3;
    const int c8 = ((t & 7) ^ ((srow >> 1) & 7)) * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int ra = tm * BM + srow + 32 * i, rb = tn * BN + srow + 32 * i;
      voA[i] = ra < g.M ? (unsigned)(((int64_t)ra * g.lda + c8) * 2) : kFar;
      voB[i] = rb < g.N ? (unsigned)(((int64_t)rb * g.ldb + c8) * 2) : kFar;
    }
  };
  const unsigned base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)smem;
  const unsigned ldsWave = base + __builtin_amdgcn_readfirstlane(wave) * 1024u;
  const int frow = lane & 15, kq = lane >> 4, swz = (frow >> 1) & 7;
  const unsigned adA0 = base + ((wm * WM + frow) * kBK + ((kq ^ swz) << 3)) * 2;
  const unsigned adA1 = base + ((wm * WM + frow) * kBK + (((4 + kq) ^ swz) << 3)) * 2;
  const unsigned adB0 = base + 65536 + ((wn * WN + frow) * kBK + ((kq ^ swz) << 3)) * 2;
  const unsigned adB1 = base + 65536 + ((wn * WN + frow) * kBK + (((4 + kq) ^ swz) << 3)) * 2;
  const int pairs = g.K / (2 * kBK);
  unsigned kcur = 0, m0s = 0;
  T* out = reinterpret_cast<T*>(g.out) + (int64_t)batch * g.sOb;
  const T* cin = g.Cin ? reinterpret_cast<const T*>(g.Cin) + (int64_t)batch * g.sCb : nullptr;
  const T* bias = reinterpret_cast<const T*>(g.bias);
#define GEMM4W_OPERANDS                                                                                              \
  : [kcur] "+s"(kcur), [m0s] "+s"(m0s)                                                                               \
  : [voA0] "v"(voA[0]), [voA1] "v"(voA[1]), [voA2] "v"(voA[2]), [voA3] "v"(voA[3]), [voA4] "v"(voA[4]),              \
    [voA5] "v"(voA[5]), [voA6] "v"(voA[6]), [voA7] "v"(voA[7]), [voB0] "v"(voB[0]), [voB1] "v"(voB[1]),              \
    [voB2] "v"(voB[2]), [voB3] "v"(voB[3]), [voB4] "v"(voB[4]), [voB5] "v"(voB[5]), [voB6] "v"(voB[6]),              \
    [voB7] "v"(voB[7]), [adA0] "v"(adA0), [adA1] "v"(adA1), [adB0] "v"(adB0), [adB1] "v"(adB1), [rsA] "s"(rsA),      \
    [rsB] "s"(rsB), [lds] "s"(ldsWave)                                                                               \
  : "memory", "scc", GEMM4W_CLOBBERS
#define GEMM4W_RUN(NAME)                                                         \
  do {                                                                           \
    if constexpr (std::is_same<T, bf16_t>::value)                                \
      asm volatile(GEMM4W_##NAME##_BF16 GEMM4W_OPERANDS);                        \
    else                                                                         \
      asm volatile(GEMM4W_##NAME##_F16 GEMM4W_OPERANDS);                         \
  } while (0)
  int pid = blockIdx.x, tm, tn;
  tileOf(pid, tm, tn);
  laneOffsets(tm, tn);
  bool first = true;
  while (true) {
    if (first)
      GEMM4W_RUN(PROLOGUE);
    else
      GEMM4W_RUN(PROLOGUE_LOADED);
    for (int p = 1; p < pairs; ++p) GEMM4W_RUN(BODY);
    // (rotary tables through LDS: this output tile's entries are copied now, behind every tile load of its K loop; tiles
    // of v heads need none; the decision is the same for the whole workgroup)
    if constexpr (EPI == kEpiRotaryLds) {
      if (tn * BN < g.rotCols) rotaryTablesToLds<T>(g, tm * BM, waveS, laneNow(), base + 131072u);
    }
    // (addend through LDS: every wave copies the addend of its own first two fragment rows, likewise behind the tile loads)
    if constexpr (EPI == kEpiAddendLds)
      addendToLds<T>(g, cin, tm * BM + (waveS >> 1) * WM, tn * BN + (waveS & 1) * WN, laneNow(), base + 131072u + (unsigned)waveS * 8192u);
    const int next = pid + (int)gridDim.x;
    int ntm = 0, ntn = 0;
    if (next < total) {
      // the last K tile also issues the first loads of the next output tile: they land while the epilogue runs
      tileOf(next, ntm, ntn);
      laneOffsets(ntm, ntn);
      GEMM4W_RUN(TAIL_NEXT);
    } else {
      GEMM4W_RUN(TAIL);
    }
    if constexpr (EPI == kEpiRotaryLds) {
      if (tn * BN < g.rotCols) {
        // this wave's table copies are older than the 32 tile loads the tail issued for the next output tile (if any)
        if (next < total) __builtin_amdgcn_s_waitcnt(0x0f70 | (32 & 15) | ((32 >> 4) << 14));
        else __builtin_amdgcn_s_waitcnt(0x0f70);
        __builtin_amdgcn_s_barrier();
      }
    }
    if constexpr (EPI == kEpiAddendLds) {
      // (a wave reads back only its own copies: no barrier)
      if (next < total) __builtin_amdgcn_s_waitcnt(0x0f70 | (32 & 15) | ((32 >> 4) << 14));
      else __builtin_amdgcn_s_waitcnt(0x0f70);
    }
    // one fragment row at a time out of the accumulation registers, which the compiler does not know to be live:
    // the epilogue stays far below the 256 ordinary registers, so it never borrows them
    // The lane's position is asked for again here: otherwise every lane-dependent value of the epilogue that does not
    // depend on the tile is hoisted out of the persistent loop, has to stay live across the K loop, and is spilled
    // (13 registers in the rotary form, reloaded behind the tile loads already issued for the next output tile).
    const int elane = laneNow(), efrow = elane & 15, ekq = elane >> 4;
    vectorEpilogue<T, EPI, TM, TN>(g, out, cin, bias, tm * BM + (waveS >> 1) * WM, tn * BN + (waveS & 1) * WN, efrow, ekq, [&](auto ic, f32x4(&row)[TN]) {
      constexpr int i = decltype(ic)::value;
      f32x4 lo[4], hi[4];
      accRegisters16<32 * i>(lo);
      accRegisters16<32 * i + 16>(hi);
#pragma unroll
      for (int j = 0; j < 4; ++j) row[j] = lo[j], row[4 + j] = hi[j];
    }, base + 131072u + (EPI == kEpiAddendLds ? (unsigned)waveS * 8192u : 0u));
    if (next >= total) break;
    pid = next, tm = ntm, tn = ntn, first = false;
  }
#undef GEMM4W_RUN
#undef GEMM4W_OPERANDS
}

// ------------------------------------------------------------ skinny M (decode) ---
// At most 64 activation rows against a large K-contiguous weight: the weight matrix is the only traffic
// that matters and is streamed exactly once. Laid out like the int8 weight-only kernel:
//   * a workgroup owns NTW tiles of 16 output columns; the KS waves of a tile split K between them and their
//     fp32 partial sums meet in LDS. NTW * KS is 15 or 16 waves: with few tiles (N / 16 below a few per CU) all of
//     them go into the K split so that a CU still has 16 waves' worth of loads in flight;
//   * with four row groups K is also split over grid.y, one staged chunk per workgroup, and workgroups are up to
//     four tiles wide: every workgroup stages all the rows, and at one tile per workgroup the activations would
//     be four times the weight bytes on the L2 -> CU path. The slices meet in fp32 workspace (splitKReduceKernel);
//   * the activation rows (G groups of 16) are staged once per workgroup in LDS (rows padded by 16 bytes)
//     by direct-to-LDS loads and read from there as the first MFMA operand; K is processed in chunks of
//     4096 / G columns so that the staged rows fit. A weight fragment is multiplied against all G groups
//     while it is in registers;
//   * lane (n = lane % 16, kgrp = lane / 16) loads 32 consecutive weights of row n per step of 128 (four
//     16-byte loads; the four kgrps of a row cover 256 contiguous bytes), one step ahead of the MFMAs. Which
//     K index sits in which MFMA slot is free as long as both operands agree, so no shuffling is needed.
struct SkinnyArgs {
  const void* A;
  const void* B;
  const void* Cin;
  const void* bias;
  void* out;
  int64_t lda, ldb, ldo, sCm, sCn;
  int M, N, K;
  float alpha, beta;
  float* partial;  // K split over grid.y: fp32 partial products [gridDim.y][M][N] for splitKReduceKernel, else null
  int kPerWg;      // K columns per grid.y slice (K when not split)
  int colsPerWg;   // gemmSkinnyLdsKernel: output columns per workgroup
  bool siluMul;    // gemmSkinnyLdsKernel: every 64 columns are 32 gate and 32 up columns; out (N / 2 wide) = silu(gate) * up
  // gemmSkinnyLdsKernel: the interleaved rotary embedding on the leading rotCols columns (heads of rotHeadDim), tables
  // [rotTableRows, rotHeadDim / 2] of T or fp32, row m uses table row m % rotTableRows; rotCols = 0: none
  const void* rotCos;
  const void* rotSin;
  int rotCols, rotHeadDim, rotTableRows;
  bool rotTableF32;
  float rotSinSign;
};

constexpr int kSkinnyStep = 128;    // K elements one wave consumes per step (4 kgrps x 32)
constexpr int kSkinnyPad = 8;       // elements appended to every staged activation row
constexpr int kSkinnyRowsK = 16 * 4096;  // staged rows x columns per pass: 16 G x (4096 / G + 8) x 2 B <= 129 KiB
constexpr int kSkinnyMaxM = 64;     // beyond this the tiled kernels take over

template <typename T, int NTW, int KS, int G>
__global__ __launch_bounds__(NTW * KS * 64) void gemmSkinnyKernel(SkinnyArgs a) {
  using Frag = typename MfmaOp<T>::Frag;
  constexpr int THREADS = NTW * KS * 64, CHUNK = kSkinnyRowsK / (16 * G);
  static_assert(CHUNK / kSkinnyStep >= KS, "every wave of the K split needs a step of the chunk");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* sx = reinterpret_cast<T*>(smem);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = wave / KS, ks = wave % KS;
  const int r16 = lane & 15, kgrp = lane >> 4;
  const int n0 = (blockIdx.x * NTW + tile) * 16;
  const T* wrow = reinterpret_cast<const T*>(a.B) + (int64_t)min(n0 + r16, a.N - 1) * a.ldb + kgrp * 32;
  const uint64_t xp = reinterpret_cast<uint64_t>(a.A);
  const u32x4 rsX = {(uint32_t)xp, (uint32_t)(xp >> 32) & 0xffffu, (uint32_t)(((int64_t)(a.M - 1) * a.lda + a.K) * sizeof(T)),
                     0x00020000u};
  const unsigned ldsBase = (unsigned)(size_t)(__attribute__((address_space(3))) char*)smem;
  f32x4 acc[G];
#pragma unroll
  for (int gi = 0; gi < G; ++gi) acc[gi] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int kBegin = blockIdx.y * a.kPerWg, kEnd = min(a.K, kBegin + a.kPerWg);
  for (int kc = kBegin; kc < kEnd; kc += CHUNK) {
    const int kcLen = min(CHUNK, kEnd - kc);  // a multiple of 128, as K and the slices are
    const int ldx = kcLen + kSkinnyPad;
    // this wave's share of the chunk: a contiguous run of 128-element steps
    const int steps = kcLen / kSkinnyStep;
    const int per = (steps + KS - 1) / KS;
    const int sBegin = ks * per, sEnd = min(steps, sBegin + per);
    const T* wk = wrow + kc;
    // the first weight loads go out before the activations are staged
    Frag w[4];
    if (sBegin < sEnd) {  // wave-uniform
#pragma unroll
      for (int t = 0; t < 4; ++t) w[t] = *reinterpret_cast<const Frag*>(wk + sBegin * kSkinnyStep + 8 * t);
    }
    if (kc > kBegin) __syncthreads();  // everyone is done with the previous chunk's activations
    // The activations go from memory straight into LDS, 512 columns of one row (1 KiB) per wave instruction:
    // the row and column of a piece are wave-uniform and travel in the scalar offset and in M0.
    const int segs = (kcLen + 511) / 512;
    for (int i = __builtin_amdgcn_readfirstlane(wave); i < a.M * segs; i += THREADS / 64) {
      const int r = i / segs, c0 = (i - r * segs) * 512;
      const int from = __builtin_amdgcn_readfirstlane((int)(((int64_t)r * a.lda + kc + c0) * sizeof(T)));
      const unsigned to = __builtin_amdgcn_readfirstlane(ldsBase + (unsigned)((r * ldx + c0) * sizeof(T)));
      if (c0 + lane * 8 < kcLen) loadToLds16(rsX, lane * 16, from, to);
    }
    __builtin_amdgcn_s_waitcnt(0x0070);  // this wave's pieces have landed
    __syncthreads();
    const T* xrow[G];  // fragment rows past M repeat the last row and are discarded
#pragma unroll
    for (int gi = 0; gi < G; ++gi) xrow[gi] = sx + min(gi * 16 + r16, a.M - 1) * ldx + kgrp * 32;
    for (int s = sBegin; s < sEnd; ++s) {
      Frag c[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) c[t] = w[t];
      if (s + 1 < sEnd) {
#pragma unroll
        for (int t = 0; t < 4; ++t) w[t] = *reinterpret_cast<const Frag*>(wk + (s + 1) * kSkinnyStep + 8 * t);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int gi = 0; gi < G; ++gi)
          acc[gi] = MfmaOp16<T>::run(*reinterpret_cast<const Frag*>(xrow[gi] + s * kSkinnyStep + 8 * t), c[t], acc[gi]);
    }
  }
  // the partial sums of the K split meet where the activations were
  __syncthreads();
  float* red = reinterpret_cast<float*>(smem);  // [NTW * KS][G][4][64]
#pragma unroll
  for (int gi = 0; gi < G; ++gi)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[((wave * G + gi) * 4 + r) * 64 + lane] = acc[gi][r];
  __syncthreads();
  const int col = n0 + r16;
  if (ks == 0 && col < a.N) {
    T* out = reinterpret_cast<T*>(a.out);
    const T* cin = reinterpret_cast<const T*>(a.Cin);
    const float bv = a.bias ? static_cast<float>(reinterpret_cast<const T*>(a.bias)[col]) : 0.f;
#pragma unroll
    for (int gi = 0; gi < G; ++gi)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = gi * 16 + kgrp * 4 + r;
        if (row < a.M) {
          float v = 0.f;
#pragma unroll
          for (int w2 = 0; w2 < KS; ++w2) v += red[(((tile * KS + w2) * G + gi) * 4 + r) * 64 + lane];
          if (a.partial) {  // this slice's sum; the reduction pass applies the epilogue
            a.partial[((int64_t)blockIdx.y * a.M + row) * a.N + col] = v;
            continue;
          }
          v = v * a.alpha + bv;
          if (cin) v += a.beta * static_cast<float>(cin[(int64_t)row * a.sCm + (int64_t)col * a.sCn]);
          out[(int64_t)row * a.ldo + col] = static_cast<T>(v);
        }
      }
  }
}

// 33 to 64 rows against a wide weight (at least 512 column tiles): no K split over the grid, so no partial products
// and no reduction pass. One workgroup owns NTW column tiles for the whole of K and walks it in chunks of 256: the
// four waves of a tile each take 64 columns of the chunk.
//   * The activations of a chunk (64 rows x 512 bytes) go from memory straight into one of four LDS buffers, three
//     chunks ahead of the one being multiplied (16-byte pieces XOR-swizzled by row on the global side; rows past M
//     lie past the end of the buffer descriptor and read as zeros). Nothing passes through registers, and the one
//     barrier per chunk waits for loads that were issued three chunks earlier.
//   * The weights are fetched kSkinnyWDepth chunks ahead into a ring of registers by ordinary loads at clamped
//     (always valid) addresses. Loads return in order, and the compiler counts only its own when it waits for a
//     ring slot, so the ring is deeper than the activation queue: the wait for chunk c then covers the activation
//     copy of chunk c + 1 and leaves the newer ones in flight.
constexpr int kSkinnyWChunk = 256, kSkinnyWBufs = 4, kSkinnyWDepth = 5;

template <typename T, int NTW>
__global__ __launch_bounds__(NTW * 4 * 64) void gemmSkinnyWideKernel(SkinnyArgs a) {
  using Frag = typename MfmaOp<T>::Frag;
  constexpr int KS = 4, G = 4, NW = NTW * KS, CHUNK = kSkinnyWChunk, NBUF = kSkinnyWBufs, DEPTH = kSkinnyWDepth;
  constexpr int SLOTS = DEPTH + 1, UNROLL = SLOTS * NBUF / (SLOTS % 2 == 0 ? 2 : 1);  // a common multiple of both rings
  static_assert(UNROLL % SLOTS == 0 && UNROLL % NBUF == 0, "ring indices must be compile-time");
  constexpr int BUF = 64 * CHUNK;       // elements of one activation buffer
  constexpr int XPW = (32 + NW - 1) / NW;  // copy instructions (two rows each) per wave and chunk, at most
  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* sx = reinterpret_cast<T*>(smem);  // NBUF buffers of 64 rows x CHUNK
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int tile = wave / KS, ks = wave % KS;
  const int r16 = lane & 15, kgrp = lane >> 4;
  const int n0 = (blockIdx.x * NTW + tile) * 16;
  const int kBegin = blockIdx.y * a.kPerWg, kEnd = min(a.K, kBegin + a.kPerWg);  // grid.y slices K (whole chunks)
  const int nChunks = (kEnd - kBegin + CHUNK - 1) / CHUNK;
  // lane (n = lane % 16, kgrp = lane / 16) takes 16 consecutive weights of row n per chunk: two 16-byte loads,
  // the K slots of two MFMAs. Columns past the end of K read the last valid ones instead and are not used.
  const T* wbase = reinterpret_cast<const T*>(a.B) + (int64_t)min(n0 + r16, a.N - 1) * a.ldb + kgrp * 16;
  auto loadW = [&](int c, Frag (&w)[2]) {
    const T* src = wbase + min(kBegin + min(c, nChunks - 1) * CHUNK + ks * 64, kEnd - 64);
    w[0] = *reinterpret_cast<const Frag*>(src);
    w[1] = *reinterpret_cast<const Frag*>(src + 8);
  };
  const uint64_t xp = reinterpret_cast<uint64_t>(a.A);
  const u32x4 rsX = {(uint32_t)xp, (uint32_t)(xp >> 32) & 0xffffu, (uint32_t)(((int64_t)(a.M - 1) * a.lda + a.K) * sizeof(T)),
                     0x00020000u};
  const unsigned ldsBase = (unsigned)(size_t)(__attribute__((address_space(3))) char*)smem;
  // copy instruction j of a chunk fills rows 2 j and 2 j + 1 of the buffer (1 KiB): lane l owns physical 16-byte
  // piece l % 32 of row 2 j + l / 32 and fetches the logical piece the swizzle puts there
  int xoff[XPW];
#pragma unroll
  for (int i = 0; i < XPW; ++i) {
    const int row = 2 * (wave + i * NW) + (lane >> 5);
    xoff[i] = (int)(((int64_t)row * a.lda + (((lane & 31) ^ (row & 15)) << 3)) * sizeof(T));
  }
  // (a chunk past the end copies the last one again, into a buffer nobody reads any more: every wave then has
  // the same number of copies in flight at every barrier, which is what the wait below counts on)
  auto copyX = [&](int c, int buf) {
    const int from = (kBegin + min(c, nChunks - 1) * CHUNK) * (int)sizeof(T);
#pragma unroll
    for (int i = 0; i < XPW; ++i)
      if (wave + i * NW < 32) loadToLds16(rsX, xoff[i], from, ldsBase + (unsigned)((buf * BUF) * sizeof(T)) + (unsigned)(wave + i * NW) * 1024u);
  };
  f32x4 acc[G];
#pragma unroll
  for (int gi = 0; gi < G; ++gi) acc[gi] = f32x4{0.f, 0.f, 0.f, 0.f};
  // fragment rows: group gi, row r16; logical piece ks * 8 + kgrp * 2 + t sits at that index XOR r16
  const T* xlane[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) xlane[t] = sx + r16 * CHUNK + (((ks * 8 + kgrp * 2 + t) ^ r16) << 3);

  Frag w[SLOTS][2];
#pragma unroll
  for (int c = 0; c < NBUF - 1; ++c) copyX(c, c);
#pragma unroll
  for (int c = 0; c < DEPTH; ++c) loadW(c, w[c]);
  for (int c0 = 0; c0 < nChunks; c0 += UNROLL) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u;
      if (c < nChunks) {  // workgroup-uniform
        // This wave's copies of chunk c have landed: loads return in order, and what it requested after them is
        // the copies of NBUF - 2 chunks (at least 32 / NW instructions each) and the weights of NBUF - 1 (two
        // loads each). Past the barrier the whole chunk is in LDS and every wave has left the buffer of chunk c - 1.
        constexpr int kAfter = (NBUF - 2) * (32 / NW) + (NBUF - 1) * 2;
        __builtin_amdgcn_s_waitcnt(0x0f70 | (kAfter & 15) | ((kAfter >> 4) << 14));
        __builtin_amdgcn_s_barrier();
        copyX(c + NBUF - 1, (u + NBUF - 1) % NBUF);
        loadW(c + DEPTH, w[(u + DEPTH) % SLOTS]);
        if (kBegin + c * CHUNK + ks * 64 < kEnd) {  // wave-uniform: this wave's columns of the chunk exist
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int gi = 0; gi < G; ++gi)
              acc[gi] = MfmaOp16<T>::run(*reinterpret_cast<const Frag*>(xlane[t] + (u % NBUF) * BUF + gi * 16 * CHUNK), w[u % SLOTS][t], acc[gi]);
        }
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0070);
  __syncthreads();
  // the four K shares of a tile meet where the activations were
  float* red = reinterpret_cast<float*>(smem);  // [NTW * KS][G][4][64]
#pragma unroll
  for (int gi = 0; gi < G; ++gi)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[((wave * G + gi) * 4 + r) * 64 + lane] = acc[gi][r];
  __syncthreads();
  const int col = n0 + r16;
  if (ks == 0 && col < a.N) {
    T* out = reinterpret_cast<T*>(a.out);
    const T* cin = reinterpret_cast<const T*>(a.Cin);
    const float bv = a.bias ? static_cast<float>(reinterpret_cast<const T*>(a.bias)[col]) : 0.f;
#pragma unroll
    for (int gi = 0; gi < G; ++gi)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = gi * 16 + kgrp * 4 + r;
        if (row < a.M) {
          float v = 0.f;
#pragma unroll
          for (int w2 = 0; w2 < KS; ++w2) v += red[(((tile * KS + w2) * G + gi) * 4 + r) * 64 + lane];
          if (a.partial) {  // this slice's sum; the reduction pass applies the epilogue
            a.partial[((int64_t)blockIdx.y * a.M + row) * a.N + col] = v;
            continue;
          }
          v = v * a.alpha + bv;
          if (cin) v += a.beta * static_cast<float>(cin[(int64_t)row * a.sCm + (int64_t)col * a.sCn]);
          out[(int64_t)row * a.ldo + col] = static_cast<T>(v);
        }
      }
  }
}

// Up to 64 rows, both operands staged through LDS. Weight loads that deliver MFMA fragments straight into registers
// touch 16 rows x 64 bytes per instruction, and that pattern streams at 3.3 - 4.8 TB/s where whole-row pieces stream
// at 6.5 (measured on a [11008, 4096] bf16 matrix, cold). Here the copy instructions take 256 contiguous bytes of 4
// rows each (two full cache lines per row), for the weights as for the activations, and land in LDS without passing
// through registers; the MFMA fragments are then LDS reads (16-byte pieces XOR-swizzled by row on the global side of
// the copy, so those reads are conflict-free).
//   * a workgroup of eight waves owns colsPerWg output columns (at most 32 NTP: 64 or 128) for the whole of K (or a
//     grid.y slice of it); the host deals the columns evenly over the CUs, and weight rows past a workgroup's share
//     are not fetched. Wave w multiplies k-step w % 4 of every stage (32 of its 128 columns), all G row groups
//     against the NTP column tiles of its half: G + NTP fragment reads for G NTP MFMAs. The four k-step shares meet
//     in LDS at the end, where wave w finishes row group w % 4;
//   * K moves in stages of 128 columns. Loads return to a wave in the order it issued them, so a wave that copied
//     both operands could not keep the weights (from HBM: long latency, the traffic that matters) further ahead than the
//     activations (from L2). The two are therefore copied by different waves: waves 0-3 keep WST - 1 weight stages
//     (32 NTP rows x 256 bytes) in flight, waves 4-7 keep XST - 1 activation stages (16 G rows x 256 bytes) in flight,
//     each waits only for its own stage, and one barrier per stage publishes both. Rows past M and past N lie past
//     the end of the buffer descriptors and read as zeros. The weight copies are marked non-temporal: read once,
//     they would otherwise push the activations out of L2, and a weight stream larger than the 256 MiB memory-side
//     cache gains nothing from passing through it (at one row, cold: 18.3 -> 16.4 us; a weight that does fit in that
//     cache and is re-read at once loses 1 us);
//   * workgroup b starts its walk over K at stage (13 b) mod stages and wraps around: with every workgroup on the same
//     columns at the same time the requests fall on a fraction of the memory channels (measured at 16 rows, cold:
//     20.0 us with a common start, 18.5 with this one, 26 when neighbours start 8 stages apart);
//   * more stages in flight are slower, here as in the other streaming kernels (weights 5 or 7 stages ahead instead
//     of 3: 16.9 -> 18.8 and 18.0 us at one row; at 64 rows rings of 5 + 5, 6 + 3, 6 + 4, 5 + 3 and 5 + 4 stages all read
//     23.4-23.6 us against 23.1 with 4 + 4, and two activation stages 31.8), and so is leaving the copies to four extra
//     waves that do nothing else, or to eight of sixteen (a workgroup of 1024 with the roles apart: 22.5 -> 23.8 us at 64
//     rows, 15.8 -> 16.9 at one).
//     What bounds 64 rows is the bytes a CU takes in: every workgroup reads all the activations (from L2), as many
//     bytes again as its share of the weights. Splitting K over grid.y (each workgroup then takes in half or a quarter
//     of the activations) loses more to the fp32 slices and their reduction pass: 23.5 -> 26.1 us two ways, 35.8 four ways.
constexpr int kSkinnyLdsBK = 128, kSkinnyLdsStagger = 13;

template <typename T, int G, int NTP, int WST, int XST>
__global__ __launch_bounds__(512) void gemmSkinnyLdsKernel(SkinnyArgs a) {
  using Frag = typename MfmaOp<T>::Frag;
  constexpr int BK = kSkinnyLdsBK, BN = 32 * NTP;  // NTP column tiles of 16 per wave, two waves side by side
  constexpr int WIPW = BN / 4 / 4, XIPW = G;      // copy instructions (4 rows x 256 bytes) per wave and stage: weights, activations
  constexpr int WBUF = BN * BK, XBUF = G * 16 * BK;  // elements per stage buffer
  constexpr int UNROLL = WST % XST == 0 ? WST : (XST % WST == 0 ? XST : WST * XST);
  constexpr int IPW = WIPW > XIPW ? WIPW : XIPW;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* sw = reinterpret_cast<T*>(smem);   // WST weight buffers
  T* sx = sw + WST * WBUF;              // XST activation buffers
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, kgrp = lane >> 4;
  const int ci = wave & 3;               // copy instruction slot of this wave (rows 4 ci + 16 i of a buffer)
  const int kq = wave & 3, nb = wave >> 2;  // multiplies k-step kq of every stage against column tiles NTP nb ... NTP nb + NTP - 1
  const int n0 = blockIdx.x * a.colsPerWg, nCols = min(a.colsPerWg, a.N - n0);  // this workgroup's columns: at most BN
  const int kBegin = blockIdx.y * a.kPerWg, kEnd = min(a.K, kBegin + a.kPerWg);
  const int nStages = (kEnd - kBegin) / BK;  // K and the slices are multiples of 128
  const int kStart = (int)((blockIdx.x * (unsigned)kSkinnyLdsStagger) % (unsigned)nStages);
  auto descriptor = [](const void* base, int64_t bytes) {
    const uint64_t p = reinterpret_cast<uint64_t>(base);
    u32x4 d = {(uint32_t)p, (uint32_t)(p >> 32) & 0xffffu, (uint32_t)bytes, 0x00020000u};
    return d;
  };
  // waves 0-3 copy weights, waves 4-7 activations (wave-uniform): descriptor, row stride and first row differ
  const bool copiesW = wave < 4;
  const u32x4 rs = copiesW ? descriptor(a.B, ((int64_t)(a.N - 1) * a.ldb + a.K) * sizeof(T))
                           : descriptor(a.A, ((int64_t)(a.M - 1) * a.lda + a.K) * sizeof(T));
  const int ipw = copiesW ? WIPW : XIPW;
  const unsigned ldsBase = (unsigned)(size_t)(__attribute__((address_space(3))) char*)(copiesW ? sw : sx);
  const unsigned bufBytes = (unsigned)((copiesW ? WBUF : XBUF) * sizeof(T));
  // copy instruction q = ci + 4 i of a stage fills rows 4 q .. 4 q + 3 of the buffer; lane l owns physical piece l % 16
  // of row l / 16 and fetches the logical piece the swizzle puts there
  unsigned voff[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int row = 4 * (ci + 4 * i) + (lane >> 4), piece = ((lane & 15) ^ (row & 15)) << 3;
    // (weight rows past this workgroup's columns: an offset past the end of the descriptor, which reads zeros without traffic)
    voff[i] = copiesW ? (row < nCols ? (unsigned)(((int64_t)(n0 + row) * a.ldb + piece) * sizeof(T)) : 0x80000000u)
                      : (unsigned)(((int64_t)row * a.lda + piece) * sizeof(T));
  }
  // (a stage past the end copies the last one again, into a buffer nobody reads any more: a wave then has the
  // same number of copies in flight at every barrier, which is what its wait counts on)
  auto copyStage = [&](int c, int buf) {
    int cc = min(c, nStages - 1) + kStart;
    if (cc >= nStages) cc -= nStages;
    const int from = (kBegin + cc * BK) * (int)sizeof(T);
#pragma unroll
    for (int i = 0; i < IPW; ++i)
      if (i < ipw) {
        const unsigned to = ldsBase + (unsigned)buf * bufBytes + (unsigned)(ci + 4 * i) * 1024u;
        if (copiesW) loadToLds16Stream(rs, (int)voff[i], from, to);  // read once: must not push the activations out of L2
        else loadToLds16(rs, (int)voff[i], from, to);
      }
  };
  f32x4 acc[G][NTP];
#pragma unroll
  for (int gi = 0; gi < G; ++gi)
#pragma unroll
    for (int j = 0; j < NTP; ++j) acc[gi][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  // this wave's fragments: logical piece 4 kq + kgrp of row r16 (activations: + 16 gi rows; weights: + 16 (NTP nb + j) rows).
  // Every staged byte is read by two waves (activations) or one (weights): LDS bandwidth is what bounds 64 rows.
  const int off = ((4 * kq + kgrp) ^ r16) << 3;
  const T* xlane = sx + r16 * BK + off;
  const T* wlane = sw + (nb * NTP * 16 + r16) * BK + off;

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
        // this wave's copies of stage c have landed: loads return in order, and only the stages it requested after that
        // one are still in flight. Past the barrier both operands of the stage are in LDS and every wave has left the
        // buffers of stage c - 1, which the next copies overwrite.
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
        const T* xs = xlane + (u % XST) * XBUF;
        const T* ws = wlane + (u % WST) * WBUF;
        Frag wf[NTP];
#pragma unroll
        for (int j = 0; j < NTP; ++j) wf[j] = *reinterpret_cast<const Frag*>(ws + j * 16 * BK);
#pragma unroll
        for (int gi = 0; gi < G; ++gi) {
          const Frag xf = *reinterpret_cast<const Frag*>(xs + gi * 16 * BK);
#pragma unroll
          for (int j = 0; j < NTP; ++j) acc[gi][j] = MfmaOp16<T>::run(xf, wf[j], acc[gi][j]);
        }
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // the repeated copies of the last stage: nothing may land after the workgroup has gone
  __syncthreads();
  // the four k-step shares of a column tile pair meet where the stages were; wave (nb, kq) then finishes row group kq
  float* red = reinterpret_cast<float*>(smem);  // [8 waves][G][NTP][4][64]
#pragma unroll
  for (int gi = 0; gi < G; ++gi)
#pragma unroll
    for (int j = 0; j < NTP; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[(((wave * G + gi) * NTP + j) * 4 + r) * 64 + lane] = acc[gi][j][r];
  __syncthreads();
  const int gi = kq;
  if (a.siluMul) {
    // A workgroup's columns are whole blocks of 64: 32 gate columns, then the up columns of the same 32 channels.
    // Output tile t of 16 channels takes its gate values from column tile 4 (t / 2) + t % 2 and its up values from the
    // tile two further on; both sit at this lane's place in the partial sums, whichever waves produced them.
    constexpr int OTW = BN / 64;  // output tiles per wave half
    if (gi < G) {
      T* out = reinterpret_cast<T*>(a.out);
#pragma unroll
      for (int tt = 0; tt < OTW; ++tt) {
        const int t = nb * OTW + tt, tg = 4 * (t >> 1) + (t & 1), tu = tg + 2;
        if (tg * 16 >= nCols) continue;
        const int oc = n0 / 2 + (t >> 1) * 32 + (t & 1) * 16 + r16;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = gi * 16 + kgrp * 4 + r;
          if (row < a.M) {
            float gsum = 0.f, usum = 0.f;
#pragma unroll
            for (int k2 = 0; k2 < 4; ++k2) {
              gsum += red[(((((tg / NTP) * 4 + k2) * G + gi) * NTP + tg % NTP) * 4 + r) * 64 + lane];
              usum += red[(((((tu / NTP) * 4 + k2) * G + gi) * NTP + tu % NTP) * 4 + r) * 64 + lane];
            }
            out[(int64_t)row * a.ldo + oc] = static_cast<T>(gsum * __builtin_amdgcn_rcpf(1.f + __expf(-gsum)) * usum);
          }
        }
      }
    }
    return;
  }
  if (gi < G) {
    T* out = reinterpret_cast<T*>(a.out);
    const T* cin = reinterpret_cast<const T*>(a.Cin);
#pragma unroll
    for (int j = 0; j < NTP; ++j) {
      const int lc = (nb * NTP + j) * 16 + r16, col = n0 + lc;
      if (lc >= nCols) continue;
      const float bv = a.bias ? static_cast<float>(reinterpret_cast<const T*>(a.bias)[col]) : 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = gi * 16 + kgrp * 4 + r;
        if (row < a.M) {
          float v = 0.f;
#pragma unroll
          for (int k2 = 0; k2 < 4; ++k2) v += red[((((nb * 4 + k2) * G + gi) * NTP + j) * 4 + r) * 64 + lane];
          if (a.partial) {  // this slice's sum; the reduction pass applies the epilogue
            a.partial[((int64_t)blockIdx.y * a.M + row) * a.N + col] = v;
            continue;
          }
          v = v * a.alpha + bv;
          if (cin) v += a.beta * static_cast<float>(cin[(int64_t)row * a.sCm + (int64_t)col * a.sCn]);
          if (a.rotCols > 0) {
            // adjacent columns are a pair and sit in adjacent lanes (the column shares are even): every lane takes part
            // in the exchange, columns at or past rotCols keep their value
            const float other = __shfl_xor(v, 1, 64);
            if (col < a.rotCols) {
              const int64_t ti = (int64_t)(row % a.rotTableRows) * (a.rotHeadDim >> 1) + ((col % a.rotHeadDim) >> 1);
              const float c = a.rotTableF32 ? reinterpret_cast<const float*>(a.rotCos)[ti] : static_cast<float>(reinterpret_cast<const T*>(a.rotCos)[ti]);
              const float sn = (a.rotTableF32 ? reinterpret_cast<const float*>(a.rotSin)[ti] : static_cast<float>(reinterpret_cast<const T*>(a.rotSin)[ti])) * a.rotSinSign;
              v = (col & 1) ? other * sn + v * c : v * c - other * sn;
            }
          }
          out[(int64_t)row * a.ldo + col] = static_cast<T>(v);
        }
      }
    }
  }
}

// -------------------------------------------------------------- transpose ----
// dst[b, c, r] = src[b, r, c] for 2-byte or 4-byte elements, 64x64 tiles through LDS.
template <typename U>
__global__ __launch_bounds__(256) void transposeKernel(U* __restrict__ dst, const U* __restrict__ src, int64_t rows,
                                                        int64_t cols, int64_t srcRowStride, int64_t srcColStride,
                                                        int64_t srcBatchStride, int64_t dstBatchStride) {
  __shared__ U tile[64][65];
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
  src += blockIdx.z * srcBatchStride;
  dst += blockIdx.z * dstBatchStride;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  // read with lanes along whichever source dim is contiguous
  if (srcColStride == 1) {
    for (int i = ty; i < 64; i += 4) {
      int64_t r = r0 + i, c = c0 + tx;
      if (r < rows && c < cols) tile[i][tx] = src[r * srcRowStride + c];
    }
  } else {
    for (int i = ty; i < 64; i += 4) {
      int64_t r = r0 + tx, c = c0 + i;
      if (r < rows && c < cols) tile[tx][i] = src[r * srcRowStride + c * srcColStride];
    }
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    int64_t c = c0 + i, r = r0 + tx;
    if (r < rows && c < cols) dst[c * rows + r] = tile[tx][i];
  }
}

// ---------------------------------------------------------------- FMA engine --
// ------------------------------------------------------------ fp32 on MFMA ---
// Tile of workgroup `pid` of a one-dimensional grid over tilesM x tilesN tiles: consecutive workgroup ids go to
// consecutive XCDs (own L2 each), so XCD x takes a contiguous band of the tile order, and the order walks groups of 8
// tile rows column by column: the workgroups an XCD runs at one time share few operand panels.
__device__ __forceinline__ void xcdBandTile(int pid, int tilesM, int tilesN, int* tm, int* tn) {
  const int total = tilesM * tilesN;
  const int xcd = pid & 7, idx = pid >> 3;
  const int q = total >> 3, r = total & 7;
  const int logical = xcd * q + min(xcd, r) + idx;
  constexpr int GROUP = 8;
  const int width = GROUP * tilesN;
  const int group = logical / width;
  const int first = group * GROUP;
  const int gsize = min(tilesM - first, GROUP);
  const int in = logical - group * width;
  *tm = first + in % gsize;
  *tn = in / gsize;
}

// Epilogue of the fp32 MFMA kernels: register 4 g + r of a block is output row l32, column 8 g + 4 half + r.
template <int WT>
__device__ __forceinline__ void gemmF32StoreTile(const GemmProblem& p, const f32x16 (&acc)[WT][WT], int64_t m0, int64_t n0, int64_t batch,
                                                 int wm, int wn, int l32, int half) {
  float* out = reinterpret_cast<float*>(p.out) + batch * p.sOb;
  const float* cin = p.Cin ? reinterpret_cast<const float*>(p.Cin) + batch * p.sCb : nullptr;
  const float* bias = reinterpret_cast<const float*>(p.bias);
  const bool vec = (p.N & 3) == 0 && (p.sOm & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
#pragma unroll
  for (int bm = 0; bm < WT; ++bm) {
    const int64_t row = m0 + (wm * WT + bm) * 32 + l32;
    if (row >= p.M) continue;
#pragma unroll
    for (int bn = 0; bn < WT; ++bn)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int64_t col = n0 + (wn * WT + bn) * 32 + 8 * g + 4 * half;
        if (col >= p.N) continue;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          v[r] = acc[bm][bn][4 * g + r] * p.alpha;
          if (col + r < p.N) {
            if (bias) v[r] += bias[col + r];
            if (cin) v[r] += p.beta * cin[row * p.sCm + (col + r) * p.sCn];
          }
        }
        if (vec) {
          *reinterpret_cast<f32x4*>(out + row * p.sOm + col) = f32x4{v[0], v[1], v[2], v[3]};
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (col + r < p.N) out[row * p.sOm + col + r] = v[r];
        }
      }
  }
}

// fp32 operands through v_mfma_f32_32x32x2f32 (true fp32 products and sums; 157 TFLOP/s peak against 79 for the vector
// unit): 4 waves in 2 x 2, a wave owns WT x WT blocks of 32 x 32, K in stages of BK through two LDS buffers filled
// from registers (the loads of stage t + 1 are issued before the MFMAs of stage t). The instruction takes one k per
// lane half; which two k meet in one instruction does not matter as long as both operands agree, so lane half h
// takes k = 8 q + 4 h + j at step (q, j): its four steps of a half-stage are one 16-byte LDS read per fragment.
// LDS rows are BK + 4 floats apart: 16 consecutive rows then start on 16 different 16-byte bank groups.
// Either operand may be K-contiguous ([rows, K]) or row-contiguous ([K, rows], e.g. the second operand of mm);
// the weight fragment goes first, so a lane ends up with four consecutive columns of one output row per register
// quad (16-byte stores). With the tiles staged through registers the MFMA pipe is busy 79 % of the time
// (123 TFLOP/s at 8192 x 4096 x 4096); without the global loads 135, without loads and LDS writes 148: the kernel
// below, which has neither, takes the layout that allows it.
template <int WT, int BK, bool A_BY_K, bool B_BY_K>
__global__ __launch_bounds__(256) void gemmMfmaF32Kernel(GemmProblem p) {
  constexpr int BM = 64 * WT, BN = 64 * WT, PAD = BK + 4;
  constexpr int LPT = BM * BK / 4 / 256;  // 16-byte loads per thread, stage and operand
  __shared__ __attribute__((aligned(16))) float sA[2][BM * PAD];
  __shared__ __attribute__((aligned(16))) float sB[2][BN * PAD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, half = lane >> 5;
  int tm, tn;
  xcdBandTile(blockIdx.x, (int)((p.M + BM - 1) / BM), (int)((p.N + BN - 1) / BN), &tm, &tn);
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN, batch = blockIdx.z;
  const float* A = reinterpret_cast<const float*>(p.A) + batch * p.sAb;
  const float* B = reinterpret_cast<const float*>(p.B) + batch * p.sBb;
  f32x4 ra[LPT], rb[LPT];
  // 16 bytes of an operand tile: along K when the operand is K-contiguous, along the rows otherwise. Every thread
  // keeps one running pointer per load; rows past the end are clamped to the last ones (their products land in
  // output rows or columns that are never stored), so only the last stage of a ragged K needs a predicate.
  const float* pa[LPT];
  const float* pb[LPT];
  int ka[LPT], kb[LPT];  // k of the load within its stage
  int wa[LPT], wb[LPT];  // where it goes in the LDS tile
  auto aim = [&](const float* base, auto byK, int64_t rowStride, int64_t kStride, int64_t row0, int64_t rows, const float* (&ptr)[LPT],
                 int (&kk)[LPT], int (&ww)[LPT]) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int f = tid + 256 * i;
      constexpr int RV = BM / 4, KV = BK / 4;  // 4-row vectors per k, 4-k vectors per row
      const int r = byK ? f / KV : (f % RV) * 4;
      kk[i] = byK ? (f % KV) * 4 : f / RV;
      ww[i] = r * PAD + kk[i];
      ptr[i] = base + min(row0 + r, rows - (byK ? 1 : 4)) * rowStride + kk[i] * kStride;
    }
  };
  aim(A, std::integral_constant<bool, A_BY_K>{}, p.sAm, p.sAk, m0, p.M, pa, ka, wa);
  aim(B, std::integral_constant<bool, B_BY_K>{}, p.sBn, p.sBk, n0, p.N, pb, kb, wb);
  const int64_t stepA = BK * p.sAk, stepB = BK * p.sBk;
  auto fetch = [&](int64_t k0, bool ragged) {
    if (!ragged) {
#pragma unroll
      for (int i = 0; i < LPT; ++i) {
        ra[i] = *reinterpret_cast<const f32x4*>(pa[i]);
        rb[i] = *reinterpret_cast<const f32x4*>(pb[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < LPT; ++i) {
        ra[i] = rb[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (k0 + ka[i] < p.K) ra[i] = *reinterpret_cast<const f32x4*>(pa[i]);
        if (k0 + kb[i] < p.K) rb[i] = *reinterpret_cast<const f32x4*>(pb[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      pa[i] += stepA;
      pb[i] += stepB;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      if (A_BY_K) {
        *reinterpret_cast<f32x4*>(sA[buf] + wa[i]) = ra[i];
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) sA[buf][wa[i] + j * PAD] = ra[i][j];
      }
      if (B_BY_K) {
        *reinterpret_cast<f32x4*>(sB[buf] + wb[i]) = rb[i];
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) sB[buf][wb[i] + j * PAD] = rb[i][j];
      }
    }
  };
  f32x16 acc[WT][WT];
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  const int stages = (int)((p.K + BK - 1) / BK);
  const bool raggedK = (p.K % BK) != 0;  // then the last stage is partial
  fetch(0, raggedK && stages == 1);
  stash(0);
  __syncthreads();
  for (int t = 0; t < stages; ++t) {
    const int cur = t & 1;
    if (t + 1 < stages) fetch((int64_t)(t + 1) * BK, raggedK && t + 2 == stages);
    const float* ta = sA[cur] + (wm * 32 * WT + l32) * PAD + 4 * half;
    const float* tb = sB[cur] + (wn * 32 * WT + l32) * PAD + 4 * half;
#pragma unroll
    for (int q = 0; q < BK / 8; ++q) {
      f32x4 fa[WT], fb[WT];
#pragma unroll
      for (int i = 0; i < WT; ++i) {
        fa[i] = *reinterpret_cast<const f32x4*>(ta + i * 32 * PAD + 8 * q);
        fb[i] = *reinterpret_cast<const f32x4*>(tb + i * 32 * PAD + 8 * q);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int bm = 0; bm < WT; ++bm)
#pragma unroll
          for (int bn = 0; bn < WT; ++bn)
            acc[bm][bn] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[bn][j], fa[bm][j], acc[bm][bn], 0, 0, 0);
    }
    if (t + 1 < stages) stash(cur ^ 1);
    __syncthreads();
  }
  gemmF32StoreTile<WT>(p, acc, m0, n0, batch, wm, wn, l32, half);
}

// The same product for a K-contiguous first operand and K a multiple of 32 (linear, mm, bmm): the tiles go from
// global memory straight into LDS (global_load_lds_dwordx4: lane i of a wave fills bytes 16 i .. 16 i + 15 of a 1 KiB
// piece), so no staging registers, no LDS writes by the waves and no wait between a load's return and its use other
// than the barrier. Rows are 32 floats (8 pieces of 16 bytes) without padding; piece c of row r sits at position
// c ^ swz(r), swz(r) = (r ^ (r >> 3)) & 7, chosen by the loading lane through the global address it reads, which makes
// the 16-byte fragment reads of 16 consecutive rows hit 16 different bank groups (no bank conflict is counted).
// 138 TFLOP/s at 8192 x 4096 x 4096 and at 2048 x 4096 x 4096 (88 % of the MFMA rate a register-only loop of the same
// instruction sustains, 156); what is left is the barrier and the wait for the stage's loads once per 64 MFMAs with
// two waves per SIMD. A third LDS buffer would leave room for one workgroup per compute unit only. Workgroups take
// their tiles in XCD bands (xcdBandTile): 5 % fewer L2 misses than row-major order, the same time.
__device__ __forceinline__ int f32Swz(int row) { return (row ^ (row >> 3)) & 7; }

// With B_BY_K false the second operand is [K, N] row-major (mm, bmm, matmul): its tile sits in LDS as it sits in memory,
// 32 rows of k by BN columns, and a lane reads its operand of every MFMA step on its own (4-byte reads along n:
// consecutive lanes, consecutive banks).
template <int WT, bool B_BY_K>
__global__ __launch_bounds__(256) void gemmMfmaF32DirectKernel(GemmProblem p) {
  constexpr int BM = 64 * WT, BN = 64 * WT, BK = 32;
  constexpr int LPT = BM * BK / 4 / 256;  // 16-byte pieces per thread, stage and operand
  __shared__ __attribute__((aligned(1024))) float sA[2][BM * BK];
  __shared__ __attribute__((aligned(1024))) float sB[2][BN * BK];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, half = lane >> 5;
  int tm, tn;
  xcdBandTile(blockIdx.x, (int)((p.M + BM - 1) / BM), (int)((p.N + BN - 1) / BN), &tm, &tn);
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN, batch = blockIdx.z;
  const float* A = reinterpret_cast<const float*>(p.A) + batch * p.sAb;
  const float* B = reinterpret_cast<const float*>(p.B) + batch * p.sBb;
  // piece i * 256 + tid of a tile: row (i * 256 + tid) / 8 at position tid % 8, holding chunk position ^ swz(row);
  // rows past the end are clamped (their products land in rows or columns that are never stored)
  const float* pa[LPT];
  const float* pb[LPT];
#pragma unroll
  for (int i = 0; i < LPT; ++i) {
    const int row = (i * 256 + tid) >> 3, chunk = (tid & 7) ^ f32Swz(row);
    pa[i] = A + min(m0 + row, p.M - 1) * p.sAm + chunk * 4;
    if (B_BY_K) {
      pb[i] = B + min(n0 + row, p.N - 1) * p.sBn + chunk * 4;
    } else {  // piece: k = piece / (BN / 4), columns 4 (piece % (BN / 4)) .. + 3, clamped to the last four
      const int piece = i * 256 + tid;
      pb[i] = B + (piece / (BN / 4)) * p.sBk + min(n0 + (piece % (BN / 4)) * 4, p.N - 4);
    }
  }
  const int64_t stepB = B_BY_K ? BK : BK * p.sBk;
  typedef __attribute__((address_space(3))) void* LdsPtr;
  auto fetch = [&](int buf) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      // as assembly: the compiler would wait for a load into LDS before the next LDS read of any buffer
      globalLoadToLds16(pa[i], (uint32_t)(uintptr_t)(LdsPtr)(sA[buf] + (i * 256 + wave * 64) * 4));
      globalLoadToLds16(pb[i], (uint32_t)(uintptr_t)(LdsPtr)(sB[buf] + (i * 256 + wave * 64) * 4));
      pa[i] += BK;
      pb[i] += stepB;
    }
  };
  // fragment of block row i at step q: row R = wave rows + 32 i + l32, chunk 2 q + half
  int offA[WT], offB[WT], swA[WT], swB[WT];
#pragma unroll
  for (int i = 0; i < WT; ++i) {
    const int ra = (wm * WT + i) * 32 + l32, rb = (wn * WT + i) * 32 + l32;
    offA[i] = ra * BK, offB[i] = B_BY_K ? rb * BK : 4 * half * BN + rb;
    swA[i] = f32Swz(ra) ^ half, swB[i] = f32Swz(rb) ^ half;
  }
  f32x16 acc[WT][WT];
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  const int stages = (int)(p.K / BK);
  fetch(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  for (int t = 0; t < stages; ++t) {
    const int cur = t & 1;
    if (t + 1 < stages) fetch(cur ^ 1);
    f32x4 fa[2][WT], fb[2][WT];
    auto frags = [&](int q) {
#pragma unroll
      for (int i = 0; i < WT; ++i) {
        fa[q & 1][i] = *reinterpret_cast<const f32x4*>(sA[cur] + offA[i] + (((2 * q) ^ swA[i]) << 2));
        if (B_BY_K) {
          fb[q & 1][i] = *reinterpret_cast<const f32x4*>(sB[cur] + offB[i] + (((2 * q) ^ swB[i]) << 2));
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) fb[q & 1][i][j] = sB[cur][offB[i] + (8 * q + j) * BN];
        }
      }
    };
    frags(0);
#pragma unroll
    for (int q = 0; q < BK / 8; ++q) {
      if (q + 1 < BK / 8) frags(q + 1);  // under the MFMAs of step q
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int bm = 0; bm < WT; ++bm)
#pragma unroll
          for (int bn = 0; bn < WT; ++bn)
            acc[bm][bn] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[q & 1][bn][j], fa[q & 1][bm][j], acc[bm][bn], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }
  gemmF32StoreTile<WT>(p, acc, m0, n0, batch, wm, wn, l32, half);
}

// Whether gemmMfmaF32Kernel can take the problem: each operand contiguous along K or along its rows, 16-byte pieces
// whole and aligned.
constexpr int kF32BKBig = 32;  // stage depth of the 128 x 128 tile
static bool f32MfmaEligible(const GemmProblem& p) {
  auto operand = [&](const void* base, int64_t rowStride, int64_t kStride, int64_t batchStride, int64_t rows) {
    if ((reinterpret_cast<uintptr_t>(base) & 15) != 0 || (batchStride & 3) != 0) return false;
    if (kStride == 1) return (p.K & 3) == 0 && (rowStride & 3) == 0;
    return rowStride == 1 && (rows & 3) == 0 && (kStride & 3) == 0;
  };
  return p.K > 0 && operand(p.A, p.sAm, p.sAk, p.sAb, p.M) && operand(p.B, p.sBn, p.sBk, p.sBb, p.N) &&
         ceilDiv(p.M, 64) * ceilDiv(p.N, 64) < ((int64_t)1 << 31) && p.batch <= 65535;
}

template <typename T>
__global__ __launch_bounds__(256) void gemmFmaKernel(GemmProblem p) {
  __shared__ float sA[16][64 + 4];
  __shared__ float sB[16][64 + 4];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int64_t m0 = (int64_t)blockIdx.y * 64, n0 = (int64_t)blockIdx.x * 64;
  const int64_t b = blockIdx.z;
  const T* A = reinterpret_cast<const T*>(p.A) + b * p.sAb;
  const T* B = reinterpret_cast<const T*>(p.B) + b * p.sBb;
  float acc[4][4] = {{0.f}};
  for (int64_t k0 = 0; k0 < p.K; k0 += 16) {
    // 64 rows x 16 k per operand = 1024 elements, 4 per thread
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int e = threadIdx.x + 256 * i;
      int kk, rr;
      if (p.sAk == 1) kk = e & 15, rr = e >> 4; else rr = e & 63, kk = e >> 6;
      int64_t m = m0 + rr, k = k0 + kk;
      sA[kk][rr] = (m < p.M && k < p.K) ? static_cast<float>(A[m * p.sAm + k * p.sAk]) : 0.f;
      if (p.sBk == 1) kk = e & 15, rr = e >> 4; else rr = e & 63, kk = e >> 6;
      int64_t n = n0 + rr;
      k = k0 + kk;
      sB[kk][rr] = (n < p.N && k < p.K) ? static_cast<float>(B[n * p.sBn + k * p.sBk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float a[4], bb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = sA[kk][ty * 4 + i], bb[i] = sB[kk][tx * 4 + i];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], bb[j], acc[i][j]);
    }
    __syncthreads();
  }
  T* out = reinterpret_cast<T*>(p.out) + b * p.sOb;
  const T* cin = p.Cin ? reinterpret_cast<const T*>(p.Cin) + b * p.sCb : nullptr;
  const T* bias = reinterpret_cast<const T*>(p.bias);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int64_t m = m0 + ty * 4 + i;
    if (m >= p.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int64_t n = n0 + tx * 4 + j;
      if (n >= p.N) continue;
      float v = acc[i][j] * p.alpha;
      if (bias) v += static_cast<float>(bias[n]);
      if (cin) v += p.beta * static_cast<float>(cin[m * p.sCm + n * p.sCn]);
      out[m * p.sOm + n] = static_cast<T>(v);
    }
  }
}

__global__ void gemmFmaKernelF64(GemmProblem p) {
  // double precision: one output per lane, plain loop (correctness path only)
  int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t m = blockIdx.y, b = blockIdx.z;
  if (n >= p.N) return;
  const double* A = reinterpret_cast<const double*>(p.A) + b * p.sAb + m * p.sAm;
  const double* B = reinterpret_cast<const double*>(p.B) + b * p.sBb + n * p.sBn;
  double acc = 0.0;
  for (int64_t k = 0; k < p.K; ++k) acc += A[k * p.sAk] * B[k * p.sBk];
  double v = acc * (double)p.alpha;
  if (p.bias) v += reinterpret_cast<const double*>(p.bias)[n];
  if (p.Cin) v += (double)p.beta * (reinterpret_cast<const double*>(p.Cin) + b * p.sCb)[m * p.sCm + n * p.sCn];
  (reinterpret_cast<double*>(p.out) + b * p.sOb)[m * p.sOm + n] = v;
}

// ------------------------------------------------------------------ driver ---
template <typename T, int BM, int BN>
static diopiError_t launchMfma(hipStream_t stream, const GemmProblem& p) {
  MfmaArgs g;
  g.A = p.A, g.B = p.B, g.out = p.out, g.Cin = p.Cin, g.bias = p.bias;
  g.sAb = p.sAb, g.lda = p.sAm, g.sBb = p.sBb, g.ldb = p.sBn, g.sOb = p.sOb, g.ldo = p.sOm;
  g.sCb = p.sCb, g.sCm = p.sCm, g.sCn = p.sCn;
  g.M = (int)p.M, g.N = (int)p.N, g.K = (int)p.K;
  g.tilesM = (int)ceilDiv(p.M, BM), g.tilesN = (int)ceilDiv(p.N, BN);
  g.alpha = p.alpha, g.beta = p.beta;
  g.vecEpilogue = false;
  constexpr size_t lds = 2 * (size_t)(BM + BN) * kBK * sizeof(T);
  AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&gemmMfmaKernel<T, BM, BN>), (int)lds));
  dim3 grid((unsigned)(g.tilesM * g.tilesN), 1, (unsigned)p.batch);
  hipLaunchKernelGGL((gemmMfmaKernel<T, BM, BN>), grid, dim3(256), lds, stream, g);
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

// Second pass of split-K: out = alpha * sum_s partial[s] + bias + beta * C, 8 columns per lane.
template <typename T>
__global__ __launch_bounds__(256) void splitKReduceKernel(MfmaArgs g, int splits) {
  using Frag = typename MfmaOp<T>::Frag;
  const int groups = g.N / 8;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)g.M * groups) return;
  const int row = (int)(idx / groups), col = (int)(idx - (int64_t)row * groups) * 8;
  const float* src = g.partial + (int64_t)row * g.N + col;
  // four slices' pieces are requested together (a loop of one load and one add per slice walks the slices one memory
  // round trip at a time); the additions keep the slice order
  f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = lo;
  const int64_t slice = (int64_t)g.M * g.N;
  int sp = 0;
  for (; sp + 4 <= splits; sp += 4) {
    f32x4 l4[4], h4[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      l4[u] = *reinterpret_cast<const f32x4*>(src + (sp + u) * slice);
      h4[u] = *reinterpret_cast<const f32x4*>(src + (sp + u) * slice + 4);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) lo += l4[u], hi += h4[u];
  }
  for (; sp < splits; ++sp) {
    lo += *reinterpret_cast<const f32x4*>(src + sp * slice);
    hi += *reinterpret_cast<const f32x4*>(src + sp * slice + 4);
  }
  const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  const T* cin = reinterpret_cast<const T*>(g.Cin);
  const T* bias = reinterpret_cast<const T*>(g.bias);
  Frag o, cv, bv;
  if (cin) cv = *reinterpret_cast<const Frag*>(cin + (int64_t)row * g.sCm + col);
  if (bias) bv = *reinterpret_cast<const Frag*>(bias + col);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float x = v[e] * g.alpha;
    if (bias) x += static_cast<float>(bv[e]);
    if (cin) x += g.beta * static_cast<float>(cv[e]);
    o[e] = static_cast<T>(x);
  }
  *reinterpret_cast<Frag*>(reinterpret_cast<T*>(g.out) + (int64_t)row * g.ldo + col) = o;
}

// Small reductions (decode-sized products: a few tens of thousands of lanes) go out as single waves, so that they spread
// over more CUs than they would fill workgroups of four.
template <typename T>
static void launchSplitKReduce(hipStream_t stream, const MfmaArgs& g, int splits, int64_t items) {
  const int threads = items <= 65536 ? 64 : 256;
  hipLaunchKernelGGL(splitKReduceKernel<T>, dim3((unsigned)ceilDiv(items, (int64_t)threads)), dim3(threads), 0, stream, g, splits);
}

// How many ways to split K so that a problem with few 128 x 128 tiles still fills the chip (two workgroups per CU):
// tiles * splits close to twice the CU count, at least four K tiles per split, at most 16 splits. 1 = do not split.
// *perSplit receives the K tiles per split; the last split has the remainder, never fewer than two (the kernel's
// pipeline needs two).
static int splitKWays(int64_t tiles, int64_t kTiles, int* perSplit) {
  const int64_t byChip = 2 * computeUnits() / std::max<int64_t>(tiles, 1), byK = kTiles / 4;
  int64_t splits = std::max<int64_t>(1, std::min<int64_t>(16, std::min(byChip, byK)));
  int64_t per = ceilDiv(kTiles, splits);
  while (per < kTiles && kTiles % per == 1) ++per;
  *perSplit = (int)per;
  return (int)ceilDiv(kTiles, per);
}

struct RotaryEpilogue {
  const void* cosT;
  const void* sinT;
  int cols, headDim, tableRows;
  bool tableF32;
  float sinSign;
};

// bT: the second operand is [K, N] with N contiguous and is used in place (p.sBk is then its row stride).
template <typename T, int EPI = kEpiLinear>
static diopiError_t launchMfmaPipelined(hipStream_t stream, const GemmProblem& p, float* partial = nullptr, int splits = 1,
                                        int kTilesPerSplit = 0, const RotaryEpilogue* rot = nullptr, bool bT = false) {
  MfmaArgs g;
  g.A = p.A, g.B = p.B, g.out = p.out, g.Cin = p.Cin, g.bias = p.bias;
  g.sAb = p.sAb, g.lda = p.sAm, g.sBb = p.sBb, g.ldb = bT ? p.sBk : p.sBn, g.sOb = p.sOb, g.ldo = p.sOm;
  g.sCb = p.sCb, g.sCm = p.sCm, g.sCn = p.sCn;
  g.M = (int)p.M, g.N = (int)p.N, g.K = (int)p.K;
  g.tilesM = (int)ceilDiv(p.M, 256), g.tilesN = (int)ceilDiv(p.N, 256);
  g.alpha = p.alpha, g.beta = p.beta;
  g.colScale = p.colScale, g.colScaleDtype = (int)p.colScaleDtype, g.colBias = p.colBias, g.colBiasDtype = (int)p.colBiasDtype;
  auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  // the vector epilogue addresses one batch of the output and of the addend with 32-bit byte offsets
  const bool span32 = ((p.M - 1) * p.sOm + p.N) * (int64_t)sizeof(T) < (int64_t(1) << 31) &&
                      (!p.Cin || ((p.M - 1) * p.sCm + p.N) * (int64_t)sizeof(T) < (int64_t(1) << 31));
  g.vecEpilogue = p.N % 8 == 0 && p.sOm % 8 == 0 && p.sOb % 8 == 0 && al16(p.out) && span32 &&
                  (!p.Cin || (p.sCn == 1 && p.sCm % 8 == 0 && p.sCb % 8 == 0 && al16(p.Cin))) && (!p.bias || al16(p.bias));
  constexpr size_t lds = 2 * (size_t)(256 + 256) * kBK * sizeof(T);
  if constexpr (EPI != kEpiRotaryLds && EPI != kEpiColScale) AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&gemmMfmaPipelinedKernel<T, EPI>), (int)lds));
  if (EPI == kEpiColScale) AMD_CHECK(p.colScale && g.vecEpilogue && !p.Cin && !p.bias, "column scale epilogue: needs the scale, the vector epilogue and neither addend nor bias");
  g.partial = partial;
  g.kTilesPerSplit = kTilesPerSplit;
  if (EPI == kEpiRotary || EPI == kEpiRotaryUniform || EPI == kEpiRotaryLds) {
    AMD_CHECK(rot && g.vecEpilogue && !p.Cin && p.alpha == 1.f, "rotary epilogue: needs tables, the vector epilogue and no addend");
    if (EPI != kEpiRotary) AMD_CHECK(!p.bias && rot->cols % 32 == 0, "rotary epilogue: the uniform form takes no bias and whole 32-column pieces");
    if (EPI == kEpiRotaryLds) AMD_CHECK(!rot->tableF32 && rot->headDim == 128, "rotary epilogue: tables through LDS are 16-bit, for heads of 128");
    g.rotCos = rot->cosT, g.rotSin = rot->sinT, g.rotCols = rot->cols, g.rotHeadDim = rot->headDim, g.rotTableRows = rot->tableRows;
    g.rotTableF32 = rot->tableF32, g.rotSinSign = rot->sinSign;
  }
  dim3 grid((unsigned)(g.tilesM * g.tilesN), (unsigned)splits, (unsigned)p.batch);
  if (EPI == kEpiSiluMul) AMD_CHECK(g.vecEpilogue, "gated linear: output rows must allow 16-byte stores");
  if (EPI == kEpiPartial) AMD_CHECK(g.vecEpilogue && p.batch == 1 && partial, "split-K: needs the vector epilogue and one batch");
  if constexpr (EPI == kEpiLinear) {
    if (bT) {
      AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&gemmMfmaPipelinedKernel<T, EPI, 256, true>), (int)lds));
      hipLaunchKernelGGL((gemmMfmaPipelinedKernel<T, EPI, 256, true>), grid, dim3(kPipeThreads), lds, stream, g);
      AMD_LAUNCH_CHECK();
      return diopiSuccess;
    }
  }
  AMD_CHECK(!bT, "gemm: the in-place [K, N] operand is taken by the linear epilogue only");
  if constexpr (EPI != kEpiPartial) {
    // the 4-wave kernel: an even number of K tiles, 16-byte epilogue pieces, lane offsets that fit 31 bits
    if (g.vecEpilogue && p.K % (2 * kBK) == 0 && p.M * p.sAm * 2 < (int64_t(1) << 31) && p.N * p.sBn * 2 < (int64_t(1) << 31)) {
      // one workgroup per CU (its LDS ring takes most of a CU's), each walking its share of the tiles
      const int resident = computeUnits() / 8 * 8;
      if (resident >= 8 && (int)grid.x > resident) grid.x = (unsigned)resident;
      if constexpr (EPI == kEpiLinear) {
        if (p.Cin) {
          // with an addend: the form that finds a quarter of each tile's addend in LDS (160 KiB: all of a CU's)
          constexpr size_t ldsAddend = lds + kAddendLdsBytes;
          AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&gemmMfma4WaveKernel<T, kEpiAddendLds>), (int)ldsAddend));
          hipLaunchKernelGGL((gemmMfma4WaveKernel<T, kEpiAddendLds>), grid, dim3(256), ldsAddend, stream, g);
          AMD_LAUNCH_CHECK();
          return diopiSuccess;
        }
      }
      constexpr size_t lds4 = lds + (EPI == kEpiRotaryLds ? kRotaryLdsBytes : 0);  // (160 KiB with the rotary tables: all of a CU's)
      AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&gemmMfma4WaveKernel<T, EPI>), (int)lds4));
      hipLaunchKernelGGL((gemmMfma4WaveKernel<T, EPI>), grid, dim3(256), lds4, stream, g);
      AMD_LAUNCH_CHECK();
      return diopiSuccess;
    }
  }
  if constexpr (EPI == kEpiRotaryLds) {
    setLastError("rotary epilogue: the form with tables in LDS exists for the 4-wave kernel only");
    return diopiErrorOccurred;
  } else if constexpr (EPI == kEpiColScale) {
    setLastError("column scale epilogue: exists for the 4-wave kernel only (see gemmAppliesColumnScale)");
    return diopiErrorOccurred;
  } else {
  hipLaunchKernelGGL((gemmMfmaPipelinedKernel<T, EPI>), grid, dim3(kPipeThreads), lds, stream, g);
  AMD_LAUNCH_CHECK();
  if (EPI == kEpiPartial) {
    const int64_t items = p.M * (p.N / 8);
    launchSplitKReduce<T>(stream, g, splits, items);
    AMD_LAUNCH_CHECK();
  }
  return diopiSuccess;
  }
}

// The 128 x 128 form of the pipelined kernel (4 waves, two workgroups per CU): linear epilogue, or fp32 partial
// products of a K split followed by the reduction pass.
template <typename T, int EPI = kEpiLinear>
static diopiError_t launchMfmaPipelined128(hipStream_t stream, const GemmProblem& p, float* partial = nullptr, int splits = 1,
                                           int kTilesPerSplit = 0, bool bT = false) {
  static_assert(EPI == kEpiLinear || EPI == kEpiPartial, "the 128 x 128 form has the linear and the split-K epilogues");
  MfmaArgs g;
  g.A = p.A, g.B = p.B, g.out = p.out, g.Cin = p.Cin, g.bias = p.bias;
  g.sAb = p.sAb, g.lda = p.sAm, g.sBb = p.sBb, g.ldb = p.sBn, g.sOb = p.sOb, g.ldo = p.sOm;
  g.sCb = p.sCb, g.sCm = p.sCm, g.sCn = p.sCn;
  g.M = (int)p.M, g.N = (int)p.N, g.K = (int)p.K;
  g.tilesM = (int)ceilDiv(p.M, 128), g.tilesN = (int)ceilDiv(p.N, 128);
  if (bT) g.ldb = p.sBk;
  g.alpha = p.alpha, g.beta = p.beta;
  auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool span32 = ((p.M - 1) * p.sOm + p.N) * (int64_t)sizeof(T) < (int64_t(1) << 31) &&
                      (!p.Cin || ((p.M - 1) * p.sCm + p.N) * (int64_t)sizeof(T) < (int64_t(1) << 31));
  g.vecEpilogue = p.N % 8 == 0 && p.sOm % 8 == 0 && p.sOb % 8 == 0 && al16(p.out) && span32 &&
                  (!p.Cin || (p.sCn == 1 && p.sCm % 8 == 0 && p.sCb % 8 == 0 && al16(p.Cin))) && (!p.bias || al16(p.bias));
  g.partial = partial;
  g.kTilesPerSplit = kTilesPerSplit;
  if (EPI == kEpiPartial) AMD_CHECK(g.vecEpilogue && p.batch == 1 && partial, "split-K: needs the vector epilogue and one batch");
  constexpr size_t lds = 2 * (size_t)(128 + 128) * kBK * sizeof(T);
  dim3 grid((unsigned)(g.tilesM * g.tilesN), (unsigned)splits, (unsigned)p.batch);
  if (bT) {
    AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&gemmMfmaPipelinedKernel<T, EPI, 128, true>), (int)lds));
    hipLaunchKernelGGL((gemmMfmaPipelinedKernel<T, EPI, 128, true>), grid, dim3(256), lds, stream, g);
  } else {
    AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&gemmMfmaPipelinedKernel<T, EPI, 128>), (int)lds));
    hipLaunchKernelGGL((gemmMfmaPipelinedKernel<T, EPI, 128>), grid, dim3(256), lds, stream, g);
  }
  AMD_LAUNCH_CHECK();
  if (EPI == kEpiPartial) {
    const int64_t items = p.M * (p.N / 8);
    launchSplitKReduce<T>(stream, g, splits, items);
    AMD_LAUNCH_CHECK();
  }
  return diopiSuccess;
}

template <typename T, int NTW, int KS, int G>
static diopiError_t launchSkinny(hipStream_t stream, const SkinnyArgs& a) {
  constexpr int CHUNK = kSkinnyRowsK / (16 * G);
  const size_t staged = (size_t)a.M * (std::min(a.K, CHUNK) + kSkinnyPad) * sizeof(T);
  const size_t lds = std::max(staged, (size_t)NTW * KS * G * 4 * 64 * sizeof(float));
  // the largest request (16 G rows x one chunk) covers every later one
  AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&gemmSkinnyKernel<T, NTW, KS, G>),
                          16 * G * (CHUNK + kSkinnyPad) * (int)sizeof(T)));
  const int tiles = (a.N + 15) / 16, splits = (a.K + a.kPerWg - 1) / a.kPerWg;
  dim3 grid((unsigned)((tiles + NTW - 1) / NTW), (unsigned)splits);
  hipLaunchKernelGGL((gemmSkinnyKernel<T, NTW, KS, G>), grid, dim3(NTW * KS * 64), lds, stream, a);
  AMD_LAUNCH_CHECK();
  if (a.partial) {
    MfmaArgs g;
    g.out = a.out, g.Cin = a.Cin, g.bias = a.bias, g.partial = a.partial;
    g.ldo = a.ldo, g.sCm = a.sCm, g.sCn = a.sCn;
    g.M = a.M, g.N = a.N, g.K = a.K, g.alpha = a.alpha, g.beta = a.beta;
    launchSplitKReduce<T>(stream, g, splits, (int64_t)a.M * (a.N / 8));
    AMD_LAUNCH_CHECK();
  }
  return diopiSuccess;
}

template <typename T, int G, int NTP, int WST, int XST>
static diopiError_t launchSkinnyLds(hipStream_t stream, const SkinnyArgs& a) {
  constexpr int BN = 32 * NTP;
  AMD_CHECK(a.colsPerWg >= 1 && a.colsPerWg <= BN, "skinny linear: %d columns per workgroup do not fit %d", a.colsPerWg, BN);
  const int lds = std::max((WST * BN + XST * G * 16) * kSkinnyLdsBK * (int)sizeof(T), 8 * G * NTP * 4 * 64 * (int)sizeof(float));
  AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&gemmSkinnyLdsKernel<T, G, NTP, WST, XST>), lds));
  const int splits = (a.K + a.kPerWg - 1) / a.kPerWg;
  hipLaunchKernelGGL((gemmSkinnyLdsKernel<T, G, NTP, WST, XST>), dim3((unsigned)((a.N + a.colsPerWg - 1) / a.colsPerWg), (unsigned)splits), dim3(512), lds, stream, a);
  AMD_LAUNCH_CHECK();
  if (a.partial) {
    MfmaArgs g;
    g.out = a.out, g.Cin = a.Cin, g.bias = a.bias, g.partial = a.partial;
    g.ldo = a.ldo, g.sCm = a.sCm, g.sCn = a.sCn;
    g.M = a.M, g.N = a.N, g.K = a.K, g.alpha = a.alpha, g.beta = a.beta;
    launchSplitKReduce<T>(stream, g, splits, (int64_t)a.M * (a.N / 8));
    AMD_LAUNCH_CHECK();
  }
  return diopiSuccess;
}

template <typename T, int NTW>
static diopiError_t launchSkinnyWide(hipStream_t stream, const SkinnyArgs& a) {
  const int lds = std::max(kSkinnyWBufs * 64 * kSkinnyWChunk * (int)sizeof(T), NTW * 4 * 4 * 4 * 64 * (int)sizeof(float));
  AMD_HIP(allowDynamicLds(reinterpret_cast<const void*>(&gemmSkinnyWideKernel<T, NTW>), lds));
  const int tiles = (a.N + 15) / 16;
  const int splits = (a.K + a.kPerWg - 1) / a.kPerWg;
  hipLaunchKernelGGL((gemmSkinnyWideKernel<T, NTW>), dim3((unsigned)((tiles + NTW - 1) / NTW), (unsigned)splits), dim3(NTW * 4 * 64), lds,
                     stream, a);
  AMD_LAUNCH_CHECK();
  if (a.partial) {
    MfmaArgs g;
    g.out = a.out, g.Cin = a.Cin, g.bias = a.bias, g.partial = a.partial;
    g.ldo = a.ldo, g.sCm = a.sCm, g.sCn = a.sCn;
    g.M = a.M, g.N = a.N, g.K = a.K, g.alpha = a.alpha, g.beta = a.beta;
    launchSplitKReduce<T>(stream, g, splits, (int64_t)a.M * (a.N / 8));
    AMD_LAUNCH_CHECK();
  }
  return diopiSuccess;
}

static bool mult8(int64_t v) { return (v & 7) == 0; }
static bool ptr16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T>
// With `rot` (a rotary epilogue) only the LDS-staged form qualifies: *handled tells the caller whether it ran.
static diopiError_t launchSkinnyForShape(diopiContextHandle_t ctx, hipStream_t stream, const GemmProblem& p,
                                         const RotaryEpilogue* rot = nullptr, bool* handled = nullptr) {
  SkinnyArgs a;
  a.A = p.A, a.B = p.B, a.Cin = p.Cin, a.bias = p.bias, a.out = p.out;
  a.lda = p.sAm, a.ldb = p.sBn, a.ldo = p.sOm, a.sCm = p.sCm, a.sCn = p.sCn;
  a.M = (int)p.M, a.N = (int)p.N, a.K = (int)p.K;
  a.alpha = p.alpha, a.beta = p.beta;
  a.partial = nullptr, a.kPerWg = a.K;
  a.siluMul = false, a.rotCols = 0;
  if (rot != nullptr) {
    a.rotCos = rot->cosT, a.rotSin = rot->sinT, a.rotCols = rot->cols, a.rotHeadDim = rot->headDim, a.rotTableRows = rot->tableRows;
    a.rotTableF32 = rot->tableF32, a.rotSinSign = rot->sinSign;
  }
  const int tiles = (a.N + 15) / 16, cus = computeUnits(), perCu = (tiles + cus - 1) / cus;
  // Both operands through LDS, see gemmSkinnyLdsKernel. The columns are dealt evenly over as many workgroups as there
  // are CUs (43 each at N = 11008, where 64-column blocks would leave a third of the CUs idle): a CU takes in about
  // 45 GB/s from a cold stream whatever the software pipeline depth, so the count of CUs at work sets the rate.
  // Measured cold against the forms below on K = 4096 (us, at 1 / 16 / 32 / 64 rows): N = 6144 13.7 -> 12.9,
  // 15.2 -> 13.4, 24.5 -> 14.9, 25.0 -> 18.2; N = 8192 16.6 -> 13.3, 18.0 -> 14.5, 22.5 -> 16.4, 27.3 -> 19.5;
  // N = 11008 18.5 -> 16.9, 20.4 -> 17.7, 33 -> 19.3, 30.4 -> 23.2; N = 22016 38.2 -> 30.1, 46.0 -> 31.9,
  // 52.9 -> 33.6, 55.7 -> 36.0. At N = 4096 (16 columns per workgroup: the activations are four times the weight
  // bytes on the way into a CU) only 17 to 32 rows gain (14.4 -> 12.7); one row loses (9.1 -> 11.0), and so does
  // everything narrower.
  // A 4096-wide weight (the o and down projections of a decode step) takes this form too with K split over grid.y, fp32
  // slices and the reduction pass: with K of 8192 and more at any row count, two slices up to 16 rows and four beyond
  // (us cold at K = 11008 against the register-layout kernels below: 1 row 23.9 -> 19.2, 16 rows 28.3 -> 20.3, 32 rows
  // 27.5 -> 21.6, 64 rows 34.0 -> 24.5 (27.7 with two slices); 64 x 4096 x 14336 34.2 -> 28.5). At K = 4096 two slices are
  // within the noise of what the other routes do (32 rows 12.4 -> 11.5 .. 12.3, 64 rows 14.5 -> 13.8 .. 14.8) and one row
  // loses (7.7 -> 10.0). The same split on wider weights loses (N = 11008: 23.0 -> 25.5 us, four ways 33.6).
  const bool canSplitLds = a.N % 8 == 0 && mult8(p.sOm) && ptr16(p.out) && (!p.bias || ptr16(p.bias)) &&
                           (!p.Cin || (p.sCn == 1 && mult8(p.sCm) && ptr16(p.Cin))) && rot == nullptr;
  // Weights of 5120 to 10239 rows take the K slices when K is at least twice their width (the down projections of
  // larger models; us, 1 / 16 / 32 / 64 rows: 5120 x 13824 30.7 -> 23.7, 31.8 -> 25.4, 36.1 -> 29.1, 46.5 -> 33.4;
  // 6144 x 16384 at 64 rows 55.7 -> 41.9; 8192 x 28672 at 64 rows 111.6 -> 95.2); a square 8192 x 8192 loses
  // (one row 21.5 -> 27.8).
  const bool narrow = a.N >= 4096 && (a.N < 5120 || (a.N < 10240 && a.K >= 2 * a.N)) && a.K % kSkinnyLdsBK == 0 && canSplitLds;
  const int narrowWays = narrow && a.K >= 8192 ? (a.M <= 16 ? 2 : 4) : 1;
  const bool narrowLongK = narrowWays > 1;
  if ((a.N >= 5120 || (a.N >= 4096 && a.M > 16 && a.M <= 32) || narrowLongK) &&
      ((int64_t)(a.N - 1) * a.ldb + a.K) * (int64_t)sizeof(T) < ((int64_t)1 << 31) &&
      ((int64_t)(a.M - 1) * a.lda + a.K) * (int64_t)sizeof(T) < ((int64_t)1 << 31)) {
    const int ways = narrowWays;
    const int wgs = std::max(1, cus / ways);
    const int rounds = (a.N + 128 * wgs - 1) / (128 * wgs);
    a.colsPerWg = (a.N + wgs * rounds - 1) / (wgs * rounds);
    if (ways > 1) {
      void* ws = nullptr;
      AMD_TRY(requireWorkspace(ctx, (int64_t)ways * a.M * a.N * 4, &ws));
      a.partial = static_cast<float*>(ws), a.kPerWg = ceilDiv(a.K / kSkinnyLdsBK, ways) * kSkinnyLdsBK;  // whole stages
    }
    if (rot != nullptr) a.colsPerWg = (a.colsPerWg + 1) & ~1;  // even: the two columns of a rotary pair stay together
    if (handled) *handled = true;
    if (a.colsPerWg > 64) {
      if (a.M <= 16) return launchSkinnyLds<T, 1, 4, 3, 3>(stream, a);
      if (a.M <= 32) return launchSkinnyLds<T, 2, 4, 3, 3>(stream, a);
      if (a.M <= 48) return launchSkinnyLds<T, 3, 4, 3, 3>(stream, a);
      return launchSkinnyLds<T, 4, 4, 3, 3>(stream, a);
    }
    if (a.M <= 16) return launchSkinnyLds<T, 1, 2, 4, 4>(stream, a);
    if (a.M <= 32) return launchSkinnyLds<T, 2, 2, 4, 4>(stream, a);
    if (a.M <= 48) return launchSkinnyLds<T, 3, 2, 4, 4>(stream, a);
    return launchSkinnyLds<T, 4, 2, 4, 4>(stream, a);
  }
  if (rot != nullptr) {
    if (handled) *handled = false;
    return diopiSuccess;
  }
  if (a.M <= 16) {
    // 16-column tiles per workgroup: about one workgroup per CU, the other waves of the 15 or 16 split K
    if (perCu >= 4) return launchSkinny<T, 4, 4, 1>(stream, a);
    if (perCu == 3) return launchSkinny<T, 3, 5, 1>(stream, a);
    if (perCu == 2) return launchSkinny<T, 2, 8, 1>(stream, a);
    return launchSkinny<T, 1, 16, 1>(stream, a);
  }
  // More than one group of rows: every workgroup stages all the rows, so with one 16-column tile per workgroup the
  // activations would be 2-4 times the weight bytes on the L2 -> CU path. Wider workgroups (up to 4 tiles) bring
  // that to 1:1, and K is split over grid.y as well, one staged chunk per workgroup, to keep the chip full; the
  // slices meet in fp32 workspace and the split-K reduction pass applies the epilogue.
  if (a.M > 32 && tiles >= 2 * cus && a.K >= 4096) {
    // Wide weights and a long K: whole-K workgroups with double-buffered activations, no partial products. Measured
    // at 64 rows, K = 4096, against the K-split form below: 24.2 against 25.4 us at N = 8192, 24.1 against 32.3 at
    // 9216, 24.2 against 33.5 at 11008, 24.8 against 34.6 at 12288, 30.9 against 44.4 at 16384, 46 against 61 at 22016
    // (66.6 against 110 at N = 12288, K = 11008); slower at K = 2048 (14.9 against 13.6 at N = 8192) and at K = 640
    // (10.1 against 8.3). One workgroup per CU at a time, each paying for its tiles' weights and once
    // for the activations (about one and a half tiles' worth): four tiles per workgroup, or three when that saves
    // rounds (768 tiles on 256 CUs: one round of three tiles instead of one of four).
    const int cost4 = ((tiles + 3) / 4 + cus - 1) / cus * (2 * 4 + 3), cost3 = ((tiles + 2) / 3 + cus - 1) / cus * (2 * 3 + 3);
    return cost3 < cost4 ? launchSkinnyWide<T, 3>(stream, a) : launchSkinnyWide<T, 4>(stream, a);
  }
  const bool canSplit = a.N % 8 == 0 && mult8(p.sOm) && ptr16(p.out) && (!p.bias || ptr16(p.bias)) &&
                        (!p.Cin || (p.sCn == 1 && mult8(p.sCm) && ptr16(p.Cin)));
  if (a.M > 32 && canSplit) {
    // Narrower weights with a long K: the same whole-chunk pipeline on K slices of at least 2048 (four chunks), four
    // tiles per workgroup, when the slices fill at least three quarters of the CUs; the slices meet in fp32 workspace.
    // 64 rows, against the single-chunk K-split form below: N = 4096 26.2 -> 24.2 us at K = 8192 and 37.6 -> 30.6 at
    // K = 11008 (four slices), N = 8192 25.0 -> 23.6 at K = 4096 and 45.4 -> 35.3 at K = 8192 (two slices); with
    // slices of 1024 or half the CUs idle (N = 4096, K = 4096: 17.9 and 22.2 against 15.1) it loses.
    const int wgs = (tiles + 3) / 4, ways = std::min(cus / std::max(wgs, 1), a.K / 2048);
    if (ways >= 2 && wgs * ways * 4 >= cus * 3) {
      const int per = ((a.K + ways - 1) / ways + 511) / 512 * 512, slices = (a.K + per - 1) / per;
      void* ws = nullptr;
      AMD_TRY(requireWorkspace(ctx, (int64_t)slices * a.M * a.N * 4, &ws));
      a.partial = static_cast<float*>(ws), a.kPerWg = per;
      return launchSkinnyWide<T, 4>(stream, a);
    }
  }
  const int groups = a.M <= 32 ? 2 : 4, chunk = kSkinnyRowsK / (16 * groups);
  const int splits = canSplit && groups == 4 ? (a.K + chunk - 1) / chunk : 1;  // two groups: measured no gain
  if (splits > 1) {
    void* ws = nullptr;
    AMD_TRY(requireWorkspace(ctx, (int64_t)splits * a.M * a.N * 4, &ws));
    a.partial = static_cast<float*>(ws), a.kPerWg = chunk;
  }
  const int want = std::max(1, std::min(4, tiles * splits / cus));  // tiles per workgroup that still fill the chip
  if (groups == 2) {
    if (want >= 4) return launchSkinny<T, 4, 4, 2>(stream, a);
    if (want == 3) return launchSkinny<T, 3, 5, 2>(stream, a);
    if (want == 2) return launchSkinny<T, 2, 8, 2>(stream, a);
    return launchSkinny<T, 1, 16, 2>(stream, a);
  }
  if (want >= 4) return launchSkinny<T, 4, 4, 4>(stream, a);
  if (want == 3) return launchSkinny<T, 3, 5, 4>(stream, a);
  if (want == 2) return launchSkinny<T, 2, 8, 4>(stream, a);
  return launchSkinny<T, 1, 8, 4>(stream, a);
}


template <typename U>
static diopiError_t launchTranspose(hipStream_t stream, void* dst, const void* src, int64_t batch, int64_t rows,
                                    int64_t cols, int64_t sRow, int64_t sCol, int64_t sBatch) {
  dim3 grid((unsigned)ceilDiv(cols, 64), (unsigned)ceilDiv(rows, 64), (unsigned)batch);
  hipLaunchKernelGGL(transposeKernel<U>, grid, dim3(256), 0, stream, (U*)dst, (const U*)src, rows, cols, sRow, sCol,
                     sBatch, rows * cols);
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

diopiError_t transposeCopy(hipStream_t stream, void* dst, const void* src, int itemsize, int64_t batch, int64_t rows,
                           int64_t cols, int64_t sRow, int64_t sCol, int64_t sBatch) {
  AMD_CHECK(itemsize == 2 || itemsize == 4, "transpose: %d-byte elements are not supported", itemsize);
  AMD_CHECK(batch <= 65535 && ceilDiv(rows, 64) <= 65535, "transpose: %ld batches x %ld rows exceed the grid limits", (long)batch,
            (long)rows);
  if (itemsize == 2) return launchTranspose<uint16_t>(stream, dst, src, batch, rows, cols, sRow, sCol, sBatch);
  return launchTranspose<uint32_t>(stream, dst, src, batch, rows, cols, sRow, sCol, sBatch);
}

bool gemmAppliesColumnScale(const GemmProblem& p) {
  // the conditions under which runGemm below reaches the 4-wave kernel without touching the operands
  const bool half = p.dtype == diopi_dtype_bfloat16 || p.dtype == diopi_dtype_float16;
  if (!half || p.batch != 1 || p.Cin || p.bias || p.K <= 0 || p.M >= (int64_t(1) << 31) || p.N >= (int64_t(1) << 31)) return false;
  if (p.sAk != 1 || !mult8(p.sAm) || !ptr16(p.A) || p.sBk != 1 || !mult8(p.sBn) || !ptr16(p.B)) return false;
  if (p.M <= kSkinnyMaxM) return false;
  const bool big = ceilDiv(p.M, 256) * ceilDiv(p.N, 256) >= 144 && p.N > 128 && p.K > 2 * kBK;
  const bool fits2g = ((p.M - 1) * p.sAm + p.K) * 2 < (int64_t(1) << 31) && ((p.N - 1) * p.sBn + p.K) * 2 < (int64_t(1) << 31);
  if (!big || p.K % (2 * kBK) != 0 || !fits2g) return false;
  const bool vec = p.N % 8 == 0 && p.sOm % 8 == 0 && ptr16(p.out) && ((p.M - 1) * p.sOm + p.N) * 2 < (int64_t(1) << 31);
  return vec && p.M * p.sAm * 2 < (int64_t(1) << 31) && p.N * p.sBn * 2 < (int64_t(1) << 31);
}

diopiError_t runGemm(diopiContextHandle_t ctx, hipStream_t stream, GemmProblem p) {
  if (p.batch == 0 || p.M == 0 || p.N == 0) return diopiSuccess;
  AMD_CHECK(p.batch <= 65535, "gemm: batch %ld exceeds the grid limit", (long)p.batch);
  const bool half = p.dtype == diopi_dtype_bfloat16 || p.dtype == diopi_dtype_float16;
  if (half && p.K > 0 && mult8(p.K) && p.M < (int64_t(1) << 31) && p.N < (int64_t(1) << 31)) {
    const int64_t item = 2;
    // bring both operands to K-contiguous storage: dst[b, r, k] with rows M (or N)
    if (p.sAk != 1 || !mult8(p.sAm) || !mult8(p.sAb) || !ptr16(p.A)) {
      void* ws = nullptr;
      AMD_TRY(requireWorkspace(ctx, p.batch * p.M * p.K * item, &ws));
      // source viewed as [K rows, M cols] -> destination [M, K]
      AMD_TRY(launchTranspose<uint16_t>(stream, ws, p.A, p.batch, p.K, p.M, p.sAk, p.sAm, p.sAb));
      p.A = ws, p.sAk = 1, p.sAm = p.K, p.sAb = p.M * p.K;
    }
    // A second operand that lies as [K, N] with N contiguous (mm / bmm / matmul right-hand sides) stays where it is when
    // the problem goes to the pipelined tile kernels, which read that layout in place; everything else gets a
    // K-contiguous copy.
    // From about 6000 rows on a copy pays for itself: the 4-wave kernel, which wants K-contiguous operands, is 11 %
    // faster than the kernel that reads [K, N] (8192 x 4096 x 11008: 504 against 566 us, the copy of the weight 40).
    const bool bT = p.sBn == 1 && p.sBk != 1 && p.N > 1 && mult8(p.sBk) && mult8(p.sBb) && ptr16(p.B) && p.M > kSkinnyMaxM && p.M < 6144 &&
                    p.K % kBK == 0 && p.K >= 2 * kBK && mult8(p.N) && ((p.K - 1) * p.sBk + p.N) * item < (int64_t(1) << 31) &&
                    ((p.M - 1) * p.sAm + p.K) * item < (int64_t(1) << 31);
    if (!bT && (p.sBk != 1 || !mult8(p.sBn) || !mult8(p.sBb) || !ptr16(p.B))) {
      void* ws = nullptr;
      AMD_TRY(requireWorkspace(ctx, p.batch * p.N * p.K * item, &ws));
      int64_t sbb = p.sBb;
      int64_t nb = p.batch;
      if (sbb == 0) nb = 1;  // a shared (broadcast) weight is transposed once
      AMD_TRY(launchTranspose<uint16_t>(stream, ws, p.B, nb, p.K, p.N, p.sBk, p.sBn, sbb));
      p.B = ws, p.sBk = 1, p.sBn = p.K, p.sBb = (sbb == 0) ? 0 : p.N * p.K;
    }
    // up to 32 rows always; up to 64 while N is moderate or K is long enough for the whole-K form (measured at 64
    // rows, K = 4096: K-split form + reduction pass 16 us against 50 us for the split-K tiled kernel at N = 4096, 36
    // against 52 at N = 12288, 63 against 51 at N = 22016, where the whole-K form takes 46)
    if (p.batch == 1 && (p.M <= 32 || (p.M <= kSkinnyMaxM && (p.N <= 16384 || p.K >= 4096))) && p.K % kSkinnyStep == 0 && p.N >= 16 &&
        ((p.M - 1) * p.sAm + p.K) * item < (int64_t(1) << 31))
      return p.dtype == diopi_dtype_bfloat16 ? launchSkinnyForShape<bf16_t>(ctx, stream, p)
                                             : launchSkinnyForShape<half_t>(ctx, stream, p);
    // from 144 tiles (56 % of the CUs in one round) the large-tile kernel beats the 128 x 128 one even unsplit
    // (a matrix at most 128 columns wide would leave half of every 256-wide tile empty: it takes the 128 x 128 form)
    // and so does a product of only two K tiles, which is all tile turnover: two workgroups per CU overlap one tile's
    // stores with the other's loads (bmm [128, 2048, 128] x [128, 128, 2048]: 421 -> 368 us)
    const bool big = ceilDiv(p.M, 256) * ceilDiv(p.N, 256) * p.batch >= 144 && p.N > 128 && p.K > 2 * kBK;
    const bool fits2g = bT || (((p.M - 1) * p.sAm + p.K) * 2 < (int64_t(1) << 31) && ((p.N - 1) * p.sBn + p.K) * 2 < (int64_t(1) << 31));
    if (big && p.K % kBK == 0 && p.K >= 2 * kBK && fits2g) {
      if (p.colScale)
        return p.dtype == diopi_dtype_bfloat16 ? launchMfmaPipelined<bf16_t, kEpiColScale>(stream, p)
                                               : launchMfmaPipelined<half_t, kEpiColScale>(stream, p);
      return p.dtype == diopi_dtype_bfloat16 ? launchMfmaPipelined<bf16_t>(stream, p, nullptr, 1, 0, nullptr, bT)
                                             : launchMfmaPipelined<half_t>(stream, p, nullptr, 1, 0, nullptr, bT);
    }
    AMD_CHECK(!p.colScale, "gemm: a column scale was set on a problem gemmAppliesColumnScale does not accept");
    // In between (too few 256 x 256 tiles for the chip, too many rows for the weight-streaming kernel): the same
    // large-tile kernel with K split over grid.y, fp32 partial products in workspace and a reduction pass.
    // In between (too few 256 x 256 tiles for the chip, too many rows for the weight-streaming kernels): the 128 x 128
    // form of the pipelined kernel, two workgroups per CU, and when even its tiles are fewer than the 2 x CUs the chip
    // holds, K split over grid.y with fp32 partial products in workspace and a reduction pass. Measured against
    // the 256 x 256 tiles split over K that this replaces (rows x 4096 x 4096, us): 128 rows 23.6 -> 21.5, 256 33.5 -> 22.3,
    // 512 37.4 -> 27.9, 1024 48.0 -> 41.7, 2048 71.3 -> 58.0; x 22016 x 4096: 128 rows 51.0 -> 38.8; K = 11008: 256 rows 45.0 -> 35.9.
    if (!big && p.K % kBK == 0 && p.K >= 2 * kBK && fits2g) {
      const int64_t tiles128 = ceilDiv(p.M, 128) * ceilDiv(p.N, 128) * p.batch;
      const bool vecOk = p.N % 8 == 0 && p.sOm % 8 == 0 && ptr16(p.out) && (!p.Cin || (p.sCn == 1 && p.sCm % 8 == 0 && ptr16(p.Cin))) &&
                         (!p.bias || ptr16(p.bias)) && p.M * p.N * 4 < (int64_t(1) << 31);
      int per = 0;
      const int splits = p.batch == 1 && vecOk ? splitKWays(tiles128, p.K / kBK, &per) : 1;
      if (splits >= 2) {
        void* ws = nullptr;
        AMD_TRY(requireWorkspace(ctx, (int64_t)splits * p.M * p.N * 4, &ws));
        return p.dtype == diopi_dtype_bfloat16 ? launchMfmaPipelined128<bf16_t, kEpiPartial>(stream, p, static_cast<float*>(ws), splits, per, bT)
                                               : launchMfmaPipelined128<half_t, kEpiPartial>(stream, p, static_cast<float*>(ws), splits, per, bT);
      }
      return p.dtype == diopi_dtype_bfloat16 ? launchMfmaPipelined128<bf16_t>(stream, p, nullptr, 1, 0, bT)
                                             : launchMfmaPipelined128<half_t>(stream, p, nullptr, 1, 0, bT);
    }
    AMD_CHECK(!bT, "gemm: no kernel took the in-place [K, N] operand");
    if (p.dtype == diopi_dtype_bfloat16) {
      return big ? launchMfma<bf16_t, 256, 256>(stream, p) : launchMfma<bf16_t, 128, 128>(stream, p);
    }
    return big ? launchMfma<half_t, 256, 256>(stream, p) : launchMfma<half_t, 128, 128>(stream, p);
  }
  if (p.dtype == diopi_dtype_float64) {
    dim3 grid((unsigned)ceilDiv(p.N, 256), (unsigned)p.M, (unsigned)p.batch);
    AMD_CHECK(p.M <= 65535, "gemm(float64): M exceeds the grid limit");
    hipLaunchKernelGGL(gemmFmaKernelF64, grid, dim3(256), 0, stream, p);
    AMD_LAUNCH_CHECK();
    return diopiSuccess;
  }
  if (p.dtype == diopi_dtype_float32 && p.M >= 32 && p.N >= 32 && f32MfmaEligible(p)) {
    // 128 x 128 tiles (less LDS traffic per product: 138 against 121 TFLOP/s at 2048 x 4096 x 4096) when their count
    // fills whole rounds of one workgroup per compute unit to at least 90 %; 64 x 64 tiles, whose rounds are four
    // times finer, otherwise (384 big tiles: 103 against 119 TFLOP/s)
    const int64_t tiles128 = ceilDiv(p.M, 128) * ceilDiv(p.N, 128) * p.batch, cus = computeUnits();
    const bool big = tiles128 >= cus && 10 * tiles128 >= 9 * ceilDiv(tiles128, cus) * cus;
    const int tile = big ? 128 : 64;
    dim3 grid((unsigned)(ceilDiv(p.N, tile) * ceilDiv(p.M, tile)), 1, (unsigned)p.batch);
    if (p.sAk == 1 && p.K % 32 == 0) {  // tiles straight into LDS
      if (p.sBk == 1) {
        if (big) hipLaunchKernelGGL((gemmMfmaF32DirectKernel<2, true>), grid, dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((gemmMfmaF32DirectKernel<1, true>), grid, dim3(256), 0, stream, p);
      } else {
        if (big) hipLaunchKernelGGL((gemmMfmaF32DirectKernel<2, false>), grid, dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((gemmMfmaF32DirectKernel<1, false>), grid, dim3(256), 0, stream, p);
      }
      AMD_LAUNCH_CHECK();
      return diopiSuccess;
    }
    auto launch = [&](auto aByK, auto bByK) {
      if (big)
        hipLaunchKernelGGL((gemmMfmaF32Kernel<2, kF32BKBig, decltype(aByK)::value, decltype(bByK)::value>), grid, dim3(256), 0, stream, p);
      else
        hipLaunchKernelGGL((gemmMfmaF32Kernel<1, 16, decltype(aByK)::value, decltype(bByK)::value>), grid, dim3(256), 0, stream, p);
    };
    if (p.sAk == 1 && p.sBk == 1) launch(std::true_type{}, std::true_type{});
    else if (p.sAk == 1) launch(std::true_type{}, std::false_type{});
    else if (p.sBk == 1) launch(std::false_type{}, std::true_type{});
    else launch(std::false_type{}, std::false_type{});
    AMD_LAUNCH_CHECK();
    return diopiSuccess;
  }
  AMD_CHECK(ceilDiv(p.M, 64) <= 65535, "gemm: M exceeds the grid limit of the FMA engine");
  dim3 grid((unsigned)ceilDiv(p.N, 64), (unsigned)ceilDiv(p.M, 64), (unsigned)p.batch);
  switch (p.dtype) {
    case diopi_dtype_float32: hipLaunchKernelGGL(gemmFmaKernel<float>, grid, dim3(256), 0, stream, p); break;
    case diopi_dtype_bfloat16: hipLaunchKernelGGL(gemmFmaKernel<bf16_t>, grid, dim3(256), 0, stream, p); break;
    case diopi_dtype_float16: hipLaunchKernelGGL(gemmFmaKernel<half_t>, grid, dim3(256), 0, stream, p); break;
    default: setLastError("gemm: unsupported dtype %s", dtypeName(p.dtype)); return diopiErrorOccurred;
  }
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

// ------------------------------------------------------------- entry helpers --
// Folds leading dims of a dense-enough view into one batch dim; returns false if impossible.
// ------------------------------------------------------- gated SiLU linear ----
// Second pass of the two-pass form: out[m, 32 b + j] = silu(gu[m, 64 b + j]) * gu[m, 64 b + 32 + j].
template <typename T>
__global__ __launch_bounds__(256) void gatedSiluKernel(T* __restrict__ out, const T* __restrict__ gu, int64_t rows,
                                                        int64_t f, int64_t ldo) {
  const int64_t total = rows * f;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t m = i / f, c = i - m * f;
    const T* row = gu + m * 2 * f + (c >> 5) * 64 + (c & 31);
    const float g = static_cast<float>(row[0]), u = static_cast<float>(row[32]);
    out[m * ldo + c] = static_cast<T>(g * __builtin_amdgcn_rcpf(1.f + __expf(-g)) * u);
  }
}

// out[M, F] = silu(A W_gate^T) * (A W_up^T) with the two weights interleaved in one [2F, K] matrix (see
// diopiLinearSiluMul). One launch of the large-tile kernel when the problem qualifies, else GEMM + pass.
static diopiError_t runGatedSiluGemm(diopiContextHandle_t ctx, hipStream_t stream, GemmProblem p) {
  const int64_t f = p.N / 2;
  const bool half = p.dtype == diopi_dtype_bfloat16 || p.dtype == diopi_dtype_float16;
  const bool direct = half && p.batch == 1 && p.sAk == 1 && mult8(p.sAm) && ptr16(p.A) && p.sBk == 1 && mult8(p.sBn) && ptr16(p.B) &&
                      ceilDiv(p.M, 256) * ceilDiv(p.N, 256) >= 144 && p.K % kBK == 0 && p.K >= 2 * kBK &&
                      ((p.M - 1) * p.sAm + p.K) * 2 < (int64_t(1) << 31) && ((p.N - 1) * p.sBn + p.K) * 2 < (int64_t(1) << 31) &&
                      mult8(p.sOm) && ptr16(p.out) && p.M < (int64_t(1) << 31) && p.N < (int64_t(1) << 31);
  if (direct) {
    return p.dtype == diopi_dtype_bfloat16 ? launchMfmaPipelined<bf16_t, kEpiSiluMul>(stream, p)
                                           : launchMfmaPipelined<half_t, kEpiSiluMul>(stream, p);
  }
  // decode-sized: the weight-streaming kernel that stages both operands through LDS applies the gate to its sums
  if (half && p.batch == 1 && p.M <= kSkinnyMaxM && p.K % kSkinnyLdsBK == 0 && p.N % 64 == 0 && p.N >= 4096 && p.sAk == 1 &&
      mult8(p.sAm) && ptr16(p.A) && p.sBk == 1 && mult8(p.sBn) && ptr16(p.B) && p.Cin == nullptr && p.bias == nullptr &&
      p.alpha == 1.f && ((p.M - 1) * p.sAm + p.K) * 2 < (int64_t(1) << 31) && ((p.N - 1) * p.sBn + p.K) * 2 < (int64_t(1) << 31)) {
    SkinnyArgs a;
    a.A = p.A, a.B = p.B, a.Cin = nullptr, a.bias = nullptr, a.out = p.out;
    a.lda = p.sAm, a.ldb = p.sBn, a.ldo = p.sOm, a.sCm = 0, a.sCn = 0;
    a.M = (int)p.M, a.N = (int)p.N, a.K = (int)p.K;
    a.alpha = 1.f, a.beta = 0.f, a.partial = nullptr, a.kPerWg = a.K, a.siluMul = true, a.rotCols = 0;
    // whole blocks of 64 columns per workgroup: 128 while that still gives half the CUs a workgroup
    a.colsPerWg = p.N / 128 >= computeUnits() / 2 ? 128 : 64;
    const bool bf = p.dtype == diopi_dtype_bfloat16;
#define SKINNY_SILU(G, NTP, WST, XST) \
  return bf ? launchSkinnyLds<bf16_t, G, NTP, WST, XST>(stream, a) : launchSkinnyLds<half_t, G, NTP, WST, XST>(stream, a)
    if (a.colsPerWg == 128) {
      if (a.M <= 16) SKINNY_SILU(1, 4, 3, 3);
      if (a.M <= 32) SKINNY_SILU(2, 4, 3, 3);
      if (a.M <= 48) SKINNY_SILU(3, 4, 3, 3);
      SKINNY_SILU(4, 4, 3, 3);
    }
    if (a.M <= 16) SKINNY_SILU(1, 2, 4, 4);
    if (a.M <= 32) SKINNY_SILU(2, 2, 4, 4);
    if (a.M <= 48) SKINNY_SILU(3, 2, 4, 4);
    SKINNY_SILU(4, 2, 4, 4);
#undef SKINNY_SILU
  }
  // two passes: the full-width projection into workspace, then the gate
  void* ws = nullptr;
  const int64_t item = dtypeSize(p.dtype);
  AMD_TRY(requireWorkspace(ctx, p.M * p.N * item, &ws));
  GemmProblem q = p;
  void* finalOut = p.out;
  const int64_t ldo = p.sOm;
  q.out = ws, q.sOm = p.N, q.sOb = p.M * p.N;
  AMD_TRY(runGemm(ctx, stream, q));
  int64_t blocks = std::min<int64_t>(ceilDiv(p.M * f, 256), 65536);
  switch (p.dtype) {
    case diopi_dtype_bfloat16:
      hipLaunchKernelGGL(gatedSiluKernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, (bf16_t*)finalOut, (const bf16_t*)ws, p.M, f, ldo);
      break;
    case diopi_dtype_float16:
      hipLaunchKernelGGL(gatedSiluKernel<half_t>, dim3((unsigned)blocks), dim3(256), 0, stream, (half_t*)finalOut, (const half_t*)ws, p.M, f, ldo);
      break;
    case diopi_dtype_float32:
      hipLaunchKernelGGL(gatedSiluKernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, (float*)finalOut, (const float*)ws, p.M, f, ldo);
      break;
    default: setLastError("gated linear: unsupported dtype %s", dtypeName(p.dtype)); return diopiErrorOccurred;
  }
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

static bool foldBatch(const TensorView& t, int lead, int64_t* count, int64_t* stride) {
  int64_t n = 1, s = 0;
  bool have = false;
  for (int d = lead - 1; d >= 0; --d) {
    if (t.shape[d] == 1) continue;
    if (!have) s = t.stride[d], have = true;
    else if (t.stride[d] != s * n) return false;
    n *= t.shape[d];
  }
  *count = n;
  *stride = have ? s : 0;
  return true;
}

struct MatOperand {
  TensorView v;
  int64_t batch = 1, sb = 0;
};

// out[..., M, N] = A[..., M, K] @ B[..., K, N] with equal (or size-1 / absent) batch dims.
static diopiError_t batchedMatmul(diopiContextHandle_t ctx, hipStream_t stream, const TensorView& out,
                                  const TensorView& a, const TensorView& b, const TensorView* cin, const TensorView* bias,
                                  float alpha, float beta, bool bIsNK) {
  AMD_CHECK(a.ndim >= 2 && b.ndim >= 2 && out.ndim >= 2, "matmul: operands must have rank >= 2 here");
  AMD_CHECK(a.dtype == b.dtype && a.dtype == out.dtype, "matmul: dtypes differ (%s, %s -> %s)", dtypeName(a.dtype),
            dtypeName(b.dtype), dtypeName(out.dtype));
  GemmProblem p;
  p.dtype = a.dtype;
  p.M = a.shape[a.ndim - 2];
  p.K = a.shape[a.ndim - 1];
  int64_t bK = bIsNK ? b.shape[b.ndim - 1] : b.shape[b.ndim - 2];
  p.N = bIsNK ? b.shape[b.ndim - 2] : b.shape[b.ndim - 1];
  AMD_CHECK(bK == p.K, "matmul: inner dims differ (%ld vs %ld)", (long)p.K, (long)bK);
  AMD_CHECK(out.shape[out.ndim - 2] == p.M && out.shape[out.ndim - 1] == p.N, "matmul: output is [%ld,%ld], expected [%ld,%ld]",
            (long)out.shape[out.ndim - 2], (long)out.shape[out.ndim - 1], (long)p.M, (long)p.N);
  int64_t ob, os, ab, as, bb, bs;
  TensorView oc = out, ac = a, bc = b;
  bool outTemp = false;
  if (!(out.stride[out.ndim - 1] == 1 || p.N == 1) || !foldBatch(out, out.ndim - 2, &ob, &os)) {
    diopiTensorHandle_t th;
    AMD_TRY(requireTensor(ctx, out.shape, out.ndim, out.dtype, &th, &oc));
    outTemp = true;
    foldBatch(oc, oc.ndim - 2, &ob, &os);
  }
  if (!foldBatch(ac, ac.ndim - 2, &ab, &as)) {
    AMD_TRY(makeContiguous(ctx, stream, a, &ac));
    foldBatch(ac, ac.ndim - 2, &ab, &as);
  }
  if (!foldBatch(bc, bc.ndim - 2, &bb, &bs)) {
    AMD_TRY(makeContiguous(ctx, stream, b, &bc));
    foldBatch(bc, bc.ndim - 2, &bb, &bs);
  }
  AMD_CHECK((ab == ob || ab == 1) && (bb == ob || bb == 1), "matmul: batch dims %ld and %ld do not match output batch %ld",
            (long)ab, (long)bb, (long)ob);
  p.batch = ob;
  p.A = ac.data, p.sAb = ab == 1 ? 0 : as, p.sAm = ac.stride[ac.ndim - 2], p.sAk = ac.stride[ac.ndim - 1];
  p.B = bc.data, p.sBb = bb == 1 ? 0 : bs;
  if (bIsNK) p.sBn = bc.stride[bc.ndim - 2], p.sBk = bc.stride[bc.ndim - 1];
  else p.sBk = bc.stride[bc.ndim - 2], p.sBn = bc.stride[bc.ndim - 1];
  p.out = oc.data, p.sOb = os, p.sOm = oc.stride[oc.ndim - 2];
  if (p.M == 1) p.sOm = p.N;  // a single row: its stride is never used, keep it sane
  // A shared A with per-batch B cannot fold; a shared B with per-batch A folds the batch into M.
  if (p.sBb == 0 && p.batch > 1 && p.sAb == p.M * p.sAm && p.sOb == p.M * p.sOm && cin == nullptr) {
    p.M *= p.batch;
    p.batch = 1;
    p.sAb = p.sOb = 0;
  }
  p.alpha = alpha, p.beta = beta;
  if (bias) p.bias = bias->data;
  if (cin && beta != 0.f) {
    // broadcast Cin against [batch, M, N]
    const TensorView& c = *cin;
    AMD_CHECK(c.dtype == out.dtype, "matmul: addend dtype differs from output dtype");
    p.Cin = c.data;
    auto ext = [&](int fromEnd) { return c.ndim >= fromEnd ? c.shape[c.ndim - fromEnd] : 1; };
    auto str = [&](int fromEnd) { return (c.ndim >= fromEnd && c.shape[c.ndim - fromEnd] != 1) ? c.stride[c.ndim - fromEnd] : 0; };
    AMD_CHECK(ext(1) == p.N || ext(1) == 1, "matmul: addend last dim %ld does not broadcast to %ld", (long)ext(1), (long)p.N);
    AMD_CHECK(ext(2) == p.M || ext(2) == 1, "matmul: addend rows %ld do not broadcast to %ld", (long)ext(2), (long)p.M);
    p.sCn = str(1), p.sCm = str(2);
    if (c.ndim > 2) {
      TensorView lead = c;
      int64_t cb, cs;
      AMD_CHECK(foldBatch(lead, c.ndim - 2, &cb, &cs) && (cb == p.batch || cb == 1), "matmul: addend batch dims do not match");
      p.sCb = cb == 1 ? 0 : cs;
    }
  }
  AMD_TRY(runGemm(ctx, stream, p));
  if (outTemp) AMD_TRY(stridedCopy(stream, oc, out));
  return diopiSuccess;
}

}  // namespace amd

using namespace amd;
#define GEMM_EXPORT extern "C" __attribute__((visibility("default")))

GEMM_EXPORT diopiError_t diopiMm(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t aH,
                                 diopiConstTensorHandle_t bH) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, a, b;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(aH, &a, "input"));
  AMD_TRY(getView(bH, &b, "mat2"));
  AMD_CHECK(out.defined() && a.defined() && b.defined(), "diopiMm: null tensor");
  AMD_CHECK(a.ndim == 2 && b.ndim == 2 && out.ndim == 2, "diopiMm: operands must be 2-D");
  return batchedMatmul(ctx, stream, out, a, b, nullptr, nullptr, 1.f, 0.f, false);
}

GEMM_EXPORT diopiError_t diopiBmm(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t aH,
                                  diopiConstTensorHandle_t bH) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, a, b;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(aH, &a, "input"));
  AMD_TRY(getView(bH, &b, "mat2"));
  AMD_CHECK(out.defined() && a.defined() && b.defined(), "diopiBmm: null tensor");
  AMD_CHECK(a.ndim == 3 && b.ndim == 3 && out.ndim == 3, "diopiBmm: operands must be 3-D");
  AMD_CHECK(a.shape[0] == b.shape[0] && a.shape[0] == out.shape[0], "diopiBmm: batch sizes differ");
  return batchedMatmul(ctx, stream, out, a, b, nullptr, nullptr, 1.f, 0.f, false);
}

// Views a tensor with extra unit dims so that 1-D operands become matrices.
static TensorView unsqueeze(const TensorView& t, int at) {
  TensorView r = t;
  for (int d = t.ndim; d > at; --d) r.shape[d] = t.shape[d - 1], r.stride[d] = t.stride[d - 1];
  r.shape[at] = 1;
  r.stride[at] = 0;
  r.ndim = t.ndim + 1;
  return r;
}

GEMM_EXPORT diopiError_t diopiMatmul(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t aH,
                                     diopiConstTensorHandle_t bH) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, a, b;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(aH, &a, "input"));
  AMD_TRY(getView(bH, &b, "other"));
  AMD_CHECK(out.defined() && a.defined() && b.defined(), "diopiMatmul: null tensor");
  AMD_CHECK(a.ndim >= 1 && b.ndim >= 1, "diopiMatmul: operands must have at least one dim");
  AMD_CHECK(a.ndim < kMaxDims && b.ndim < kMaxDims && out.ndim + 2 <= kMaxDims, "diopiMatmul: rank too large");
  // torch.matmul: a 1-D left operand gains a leading unit dim, a 1-D right operand a trailing one
  TensorView a2 = a, b2 = b, o2 = out;
  if (a.ndim == 1) a2 = unsqueeze(a, 0);
  if (b.ndim == 1) b2 = unsqueeze(b, 1);
  if (a.ndim == 1 && b.ndim == 1) {
    o2 = unsqueeze(unsqueeze(out, out.ndim), out.ndim + 1);
  } else if (a.ndim == 1) {
    o2 = unsqueeze(out, out.ndim - 1);
  } else if (b.ndim == 1) {
    o2 = unsqueeze(out, out.ndim);
  }
  // broadcast batch dims: expand both to the output's batch shape when they differ
  int nb = o2.ndim - 2;
  auto expandTo = [&](const TensorView& t, TensorView* e) {
    *e = o2;
    e->data = t.data;
    e->dtype = t.dtype;
    e->itemsize = t.itemsize;
    int shift = o2.ndim - t.ndim;
    for (int d = 0; d < o2.ndim; ++d) {
      if (d >= nb) {
        e->shape[d] = t.shape[d - shift];
        e->stride[d] = t.stride[d - shift];
      } else if (d < shift || t.shape[d - shift] == 1) {
        e->stride[d] = 0;
      } else {
        e->stride[d] = t.stride[d - shift];
      }
    }
    e->numel = 1;
    for (int d = 0; d < e->ndim; ++d) e->numel *= e->shape[d];
  };
  TensorView ae, be;
  AMD_CHECK(a2.ndim <= o2.ndim && b2.ndim <= o2.ndim, "diopiMatmul: output rank too small");
  expandTo(a2, &ae);
  expandTo(b2, &be);
  // fully shared operands keep a single copy (batch count 1); partially broadcast ones are materialised
  auto normalise = [&](TensorView& e, const TensorView& orig) -> diopiError_t {
    bool allZero = true, anyZero = false;
    for (int d = 0; d < nb; ++d) {
      if (e.shape[d] == 1) continue;
      if (e.stride[d] == 0) anyZero = true; else allZero = false;
    }
    if (anyZero && allZero) {
      for (int d = 0; d < nb; ++d) e.shape[d] = 1;
    } else if (anyZero) {
      TensorView dense;
      AMD_TRY(makeContiguous(ctx, stream, e, &dense));
      e = dense;
    }
    (void)orig;
    return diopiSuccess;
  };
  AMD_TRY(normalise(ae, a2));
  AMD_TRY(normalise(be, b2));
  return batchedMatmul(ctx, stream, o2, ae, be, nullptr, nullptr, 1.f, 0.f, false);
}

GEMM_EXPORT diopiError_t diopiAddmm(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t inH,
                                    diopiConstTensorHandle_t m1H, diopiConstTensorHandle_t m2H,
                                    const diopiScalar_t* beta, const diopiScalar_t* alpha) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, in, a, b;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(inH, &in, "input"));
  AMD_TRY(getView(m1H, &a, "mat1"));
  AMD_TRY(getView(m2H, &b, "mat2"));
  AMD_CHECK(out.defined() && in.defined() && a.defined() && b.defined(), "diopiAddmm: null tensor");
  AMD_CHECK(a.ndim == 2 && b.ndim == 2 && out.ndim == 2 && in.ndim <= 2, "diopiAddmm: bad ranks");
  return batchedMatmul(ctx, stream, out, a, b, &in, nullptr, (float)scalarToDouble(alpha, 1.0),
                       (float)scalarToDouble(beta, 1.0), false);
}

GEMM_EXPORT diopiError_t diopiBaddbmm(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t inH,
                                      diopiConstTensorHandle_t b1H, diopiConstTensorHandle_t b2H, double beta,
                                      double alpha) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, in, a, b;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(inH, &in, "input"));
  AMD_TRY(getView(b1H, &a, "batch1"));
  AMD_TRY(getView(b2H, &b, "batch2"));
  AMD_CHECK(out.defined() && in.defined() && a.defined() && b.defined(), "diopiBaddbmm: null tensor");
  AMD_CHECK(a.ndim == 3 && b.ndim == 3 && out.ndim == 3 && in.ndim <= 3, "diopiBaddbmm: bad ranks");
  return batchedMatmul(ctx, stream, out, a, b, &in, nullptr, (float)alpha, (float)beta, false);
}

GEMM_EXPORT diopiError_t diopiLinear(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t inH,
                                     diopiConstTensorHandle_t wH, diopiConstTensorHandle_t biasH) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, in, w, bias;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(inH, &in, "input"));
  AMD_TRY(getView(wH, &w, "weight"));
  AMD_TRY(getView(biasH, &bias, "bias"));
  AMD_CHECK(out.defined() && in.defined() && w.defined(), "diopiLinear: null tensor");
  AMD_CHECK(w.ndim == 2 && in.ndim >= 1 && out.ndim == in.ndim, "diopiLinear: weight must be [N, K], out shaped like input");
  AMD_CHECK(in.ndim + 1 <= kMaxDims, "diopiLinear: rank too large");
  TensorView cb;
  if (bias.defined()) {
    AMD_CHECK(bias.numel == w.shape[0] && bias.dtype == out.dtype, "diopiLinear: bias must hold N elements of the output dtype");
    AMD_TRY(makeContiguous(ctx, stream, bias, &cb));
  }
  TensorView in2 = in, out2 = out;
  if (in.ndim == 1) in2 = unsqueeze(in, 0), out2 = unsqueeze(out, 0);
  return batchedMatmul(ctx, stream, out2, in2, w, nullptr, bias.defined() ? &cb : nullptr, 1.f, 0.f, true);
}

// out[..., F] = silu(input W_gate^T) * (input W_up^T), weight = the two [F, K] matrices interleaved in blocks
// of 32 rows (see functions_ext.h). The reference model runs two linears, silu and mul
// (dicp/test/model/llama/model.py:196-200; diopi_functions.yaml:902-909,1767-1775,181-196).
GEMM_EXPORT diopiError_t diopiLinearSiluMul(diopiContextHandle_t ctx, diopiTensorHandle_t outH,
                                            diopiConstTensorHandle_t inH, diopiConstTensorHandle_t wH) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, in, w;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(inH, &in, "input"));
  AMD_TRY(getView(wH, &w, "weight"));
  AMD_CHECK(out.defined() && in.defined() && w.defined(), "diopiLinearSiluMul: null tensor");
  AMD_CHECK(w.ndim == 2 && in.ndim >= 1 && out.ndim == in.ndim, "diopiLinearSiluMul: weight must be [2F, K], out shaped like input");
  AMD_CHECK(in.dtype == out.dtype && w.dtype == out.dtype, "diopiLinearSiluMul: input, weight and out must share a dtype");
  const int64_t k = in.shape[in.ndim - 1], f = out.shape[out.ndim - 1];
  AMD_CHECK(w.shape[1] == k && w.shape[0] == 2 * f, "diopiLinearSiluMul: weight is [%ld, %ld], expected [%ld, %ld]",
            (long)w.shape[0], (long)w.shape[1], (long)(2 * f), (long)k);
  AMD_CHECK(f % 32 == 0, "diopiLinearSiluMul: %ld output channels are not a multiple of the 32-row interleave", (long)f);
  for (int d = 0; d + 1 < in.ndim; ++d)
    AMD_CHECK(in.shape[d] == out.shape[d], "diopiLinearSiluMul: leading extent mismatch at dim %d", d);
  if (out.numel == 0) return diopiSuccess;
  TensorView cin, cw;
  AMD_TRY(makeContiguous(ctx, stream, in, &cin));
  AMD_TRY(makeContiguous(ctx, stream, w, &cw));
  TensorView cout = out;
  const bool outTemp = !out.isContiguous();
  if (outTemp) {
    diopiTensorHandle_t th;
    AMD_TRY(requireTensor(ctx, out.shape, out.ndim, out.dtype, &th, &cout));
  }
  GemmProblem p;
  p.dtype = out.dtype;
  p.M = in.numel / k, p.N = 2 * f, p.K = k;
  p.A = cin.data, p.sAm = k, p.sAk = 1;
  p.B = cw.data, p.sBn = k, p.sBk = 1;
  p.out = cout.data, p.sOm = f;
  AMD_TRY(runGatedSiluGemm(ctx, stream, p));
  if (outTemp) AMD_TRY(stridedCopy(stream, cout, out));
  return diopiSuccess;
}

// out[..., N] = input W^T + bias, then the rotary embedding on the first rotary_cols columns viewed as heads of
// head_dim columns, with one table row per row of the flattened input (cos / sin of shape [rows, head_dim / 2]):
// the q and k heads of a stacked QKV projection come out rotated and v passes through. The reference model
// runs the projections and the rotation as separate steps (dicp/test/model/llama/model.py:108-160 with the
// interleaved rotation of :58-69; the half-split form is dicp/dicp/vendor/AscendGraph/ext_ops.py:24-33).
// One launch of the large-tile kernel for the interleaved form when the problem qualifies (the pairs of a head
// are then adjacent columns, which one lane holds), else the projection followed by the rotary kernel.
GEMM_EXPORT diopiError_t diopiLinearRotary(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t inH,
                                           diopiConstTensorHandle_t wH, diopiConstTensorHandle_t biasH,
                                           diopiConstTensorHandle_t cosH, diopiConstTensorHandle_t sinH,
                                           int64_t rotaryCols, int64_t headDim, bool conj, bool interleaved) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, in, w, bias, c, s;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(inH, &in, "input"));
  AMD_TRY(getView(wH, &w, "weight"));
  AMD_TRY(getView(biasH, &bias, "bias"));
  AMD_TRY(getView(cosH, &c, "cos"));
  AMD_TRY(getView(sinH, &s, "sin"));
  AMD_CHECK(out.defined() && in.defined() && w.defined() && c.defined() && s.defined(), "diopiLinearRotary: null tensor");
  AMD_CHECK(w.ndim == 2 && in.ndim >= 1 && out.ndim == in.ndim, "diopiLinearRotary: weight must be [N, K], out shaped like input");
  AMD_CHECK(in.dtype == out.dtype && w.dtype == out.dtype, "diopiLinearRotary: input, weight and out must share a dtype");
  const int64_t k = in.shape[in.ndim - 1], n = out.shape[out.ndim - 1];
  AMD_CHECK(w.shape[1] == k && w.shape[0] == n, "diopiLinearRotary: weight is [%ld, %ld], expected [%ld, %ld]", (long)w.shape[0],
            (long)w.shape[1], (long)n, (long)k);
  AMD_CHECK(headDim > 0 && headDim % 2 == 0 && rotaryCols >= 0 && rotaryCols <= n && rotaryCols % headDim == 0,
            "diopiLinearRotary: rotary_cols %ld must be a multiple of the even head_dim %ld and at most %ld", (long)rotaryCols,
            (long)headDim, (long)n);
  for (int d = 0; d + 1 < in.ndim; ++d) AMD_CHECK(in.shape[d] == out.shape[d], "diopiLinearRotary: leading extent mismatch at dim %d", d);
  if (out.numel == 0) return diopiSuccess;
  const int64_t rows = in.numel / k, half = headDim / 2;
  const int64_t tableRows = c.numel / half;
  AMD_CHECK(c.dtype == s.dtype && c.numel == s.numel && tableRows > 0 && c.numel == tableRows * half && rows % tableRows == 0,
            "diopiLinearRotary: cos and sin must both hold [t, %ld] values with t dividing the %ld rows", (long)half, (long)rows);
  TensorView cin, cw, cb, cc, cs;
  AMD_TRY(makeContiguous(ctx, stream, in, &cin));
  AMD_TRY(makeContiguous(ctx, stream, w, &cw));
  AMD_TRY(makeContiguous(ctx, stream, c, &cc));
  AMD_TRY(makeContiguous(ctx, stream, s, &cs));
  if (bias.defined()) {
    AMD_CHECK(bias.numel == n && bias.dtype == out.dtype, "diopiLinearRotary: bias must hold N elements of the output dtype");
    AMD_TRY(makeContiguous(ctx, stream, bias, &cb));
  }
  TensorView cout = out;
  const bool outTemp = !out.isContiguous();
  if (outTemp) {
    diopiTensorHandle_t th;
    AMD_TRY(requireTensor(ctx, out.shape, out.ndim, out.dtype, &th, &cout));
  }
  GemmProblem p;
  p.dtype = out.dtype;
  p.M = rows, p.N = n, p.K = k;
  p.A = cin.data, p.sAm = k, p.sAk = 1;
  p.B = cw.data, p.sBn = k, p.sBk = 1;
  p.out = cout.data, p.sOm = n;
  if (bias.defined()) p.bias = cb.data;
  const bool halfT = p.dtype == diopi_dtype_bfloat16 || p.dtype == diopi_dtype_float16;
  const bool tableOk = (cc.dtype == out.dtype || cc.dtype == diopi_dtype_float32) && ptr16(cc.data) && ptr16(cs.data) && half % 4 == 0 &&
                       tableRows * half * 4 < (int64_t(1) << 31);
  const bool direct = interleaved && rotaryCols > 0 && halfT && headDim % 8 == 0 && tableOk && mult8(k) && ptr16(p.A) && ptr16(p.B) &&
                      ceilDiv(p.M, 256) * ceilDiv(p.N, 256) >= 144 && k % kBK == 0 && k >= 2 * kBK && n % 8 == 0 && ptr16(p.out) &&
                      (!p.bias || ptr16(p.bias)) && p.M * k * 2 < (int64_t(1) << 31) && n * k * 2 < (int64_t(1) << 31) &&
                      p.M * n * 2 < (int64_t(1) << 31);
  if (direct) {
    RotaryEpilogue r;
    r.cosT = cc.data, r.sinT = cs.data, r.cols = (int)rotaryCols, r.headDim = (int)headDim, r.tableRows = (int)tableRows;
    r.tableF32 = cc.dtype == diopi_dtype_float32, r.sinSign = conj ? -1.f : 1.f;
    // (what launchMfmaPipelined asks of a problem before it takes the 4-wave kernel, whose LDS has room for the tables)
    const bool fourWave = k % (2 * kBK) == 0 && n % 8 == 0 && ptr16(p.out) && p.M * k * 2 < (int64_t(1) << 31) && n * k * 2 < (int64_t(1) << 31) &&
                          (p.M - 1) * n * 2 + n * 2 < (int64_t(1) << 31);
    if (!p.bias && r.cols % 32 == 0 && !r.tableF32 && r.headDim == 128 && fourWave)
      AMD_TRY(p.dtype == diopi_dtype_bfloat16 ? (launchMfmaPipelined<bf16_t, kEpiRotaryLds>(stream, p, nullptr, 1, 0, &r))
                                              : (launchMfmaPipelined<half_t, kEpiRotaryLds>(stream, p, nullptr, 1, 0, &r)));
    else if (!p.bias && r.cols % 32 == 0)
      AMD_TRY(p.dtype == diopi_dtype_bfloat16 ? (launchMfmaPipelined<bf16_t, kEpiRotaryUniform>(stream, p, nullptr, 1, 0, &r))
                                              : (launchMfmaPipelined<half_t, kEpiRotaryUniform>(stream, p, nullptr, 1, 0, &r)));
    else
      AMD_TRY(p.dtype == diopi_dtype_bfloat16 ? (launchMfmaPipelined<bf16_t, kEpiRotary>(stream, p, nullptr, 1, 0, &r))
                                              : (launchMfmaPipelined<half_t, kEpiRotary>(stream, p, nullptr, 1, 0, &r)));
  } else {
    // decode-sized: the weight-streaming kernel that stages both operands through LDS rotates its sums
    bool fused = false;
    if (interleaved && rotaryCols > 0 && halfT && tableOk && p.M <= kSkinnyMaxM && k % kSkinnyLdsBK == 0 && ptr16(p.A) && ptr16(p.B) &&
        (p.M - 1) * k * 2 + k * 2 < (int64_t(1) << 31)) {
      RotaryEpilogue r;
      r.cosT = cc.data, r.sinT = cs.data, r.cols = (int)rotaryCols, r.headDim = (int)headDim, r.tableRows = (int)tableRows;
      r.tableF32 = cc.dtype == diopi_dtype_float32, r.sinSign = conj ? -1.f : 1.f;
      AMD_TRY(p.dtype == diopi_dtype_bfloat16 ? launchSkinnyForShape<bf16_t>(ctx, stream, p, &r, &fused)
                                              : launchSkinnyForShape<half_t>(ctx, stream, p, &r, &fused));
    }
    if (!fused) AMD_TRY(runGemm(ctx, stream, p));
    if (!fused && rotaryCols > 0) {
      TensorView v;
      v.data = cout.data, v.ndim = 3, v.dtype = out.dtype, v.itemsize = out.itemsize;
      v.shape[0] = rows, v.shape[1] = rotaryCols / headDim, v.shape[2] = headDim;
      v.stride[0] = n, v.stride[1] = headDim, v.stride[2] = 1;
      v.numel = rows * rotaryCols;
      // the tables as [t, head_dim / 2] whatever shape the caller's dense tensors have, as the one-launch form reads them
      auto asTable = [&](TensorView t) {
        t.ndim = 2;
        t.shape[0] = tableRows, t.shape[1] = half;
        t.stride[0] = half, t.stride[1] = 1;
        return t;
      };
      AMD_TRY(runRotary(ctx, stream, v, v, asTable(cc), asTable(cs), conj, interleaved));
    }
  }
  if (outTemp) AMD_TRY(stridedCopy(stream, cout, out));
  return diopiSuccess;
}
