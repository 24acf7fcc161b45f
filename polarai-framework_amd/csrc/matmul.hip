// fmatmul_{f,t}_{f,t} for gfx950: C[M x N] = opA(A) * opB(B), fp32 in, fp32
// accumulate, C overwritten.
//
// The contraction runs on the matrix cores with v_mfma_f32_32x32x2_f32 (true
// fp32; gfx950 has no reduced-precision fp32 matrix path).  A work-group owns a
// BM x BN tile of C and walks K in steps of BK.  Both operand tiles are staged
// in LDS k-major (S[k][x], x = row of C for A, column of C for B) whatever the
// storage order in HBM, so the four transpose variants differ only in how a
// tile is fetched:
//   * operand contiguous along k (A not transposed, B transposed): a lane
//     loads 4 consecutive k of one row and scatters them to 4 LDS rows;
//   * operand contiguous along x (A transposed, B not transposed): a lane
//     loads 4 consecutive x of one k and stores them as one 16-byte LDS write.
// The next tile is fetched into registers while the current one is multiplied
// (two LDS stages, one barrier per step); tiles smaller than 256 x 256 fetch two
// steps ahead, because one of their k-steps (0.8-2.6 us) is shorter than a
// trip to memory.  Each wave owns a (BM/WM) x (BN/WN)
// sub-tile as TM x TN accumulator blocks of 32x32; per k-pair it reads TM + TN
// LDS words per lane and issues TM*TN MFMAs.  The LDS row pitch is chosen per
// operand so that neither the fill nor the fragment reads collide on banks.
//
// What bounds the 4096^3 case on MI355X (measured): the matrix pipes need 2^31
// busy cycles over 1024 SIMDs; under this kernel's LDS and L2 traffic the chip
// clocks at 2.0-2.2 GHz instead of 2.4, and a SIMD that interleaves MFMAs of
// four waves sustains only 80 % of the rate it reaches with one or two (124 vs
// 155 TFLOP/s in a register-only loop).  A hand-pipelined variant (three LDS
// stages, register prefetch two steps ahead, fragments read one k-pair ahead,
// occupancy capped at two waves per SIMD) landed on the same plateau and was
// dropped; larger tiles (less LDS and L2 traffic per flop) gained 5-7 %, hence
// the 256 x 256 x 32 configuration for big shapes.
//
// Work-groups are numbered so that the groups resident on one XCD (which share
// an L2) cover a compact block of C tiles and therefore re-use the same rows
// of A and columns of B.
//
// Shapes that are not multiples of the tile, leading dimensions that are not
// multiples of 4 and unaligned base pointers are handled by predicated /
// scalar fetch variants chosen on the host.
//
// Shapes whose C has too few tiles to occupy the chip (skinny outputs, long
// K) are split along K: every split writes its partial product to a workspace
// from the device pool and a second kernel adds the partials in split order,
// so the result does not depend on scheduling.  Tile shape and split count
// come from a small cost model (planMatmul) of rounds x k-steps x step time,
// with step times measured per tile shape on the full chip.
#include "internal.h"
#include "matmul_epilogue.h"

#include <cmath>
#include <type_traits>


using namespace polar_hip_detail;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

// LDS row pitch of a BX-wide operand stage.  A stage that is filled by 16-byte
// writes (operand contiguous along x) needs a pitch that is a multiple of 4
// words; BX + 4 also puts the two rows a wave reads per fragment four banks
// apart.  A stage that is filled by scattered single words (operand contiguous
// along k: a lane writes 4 consecutive k of one x, i.e. 4 rows) gets an odd
// pitch: within a half-wave the 8 rows and 4 columns written by one instruction
// then fall on 32 different banks (with BX + 4 they fell on 8).
template <int BX, bool KCONTIG> constexpr int ldsPitch() { return BX + (KCONTIG ? 1 : 4); }
constexpr int kXcds = 8;
#ifndef FUSED_SPLITS
#define FUSED_SPLITS 8
#endif
constexpr uint32_t kFusedSplits = FUSED_SPLITS;  // most parts of K that are added by the last group of a tile

struct MatmulArgs {
  const float* A;
  const float* B;
  float* C;        // final output, or the workspace when kSplits > 1
  uint32_t M, N, K;
  uint32_t tilesM, tilesN;
  uint32_t kSplits;   // work-groups [s*tiles, (s+1)*tiles) handle split s
  uint32_t kPerSplit; // multiple of BK
  // fused epilogue of the extended builtins (kEpi*); applied where the final
  // value of an element is produced: the kernel's store, or the split-K
  // reduction
  int epilogue;
  const float* bias;  // M x N, dense (the framework's fadd does not broadcast)
  float scaleAcc, scaleBias;
  // Split contraction whose last-arriving work-group adds the partial products
  // itself: one arrival counter per C tile (all zero when the kernel starts)
  // and the final output.  C then points at the workspace, where split s of
  // tile t keeps its BM x BN accumulators at [(t kSplits + s) BM BN], in the
  // order the lanes hold them.  Null: partial products go to C as whole
  // matrices, one per split, for a second kernel to add.
  uint32_t* tileCounters;
  float* finalC;
};

// Fetch of one operand tile (BX x BK) from HBM into registers, and its store
// into the k-major LDS stage.  KCONTIG: element (x, k) lives at
// X[(x0+x)*ld + k0+k]; otherwise at X[(k0+k)*ld + x0+x].
template <int BX, int BK, int NT, bool KCONTIG, bool VEC, bool EDGE>
struct TileFetch {
  static constexpr int kVecs = BX * BK / 4 / NT;  // 16-byte loads per lane
  static constexpr int kScalars = BX * BK / NT;   // dword loads per lane
  static_assert(BX * BK % (4 * NT) == 0, "tile must divide over the lanes");
  float r[kScalars];

  __device__ __forceinline__ void load(const float* X, size_t ld, uint32_t x0,
                                       uint32_t k0, uint32_t xdim,
                                       uint32_t kdim, int t) {
    if constexpr (VEC) {
#pragma unroll
      for (int v = 0; v < kVecs; ++v) {
        const int vid = t + v * NT;
        uint32_t x, k;
        if constexpr (KCONTIG) {
          x = vid / (BK / 4);
          k = (vid % (BK / 4)) * 4;
        } else {
          k = vid / (BX / 4);
          x = (vid % (BX / 4)) * 4;
        }
        const size_t off = KCONTIG ? size_t(x0 + x) * ld + (k0 + k)
                                   : size_t(k0 + k) * ld + (x0 + x);
        v4f g;
        if (!EDGE || (x0 + x < xdim && k0 + k < kdim)) {
          g = *reinterpret_cast<const v4f*>(X + off);
        } else {
          g = v4f{0.f, 0.f, 0.f, 0.f};
        }
        r[4 * v + 0] = g.x;
        r[4 * v + 1] = g.y;
        r[4 * v + 2] = g.z;
        r[4 * v + 3] = g.w;
      }
    } else {
#pragma unroll
      for (int s = 0; s < kScalars; ++s) {
        const int sid = t + s * NT;
        uint32_t x, k;
        if constexpr (KCONTIG) {
          x = sid / BK;
          k = sid % BK;
        } else {
          k = sid / BX;
          x = sid % BX;
        }
        const size_t off = KCONTIG ? size_t(x0 + x) * ld + (k0 + k)
                                   : size_t(k0 + k) * ld + (x0 + x);
        r[s] = (!EDGE || (x0 + x < xdim && k0 + k < kdim)) ? X[off] : 0.f;
      }
    }
  }

  __device__ __forceinline__ void store(float* S, int t) const {
    constexpr int LD = ldsPitch<BX, KCONTIG>();
    if constexpr (VEC) {
#pragma unroll
      for (int v = 0; v < kVecs; ++v) {
        const int vid = t + v * NT;
        if constexpr (KCONTIG) {
          const int x = vid / (BK / 4);
          const int k = (vid % (BK / 4)) * 4;
#pragma unroll
          for (int c = 0; c < 4; ++c) S[(k + c) * LD + x] = r[4 * v + c];
        } else {
          const int k = vid / (BX / 4);
          const int x = (vid % (BX / 4)) * 4;
          *reinterpret_cast<v4f*>(&S[k * LD + x]) =
              v4f{r[4 * v], r[4 * v + 1], r[4 * v + 2], r[4 * v + 3]};
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < kScalars; ++s) {
        const int sid = t + s * NT;
        const int x = KCONTIG ? sid / BK : sid % BX;
        const int k = KCONTIG ? sid % BK : sid / BX;
        S[k * LD + x] = r[s];
      }
    }
  }
};

// Linear work-group id -> C tile, such that the groups an XCD receives
// (ids congruent modulo 8) are consecutive in a panel-major walk over C.
__device__ __forceinline__ void tileOfGroup(uint32_t bid, uint32_t nGroups,
                                            uint32_t tilesM, uint32_t tilesN,
                                            uint32_t& tm, uint32_t& tn) {
  uint32_t lin = bid;
  if (nGroups % kXcds == 0) lin = (bid % kXcds) * (nGroups / kXcds) + bid / kXcds;
  constexpr uint32_t kPanel = 8; // tile rows walked together
  const uint32_t perPanel = kPanel * tilesN;
  const uint32_t panel = lin / perPanel;
  const uint32_t first = panel * kPanel;
  const uint32_t rows = tilesM - first < kPanel ? tilesM - first : kPanel;
  const uint32_t in = lin % perPanel;
  tm = first + in % rows;
  tn = in / rows;
}

// PF = how many k-steps ahead operand tiles are fetched into registers: 1 (the
// tile of step kt + 1 travels while step kt is multiplied) or 2 (two tiles in
// flight, for small tiles whose k-step is shorter than the memory latency).
template <int BM, int BN, int BK, int WM, int WN, int PF, bool TA, bool TB, bool VEC,
          bool EDGE>
__global__ __launch_bounds__(WM* WN * 64) void matmulKernel(MatmulArgs p) {
  static_assert(PF == 1 || PF == 2, "prefetch distance");
  constexpr int NT = WM * WN * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int LDA = ldsPitch<BM, !TA>(), LDB = ldsPitch<BN, TB>();
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile is made of 32x32");
  static_assert(BK % 4 == 0, "BK multiple of 4");

  __shared__ __attribute__((aligned(16))) float As[2][BK * LDA];
  __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

  const int t = threadIdx.x;
  const int lane = t % 64;
  const int wave = t / 64;
  const int wm = wave / WN, wn = wave % WN;

  const uint32_t tiles = p.tilesM * p.tilesN;
  const uint32_t split = blockIdx.x / tiles;
  uint32_t tm, tn;
  tileOfGroup(blockIdx.x % tiles, tiles, p.tilesM, p.tilesN, tm, tn);
  const uint32_t m0 = tm * BM, n0 = tn * BN;
  const uint32_t kBegin = split * p.kPerSplit;
  const uint32_t kEnd = kBegin + p.kPerSplit < p.K ? kBegin + p.kPerSplit : p.K;
  float* const out = p.C + size_t(split) * p.M * p.N;

  // A: k-contiguous when not transposed ([M x K]); B: k-contiguous when
  // transposed ([N x K]).
  TileFetch<BM, BK, NT, !TA, VEC, EDGE> fa[PF];
  TileFetch<BN, BK, NT, TB, VEC, EDGE> fb[PF];
  const size_t lda = TA ? p.M : p.K;
  const size_t ldb = TB ? p.K : p.N;

  v16f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const uint32_t nk = kEnd > kBegin ? (kEnd - kBegin + BK - 1) / BK : 0;
  if (nk != 0) { // uniform; the host never creates an empty split
    fa[0].load(p.A, lda, m0, kBegin, p.M, kEnd, t);
    fb[0].load(p.B, ldb, n0, kBegin, p.N, kEnd, t);
    fa[0].store(As[0], t);
    fb[0].store(Bs[0], t);
    if (PF == 2 && nk > 1) { // the tile of step 1 stays in registers until step 0 ends
      fa[0].load(p.A, lda, m0, kBegin + BK, p.M, kEnd, t);
      fb[0].load(p.B, ldb, n0, kBegin + BK, p.N, kEnd, t);
    }
  }
  __syncthreads();

  const int aBase = wm * WTM + (lane % 32);
  const int bBase = wn * WTN + (lane % 32);
  const int kLane = lane / 32;

  if constexpr (PF == 1) {
    for (uint32_t kt = 0; kt < nk; ++kt) {
      const int cur = kt & 1;
      const bool more = kt + 1 < nk;
      if (more) {
        fa[0].load(p.A, lda, m0, kBegin + (kt + 1) * BK, p.M, kEnd, t);
        fb[0].load(p.B, ldb, n0, kBegin + (kt + 1) * BK, p.N, kEnd, t);
      }
      const float* as = As[cur];
      const float* bs = Bs[cur];
#pragma unroll
      for (int kk = 0; kk < BK; kk += 2) {
        float a[TM], b[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) a[i] = as[(kk + kLane) * LDA + aBase + i * 32];
#pragma unroll
        for (int j = 0; j < TN; ++j) b[j] = bs[(kk + kLane) * LDB + bBase + j * 32];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j],
                                                            0, 0, 0);
      }
      if (more) {
        fa[0].store(As[cur ^ 1], t);
        fb[0].store(Bs[cur ^ 1], t);
      }
      __syncthreads();
    }
  } else {
    // One k-step: fetch the tile two steps ahead into register set `into`,
    // multiply the LDS stage of step kt, then move the tile of step kt + 1
    // (register set `from`) into the other stage.
    auto step = [&](uint32_t kt, auto fromTag, auto intoTag) {
      constexpr int from = decltype(fromTag)::value, into = decltype(intoTag)::value;
      const int cur = kt & 1;
      if (kt + 2 < nk) {
        fa[into].load(p.A, lda, m0, kBegin + (kt + 2) * BK, p.M, kEnd, t);
        fb[into].load(p.B, ldb, n0, kBegin + (kt + 2) * BK, p.N, kEnd, t);
      }
      const float* as = As[cur];
      const float* bs = Bs[cur];
#pragma unroll
      for (int kk = 0; kk < BK; kk += 2) {
        float a[TM], b[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) a[i] = as[(kk + kLane) * LDA + aBase + i * 32];
#pragma unroll
        for (int j = 0; j < TN; ++j) b[j] = bs[(kk + kLane) * LDB + bBase + j * 32];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j],
                                                            0, 0, 0);
      }
      if (kt + 1 < nk) {
        fa[from].store(As[cur ^ 1], t);
        fb[from].store(Bs[cur ^ 1], t);
      }
      __syncthreads();
    };
    // at the start of step kt register set kt % 2 holds the tile of step kt + 1
    using Set0 = std::integral_constant<int, 0>;
    using Set1 = std::integral_constant<int, PF - 1>;
    for (uint32_t kt = 0; kt < nk; kt += 2) {
      step(kt, Set0{}, Set1{});
      if (kt + 1 < nk) step(kt + 1, Set1{}, Set0{});
    }
  }

  float* finalOut = out;
  bool finalValues = p.kSplits == 1;  // what is stored is an element of the product (the epilogue applies)
  if (p.tileCounters != nullptr) {  // (uniform)
    // Partial products meet in the workspace, and the group that arrives last
    // at a tile adds them.  The XCDs' L2 caches are not coherent with each
    // other, and a device-scope fence per group (write back and invalidate the
    // whole L2) costs more than the product: 1024x1024x4096 in four parts 168
    // us with fences against 82 with a second kernel.  So the partial products
    // leave through write-through stores (16 bytes per lane, the lanes of a
    // store side by side: whole lines, which matters for stores that go to
    // memory as they are) and are ordered by hand: every thread
    // waits until its stores are acknowledged, the group meets at a barrier,
    // and only then one thread counts the group in.  The group that sees
    // kSplits - 1 earlier arrivals is the last; what the others stored was in
    // memory before they counted themselves in.  Its loads of their partial
    // products are ordinary ones: a launch starts with every L2 invalidated, and
    // until now nothing in this launch has read those lines, so they cannot be
    // stale in this XCD's L2.  It adds the partial products in split order --
    // its own from registers, in its place -- so the sum does not depend on
    // which group came last, and leaves the counter at zero for the next
    // launch.
    __shared__ uint32_t arrivedBefore;
    const uint32_t tile = blockIdx.x % tiles;
    constexpr uint32_t kTileFloats = uint32_t(BM) * BN;
    float* const partials = p.C + size_t(tile) * p.kSplits * kTileFloats;
    float* const mine = partials + size_t(split) * kTileFloats;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; r += 4)
          streamStore(v4f{acc[i][j][r], acc[i][j][r + 1], acc[i][j][r + 2], acc[i][j][r + 3]},
                      reinterpret_cast<v4f*>(mine + (((i * TN + j) * 4 + r / 4) * NT + t) * 4));
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (t == 0)
      arrivedBefore = __hip_atomic_fetch_add(&p.tileCounters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (arrivedBefore != p.kSplits - 1) return;
    if (t == 0) __hip_atomic_store(&p.tileCounters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        // quarter q of the block's sixteen values: [((block 4 + q) lanes + lane) 4]
        auto partOf = [&](uint32_t s) {
          const float* const from = partials + size_t(s) * kTileFloats + (((i * TN + j) * 4) * NT + t) * 4;
          v16f v;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const v4f piece = *reinterpret_cast<const v4f*>(from + q * NT * 4);
#pragma unroll
            for (int c = 0; c < 4; ++c) v[4 * q + c] = piece[c];
          }
          return v;
        };
        v16f total = split == 0 ? acc[i][j] : partOf(0);
        for (uint32_t s = 1; s < p.kSplits; ++s) total += s == split ? acc[i][j] : partOf(s);
        acc[i][j] = total;
      }
    finalOut = p.finalC;
    finalValues = true;
  }

  // Accumulator block layout of the 32x32 MFMA: register r of lane l holds
  // row 8*(r/4) + 4*(l/32) + r%4, column l%32.
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint32_t col = n0 + wn * WTN + j * 32 + (lane % 32);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const uint32_t row =
            m0 + wm * WTM + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
        if (!EDGE || (row < p.M && col < p.N)) {
          const size_t idx = size_t(row) * p.N + col;
          finalOut[idx] = finalValues ? applyEpilogue(p.epilogue, acc[i][j][r], p.bias,
                                                      p.scaleAcc, p.scaleBias, idx)
                                      : acc[i][j][r];
        }
      }
    }
  }
}

// C[i] = sum over splits of partial[s][i], in a fixed order: a work-group owns
// 64 consecutive elements (one per lane); wave w adds the splits s = w, w+W,
// w+2W, ... one after the other (loads four ahead), and the W wave sums are
// then added in wave order.  Which lane adds what depends only on the indices,
// so the result is the same on every run.  Many splits of a small C (33 x 127
// in 256 splits) would otherwise be one long chain of dependent loads per
// element (61 us for that shape; 6 us like this).
// kReduceWaves = W is chosen from the number of splits (2, 4, 8 or 16).
template <int kReduceWaves>
__global__ __launch_bounds__(64 * kReduceWaves) void splitKReduceKernel(
    const float* __restrict__ partial, float* __restrict__ c, uint64_t count, uint32_t splits,
    int epilogue, const float* bias, float scaleAcc, float scaleBias) {
  __shared__ float sums[kReduceWaves][64];
  const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const uint64_t i = uint64_t(blockIdx.x) * 64 + lane;
  float acc = 0.0f;
  if (i < count) {
    uint32_t s = wave;
    for (; s + 3 * kReduceWaves < splits; s += 4 * kReduceWaves) {
      const float v0 = partial[uint64_t(s) * count + i];
      const float v1 = partial[uint64_t(s + kReduceWaves) * count + i];
      const float v2 = partial[uint64_t(s + 2 * kReduceWaves) * count + i];
      const float v3 = partial[uint64_t(s + 3 * kReduceWaves) * count + i];
      acc = (((acc + v0) + v1) + v2) + v3;
    }
    for (; s < splits; s += kReduceWaves) acc += partial[uint64_t(s) * count + i];
  }
  sums[wave][lane] = acc;
  __syncthreads();
  if (wave == 0 && i < count) {
    float total = sums[0][lane];
#pragma unroll
    for (int w = 1; w < kReduceWaves; ++w) total += sums[w][lane];
    c[i] = applyEpilogue(epilogue, total, bias, scaleAcc, scaleBias, i);
  }
}

hipError_t launchReduce(polar_hip_device* dev, const float* partial, float* c, uint64_t count,
                        uint32_t splits, const MatmulArgs& p) {
  const dim3 grid(static_cast<unsigned>((count + 63) / 64));
  if (splits <= 2)
    return launchKernel(dev, splitKReduceKernel<2>, grid, dim3(128), partial, c, count, splits,
                        p.epilogue, p.bias, p.scaleAcc, p.scaleBias);
  if (splits <= 4)
    return launchKernel(dev, splitKReduceKernel<4>, grid, dim3(256), partial, c, count, splits,
                        p.epilogue, p.bias, p.scaleAcc, p.scaleBias);
  if (splits <= 8)
    return launchKernel(dev, splitKReduceKernel<8>, grid, dim3(512), partial, c, count, splits,
                        p.epilogue, p.bias, p.scaleAcc, p.scaleBias);
  return launchKernel(dev, splitKReduceKernel<16>, grid, dim3(1024), partial, c, count, splits,
                      p.epilogue, p.bias, p.scaleAcc, p.scaleBias);
}

template <int BM, int BN, int BK, int WM, int WN, int PF, bool TA, bool TB>
int launchLayout(polar_hip_device* dev, const MatmulArgs& p, bool vec, bool edge) {
  const uint64_t groups = uint64_t(p.tilesM) * p.tilesN * p.kSplits;
  const dim3 grid(static_cast<unsigned>(groups)), block(WM * WN * 64);
  if (vec && !edge)
    POLAR_HIP_TRY(launchKernel(
        dev, matmulKernel<BM, BN, BK, WM, WN, PF, TA, TB, true, false>, grid, block, p));
  else if (vec && edge)
    POLAR_HIP_TRY(launchKernel(
        dev, matmulKernel<BM, BN, BK, WM, WN, PF, TA, TB, true, true>, grid, block, p));
  else
    POLAR_HIP_TRY(launchKernel(
        dev, matmulKernel<BM, BN, BK, WM, WN, 1, TA, TB, false, true>, grid, block, p));
  return POLAR_HIP_OK;
}

template <int BM, int BN, int BK, int WM, int WN, int PF = 1>
int launchTile(polar_hip_device* dev, bool ta, bool tb, const MatmulArgs& p0,
               uint32_t splits, bool lastGroupAdds) {
  MatmulArgs p = p0;
  p.tilesM = (p.M + BM - 1) / BM;
  p.tilesN = (p.N + BN - 1) / BN;
  const uint32_t kSteps = (p.K + BK - 1) / BK;
  // Equal shares of whole k-steps; the number of splits is then what those
  // shares need, so that no split starts at or beyond K (an empty split would
  // prefetch its first tile from outside the operands).
  const uint32_t stepsPerSplit = (kSteps + splits - 1) / splits;
  splits = (kSteps + stepsPerSplit - 1) / stepsPerSplit;
  p.kSplits = splits;
  p.kPerSplit = stepsPerSplit * BK;
  // 16-byte fetches need aligned bases and a contiguous dimension that is a
  // multiple of 4 for both operands.
  const uint32_t contigA = ta ? p.M : p.K;
  const uint32_t contigB = tb ? p.K : p.N;
  const bool vec = aligned16(p.A) && aligned16(p.B) && contigA % 4 == 0 &&
                   contigB % 4 == 0;
  const bool edge = p.M % BM != 0 || p.N % BN != 0 || p.K % BK != 0;

  float* const c = p.C;
  const uint64_t count = uint64_t(p.M) * p.N;
  // partial products go to the device's workspace; the lock keeps another
  // thread's call from enqueuing its own user of the workspace between this
  // call's two kernels
  std::unique_lock<std::mutex> workspaceLock(dev->workspaceMu, std::defer_lock);
  void* workspace = nullptr;
  // Up to kFusedSplits parts of K: the group that arrives last at a tile adds
  // the tile's partial products itself (they sit in the workspace tile by tile)
  // and no second kernel runs.  With more parts one group would add for too
  // long while the rest of the chip idles; those keep the reduction kernel.
  const uint64_t tiles = uint64_t(p.tilesM) * p.tilesN;
  const uint64_t fusedBytes = tiles * splits * BM * BN * sizeof(float);
  const bool fused = lastGroupAdds && splits > 1 && splits <= kFusedSplits && tiles <= kTileCounters && fusedBytes <= kWorkspaceBytes;
  p.tileCounters = nullptr;
  p.finalC = c;
  if (splits > 1) {
    workspaceLock.lock();
    int st = workspaceFor(dev, fused ? fusedBytes : count * splits * sizeof(float), &workspace);
    if (st != POLAR_HIP_OK) return st;
    p.C = static_cast<float*>(workspace);
    if (fused) p.tileCounters = dev->tileCounters;
  }
  int st;
  if (!ta && !tb) st = launchLayout<BM, BN, BK, WM, WN, PF, false, false>(dev, p, vec, edge);
  else if (!ta && tb) st = launchLayout<BM, BN, BK, WM, WN, PF, false, true>(dev, p, vec, edge);
  else if (ta && !tb) st = launchLayout<BM, BN, BK, WM, WN, PF, true, false>(dev, p, vec, edge);
  else st = launchLayout<BM, BN, BK, WM, WN, PF, true, true>(dev, p, vec, edge);
  if (splits > 1 && !fused && st == POLAR_HIP_OK) {
    hipError_t e = launchReduce(dev, static_cast<const float*>(workspace), c, count, splits, p);
    if (e != hipSuccess) st = failHip(e, "splitKReduceKernel");
  }
  return st;
}

// ---- tile shape and split count -----------------------------------------------
struct TileConfig {
  int bm, bn, bk;
  int residentGroups; // groups of this shape one CU holds (LDS, lanes)
  // Microseconds per k-step, measured with every CU busy (cold clock, as a lone
  // launch in a graph finds it; a settled clock runs them 7-10 % faster, the
  // 128x128 tile with one group per CU 22 %, for which its entry sits between
  // the two): stepAlone with one group on the CU, and what
  // every co-resident group adds once the groups no longer hide in each other's
  // latency; a step with r groups resident takes max(stepAlone, r * stepPerGroup).
  float stepAlone, stepPerGroup;
};
// order = the switch in matmulWithEpilogue
constexpr TileConfig kConfigs[] = {
    {256, 256, 32, 1, 8.2f, 8.2f},   // 4x4 waves of 64x64: one group per CU; 7.8 warm, 8.4-9.0 cold
    {128, 128, 32, 2, 2.4f, 2.28f},  // 2x4 waves of 64x32, tiles fetched two steps ahead (alone: 2.6 cold, 2.04 settled)
    {64, 64, 32, 4, 0.79f, 0.62f},   // 2x2 waves of 32x32, two steps ahead (per group: 0.74 cold, 0.58 settled)
    {128, 32, 32, 3, 0.85f, 0.77f},  // skinny N
    {32, 128, 32, 3, 0.85f, 0.77f},  // skinny M
    {32, 32, 32, 8, 1.0f, 0.22f},    // one wave (0.78 in a long loop; short loops measured 10 % behind the others)
    {256, 128, 32, 1, 4.65f, 4.65f}, // 4x2 waves of 64x64, two steps ahead
    {128, 256, 32, 1, 4.6f, 4.6f},   // 2x4 waves of 64x64, two steps ahead
    {128, 64, 32, 3, 1.32f, 1.38f},  // 4x2 waves of 32x32, two steps ahead
    {64, 128, 32, 3, 1.32f, 1.38f},  // 2x4 waves of 32x32, two steps ahead
};

struct MatmulPlan {
  int config;
  uint32_t splits;
  bool fused;  // splits > 1: the last group of a tile adds the partial products (no second kernel)
};

// What adding the partial products of a split contraction costs, in
// microseconds, either way.  Second kernel: a launch, and every partial
// product written and read once more.  Last group of a tile: its chain of
// store acknowledgement, counter and loads (about as long as a launch), the
// write-through stores of all partial products, and one group reading the
// other s - 1 partial products of a tile at about 40 GB/s.  (Measured against
// each other on a settled clock: 3072^3 in four parts 494 -> 454 us, 1024 x
// 2048 x 4096 160 -> 140, 768^3 19.4 -> 15.7; but 512^3 9.1 -> 10.6 and 300 x
// 300 x 3000 16.2 -> 20.1, which therefore keep the second kernel.)
constexpr uint32_t kFusedTileLimit = kTileCounters;
inline double reduceKernelUs(double m, double n, uint32_t s) { return 4.0 + m * n * 4.0 * (s + 1) / 3.0e6; }
inline double lastGroupAddsUs(double m, double n, uint32_t s, int bm, int bn) {
  return 4.0 + m * n * 4.0 * s / 4.0e6 + (s - 1) * double(bm) * bn * 4.0 / 40.0e3;
}
inline bool lastGroupMayAdd(uint32_t s, double tiles) { return s > 1 && s <= kFusedSplits && tiles <= kFusedTileLimit; }

// Estimated microseconds of every tile shape and split count; the cheapest
// wins.  The groups run in rounds of (CUs x resident groups); a k-step of a
// round costs what the table says for the number of groups a CU holds in it,
// and a partly filled last round takes as long per step as its fullest CU
// (4097^3 on 256x256 tiles is 289 groups = 2 rounds, not 1.13).  On top: launch,
// filling the pipeline and storing C (a few steps' worth), and for split
// contractions the second kernel that adds the partial products.
MatmulPlan planMatmul(uint32_t m, uint32_t n, uint32_t k, int computeUnits) {
  static const uint32_t kSplitChoices[] = {1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256};
  // the cheapest plan of every tile shape first ...
  constexpr int kCount = int(sizeof(kConfigs) / sizeof(kConfigs[0]));
  double usOf[kCount], tilesOf[kCount];
  uint32_t splitsOf[kCount];
  bool fusedOf[kCount];
  for (int c = 0; c < kCount; ++c) {
    usOf[c] = 1e30;
    splitsOf[c] = 1;
    fusedOf[c] = false;
    const TileConfig& t = kConfigs[c];
    const double tiles = double((m + t.bm - 1) / t.bm) * ((n + t.bn - 1) / t.bn);
    const uint32_t kSteps = (k + t.bk - 1) / t.bk;
    auto stepUs = [&](double resident) {
      const double busy = resident * t.stepPerGroup;
      return busy > t.stepAlone ? busy : double(t.stepAlone);
    };
    for (uint32_t s : kSplitChoices) {
      if (s > 1 && (kSteps / s < 1 || double(m) * n * s * 4 > double(kWorkspaceBytes))) break;
      const double groups = tiles * s;
      const double perRound = double(computeUnits) * t.residentGroups;
      const double fullRounds = std::floor(groups / perRound + 1e-9);
      const double rest = groups - fullRounds * perRound;
      double perStep = fullRounds * stepUs(t.residentGroups);
      if (rest > 0.5) perStep += stepUs(std::ceil(rest / computeUnits - 1e-9));
      double us = ((kSteps + s - 1) / s) * perStep + 4.0 + 2.5 * t.stepAlone;
      bool fused = false;
      if (s > 1) {
        const double second = reduceKernelUs(m, n, s), last = lastGroupAddsUs(m, n, s, t.bm, t.bn);
        fused = lastGroupMayAdd(s, tiles) && last < second;
        us += fused ? last : second;
      }
      if (us < usOf[c]) {
        usOf[c] = us;
        splitsOf[c] = s;
        fusedOf[c] = fused;
      }
    }
    tilesOf[c] = tiles;
  }
  // ... then, among the shapes that split K the same way as the cheapest one
  // and whose estimate is within 4 % of it (closer than the model can tell
  // apart), the one with the fewest tiles: every tile reads its rows of A and
  // columns of B again, which the model does not price (33 x 127 x 65536: one
  // 64 x 128 tile 23.0 us, two 64 x 64 tiles 25.5).  Across different split
  // counts the rule misleads (2048^3: 168 -> 186 us) and is not applied.
  int cheapest = 0;
  for (int c = 1; c < kCount; ++c)
    if (usOf[c] < usOf[cheapest]) cheapest = c;
  int best = cheapest;
  for (int c = 0; c < kCount; ++c)
    if (splitsOf[c] == splitsOf[cheapest] && usOf[c] <= usOf[cheapest] * 1.04 && tilesOf[c] < tilesOf[best]) best = c;
  return MatmulPlan{best, splitsOf[best], fusedOf[best]};
}

} // namespace

namespace {
constexpr int kConfigCount = int(sizeof(kConfigs) / sizeof(kConfigs[0]));
static_assert(kConfigCount == POLAR_HIP_MATMUL_TILE_CONFIGS, "the header states how many there are");

// forced: a tile configuration and split count given by the caller instead of
// the planner's (config < 0: the planner, and the short-contraction kernels
// where they apply)
int matmulWithEpilogue(polar_hip_device* dev, int transA, int transB, const float* a,
                       const float* b, float* c, uint64_t m, uint64_t n, uint64_t k,
                       int epilogue, const float* bias, float scaleAcc, float scaleBias,
                       MatmulPlan forced = MatmulPlan{-1, 1, false}) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  if (m == 0 || n == 0) return POLAR_HIP_OK;
  POLAR_HIP_REQUIRE(c != nullptr, "null output");
  POLAR_HIP_REQUIRE(k == 0 || (a != nullptr && b != nullptr), "null operand");
  POLAR_HIP_REQUIRE(m < (1ull << 31) && n < (1ull << 31) && k < (1ull << 31),
                    "dimension does not fit 31 bits");
  POLAR_HIP_REQUIRE(c != a && c != b, "output aliases an operand");
  POLAR_HIP_REQUIRE(epilogue != kEpiAddSigmoid || bias != nullptr, "null bias");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  MatmulArgs p{a, b, c, static_cast<uint32_t>(m), static_cast<uint32_t>(n),
               static_cast<uint32_t>(k), 0, 0, 1, 0, epilogue, bias, scaleAcc, scaleBias, nullptr, c};
  if (k == 0) {
    // Empty contraction: the reference's loop leaves acc = 0 and stores it.
    if (epilogue == kEpiNone) return polar_hip_ffill(dev, 0.0f, c, m * n);
    const uint64_t grid = (m * n + 63) / 64;
    POLAR_HIP_REQUIRE(grid < (1ull << 31), "matrix too large for one launch");
    POLAR_HIP_TRY(launchReduce(dev, nullptr, c, m * n, 0u, p));
    return POLAR_HIP_OK;
  }
  const bool ta = transA != 0, tb = transB != 0;
  // short contraction, one long and one short output dimension: streamed in one
  // shot per block (matmul_small_k.hip)
  const MatmulCall call{a, b, c, p.M, p.N, p.K, ta, tb, epilogue, bias, scaleAcc, scaleBias};
  if (forced.config < 0 && rowsMatmulApplies(call, dev->info.compute_units)) return launchRowsMatmul(dev, call);
  if (forced.config < 0 && panelMatmulApplies(call, dev->info.compute_units)) return launchPanelMatmul(dev, call);
  if (forced.config < 0 && smallKMatmulApplies(call)) return launchSmallKMatmul(dev, call);
  if (forced.config < 0 && longKMatmulApplies(call)) return launchLongKMatmul(dev, call);
  if (forced.config < 0 && skinnyMatmulApplies(call)) return launchSkinnyMatmul(dev, call);
  const MatmulPlan plan =
      forced.config < 0 ? planMatmul(p.M, p.N, p.K, dev->info.compute_units) : forced;
  switch (plan.config) {
  case 0: return launchTile<256, 256, 32, 4, 4, 1>(dev, ta, tb, p, plan.splits, plan.fused);
  case 1: return launchTile<128, 128, 32, 2, 4, 2>(dev, ta, tb, p, plan.splits, plan.fused);
  case 2: return launchTile<64, 64, 32, 2, 2, 2>(dev, ta, tb, p, plan.splits, plan.fused);
  case 3: return launchTile<128, 32, 32, 4, 1, 2>(dev, ta, tb, p, plan.splits, plan.fused);
  case 4: return launchTile<32, 128, 32, 1, 4, 2>(dev, ta, tb, p, plan.splits, plan.fused);
  case 5: return launchTile<32, 32, 32, 1, 1, 1>(dev, ta, tb, p, plan.splits, plan.fused);
  case 6: return launchTile<256, 128, 32, 4, 2, 2>(dev, ta, tb, p, plan.splits, plan.fused);
  case 7: return launchTile<128, 256, 32, 2, 4, 2>(dev, ta, tb, p, plan.splits, plan.fused);
  case 8: return launchTile<128, 64, 32, 4, 2, 2>(dev, ta, tb, p, plan.splits, plan.fused);
  default: return launchTile<64, 128, 32, 2, 4, 2>(dev, ta, tb, p, plan.splits, plan.fused);
  }
}
} // namespace

extern "C" int polar_hip_fmatmul(polar_hip_device* dev, int transA, int transB,
                                 const float* a, const float* b, float* c,
                                 uint64_t m, uint64_t n, uint64_t k) {
  return matmulWithEpilogue(dev, transA, transB, a, b, c, m, n, k, kEpiNone, nullptr, 1.0f, 1.0f);
}

extern "C" int polar_hip_fmatmul_plan(polar_hip_device* dev, uint64_t m, uint64_t n, uint64_t k,
                                      int* tile_config, uint32_t* splits, uint32_t tile[3]) {
  POLAR_HIP_REQUIRE(dev != nullptr && tile_config != nullptr && splits != nullptr, "null argument");
  POLAR_HIP_REQUIRE(m != 0 && n != 0 && k != 0, "empty product");
  POLAR_HIP_REQUIRE(m < (1ull << 31) && n < (1ull << 31) && k < (1ull << 31),
                    "dimension does not fit 31 bits");
  // the short-contraction kernels take any layout of such a shape
  const MatmulCall call{nullptr, nullptr, nullptr, static_cast<uint32_t>(m), static_cast<uint32_t>(n),
                        static_cast<uint32_t>(k), false, false, kEpiNone, nullptr, 1.0f, 1.0f};
  if (smallKMatmulApplies(call) || longKMatmulApplies(call) || skinnyMatmulApplies(call)) {
    *tile_config = -1;
    *splits = 1;
    if (tile != nullptr) tile[0] = tile[1] = tile[2] = 0;
    return POLAR_HIP_OK;
  }
  const MatmulPlan plan = planMatmul(call.M, call.N, call.K, dev->info.compute_units);
  *tile_config = plan.config;
  *splits = plan.splits;
  if (tile != nullptr) {
    tile[0] = kConfigs[plan.config].bm;
    tile[1] = kConfigs[plan.config].bn;
    tile[2] = kConfigs[plan.config].bk;
  }
  return POLAR_HIP_OK;
}

extern "C" int polar_hip_fmatmul_with_plan(polar_hip_device* dev, int transA, int transB,
                                           const float* a, const float* b, float* c, uint64_t m,
                                           uint64_t n, uint64_t k, int tile_config,
                                           uint32_t splits) {
  POLAR_HIP_REQUIRE(tile_config >= 0 && tile_config < kConfigCount, "no such tile configuration");
  POLAR_HIP_REQUIRE(splits >= 1 && splits <= 256, "split count out of range");
  POLAR_HIP_REQUIRE(splits == 1 || m * n * splits * sizeof(float) <= kWorkspaceBytes,
                    "partial products exceed the workspace");
  return matmulWithEpilogue(dev, transA, transB, a, b, c, m, n, k, kEpiNone, nullptr, 1.0f, 1.0f,
                            MatmulPlan{tile_config, splits, splits > 1 && splits <= kFusedSplits});
}

extern "C" int polar_hip_fmatmul_fsigmoid(polar_hip_device* dev, int transA, int transB,
                                          const float* a, const float* b, float* out,
                                          uint64_t m, uint64_t n, uint64_t k) {
  return matmulWithEpilogue(dev, transA, transB, a, b, out, m, n, k, kEpiSigmoid, nullptr, 1.0f,
                            1.0f);
}

extern "C" int polar_hip_fmatmul_fadd_fsigmoid(polar_hip_device* dev, int transA, int transB,
                                               const float* a, const float* b, float scaleProduct,
                                               const float* bias, float scaleBias, float* out,
                                               uint64_t m, uint64_t n, uint64_t k) {
  POLAR_HIP_REQUIRE(bias != out, "output aliases the bias");
  return matmulWithEpilogue(dev, transA, transB, a, b, out, m, n, k, kEpiAddSigmoid, bias,
                            scaleProduct, scaleBias);
}
