// Memory-pattern probes for gfx950: small kernels that move the same bytes in
// the same pattern as a builtin but do none of its work, so that a builtin's
// HBM rate can be judged against what its access pattern allows on the very
// GPU and in the very run it is measured in.  They are a measurement aid built
// into a library of their own (libpolar_hip_probes.so); the device library
// does not contain or call them, and their results are meaningless as data.
//
// Every probe allocates its own buffers (`sets` of them, used in rotation so
// that no launch finds its operands in a cache the previous one filled), runs
// `warm` untimed and `reps` timed launches back to back on one stream, each
// timed launch carrying its own pair of events, and writes the kernel
// durations in microseconds to us[0..reps).  Return value: 0, or the hipError_t
// of the first failing call.
#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <vector>

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

#define PROBE_TRY(expr)                 \
  do {                                  \
    hipError_t e_ = (expr);             \
    if (e_ != hipSuccess) return e_;    \
  } while (0)

struct Buffers {
  std::vector<void*> blocks;
  ~Buffers() {
    for (void* b : blocks) (void)hipFree(b);
  }
  hipError_t add(size_t bytes, void** out) {
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) return e;
    blocks.push_back(p);
    e = hipMemset(p, 0, bytes);
    *out = p;
    return e;
  }
};

struct Events {
  std::vector<hipEvent_t> all;
  ~Events() {
    for (hipEvent_t e : all) (void)hipEventDestroy(e);
  }
  hipError_t make(int count) {
    for (int i = 0; i < count; ++i) {
      hipEvent_t e;
      hipError_t s = hipEventCreate(&e);
      if (s != hipSuccess) return s;
      all.push_back(e);
    }
    return hipSuccess;
  }
};

// launch(i, start, stop): enqueue launch number i on `stream`; start/stop are
// null for the untimed ones.
template <typename Launch>
hipError_t timeLaunches(hipStream_t stream, int warm, int reps, float* us, Launch launch) {
  Events ev;
  PROBE_TRY(ev.make(2 * reps));
  for (int i = 0; i < warm; ++i) launch(i, nullptr, nullptr);
  PROBE_TRY(hipStreamSynchronize(stream));
  for (int i = 0; i < reps; ++i) launch(warm + i, ev.all[2 * i], ev.all[2 * i + 1]);
  PROBE_TRY(hipStreamSynchronize(stream));
  PROBE_TRY(hipGetLastError());
  for (int i = 0; i < reps; ++i) {
    float ms = 0.0f;
    PROBE_TRY(hipEventElapsedTime(&ms, ev.all[2 * i], ev.all[2 * i + 1]));
    us[i] = ms * 1e3f;
  }
  return hipSuccess;
}

struct Stream {
  hipStream_t s = nullptr;
  ~Stream() {
    if (s) (void)hipStreamDestroy(s);
  }
  hipError_t make() { return hipStreamCreateWithFlags(&s, hipStreamNonBlocking); }
};

// ---- streams: READS input streams combined into one output stream ----------
// out[i] = max over the streams of in_s[i], 16 bytes per lane and stream, one
// pass; loads non-temporal, stores non-temporal and written through (the hints
// the builtins use).  READS = 1 is a plain copy; READS = 0 writes only (a fill).
struct StreamPointers {
  const v4f* in[4];
  v4f* out;
};
template <int READS, int BLOCK>
__global__ __launch_bounds__(BLOCK) void streamsKernel(StreamPointers p, uint64_t n4, int xcdRanges,
                                                       int plainStores) {
  // xcdRanges: the groups of one XCD (ids equal modulo 8) take a contiguous
  // eighth of the streams instead of every eighth piece
  uint32_t group = blockIdx.x;
  if (xcdRanges) {
    const uint32_t per = (gridDim.x + 7) / 8;
    group = (blockIdx.x % 8) * per + blockIdx.x / 8;
  }
  const uint64_t i = uint64_t(group) * BLOCK + threadIdx.x;
  if (i >= n4) return;
  v4f acc = {1.0f, 2.0f, 3.0f, 4.0f};
  v4f v[READS > 0 ? READS : 1];
#pragma unroll
  for (int s = 0; s < READS; ++s) v[s] = __builtin_nontemporal_load(&p.in[s][i]);
#pragma unroll
  for (int s = 0; s < READS; ++s)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = v[s][c] > acc[c] ? v[s][c] : acc[c];
  // the output may start off a 16-byte boundary (see polar_probe_streams)
  typedef float v4fu __attribute__((ext_vector_type(4), aligned(4)));
  if (plainStores)
    *reinterpret_cast<v4fu*>(&p.out[i]) = acc;
  else
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" : : "v"(&p.out[i]), "v"(acc) : "memory");
}

template <int READS, int BLOCK>
void launchStreams(hipStream_t s, hipEvent_t e0, hipEvent_t e1, const StreamPointers& p, uint64_t n4,
                   int xcdRanges, int plainStores) {
  unsigned grid = static_cast<unsigned>((n4 + BLOCK - 1) / BLOCK);
  if (xcdRanges) grid = (grid + 7) / 8 * 8;
  hipExtLaunchKernelGGL((streamsKernel<READS, BLOCK>), dim3(grid), dim3(BLOCK), 0, s, e0, e1, 0, p, n4,
                        xcdRanges, plainStores);
}

// ---- read only: every lane sums UNROLL 16-byte loads, one float per group ---
template <int UNROLL>
__global__ __launch_bounds__(256) void readKernel(const v4f* in, float* out, uint64_t n4) {
  const uint64_t base = uint64_t(blockIdx.x) * (256 * UNROLL) + threadIdx.x;
  v4f v[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const uint64_t i = base + uint64_t(u) * 256;
    v[u] = i < n4 ? __builtin_nontemporal_load(&in[i]) : v4f{0.0f, 0.0f, 0.0f, 0.0f};
  }
  float acc = 0.0f;
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) acc += (v[u][0] + v[u][1]) + (v[u][2] + v[u][3]);
  // one store per wave: the sum of the wave's lanes is not needed for a traffic
  // probe, but the loads must not be optimised away
  if (acc == 12345.678f || threadIdx.x % 64 == 0) out[blockIdx.x * 4 + threadIdx.x / 64] = acc;
}

// ---- transpose pattern: rows x cols fp32, TI input rows x TJ columns per group
// read as row segments, written as TJ chunks of TI elements that are aligned
// down to 128 bytes in the output -- the reads and writes of a tiled transpose
// whose stores cover whole lines, without the exchange through LDS and without
// any barrier.
template <int TI, int TJ, int THREADS>
__global__ __launch_bounds__(THREADS) void transposePatternKernel(const float* in, float* out,
                                                                  uint32_t R, uint32_t C,
                                                                  uint32_t rowTiles,
                                                                  uint32_t colTiles, int order) {
  constexpr int P = TI * TJ / THREADS;
  const uint32_t bid = blockIdx.x;
  uint32_t bi, bj;
  if (order == 0) { // row tiles fastest
    bi = bid % rowTiles;
    bj = bid / rowTiles;
  } else if (order == 1) { // column tiles fastest
    bj = bid % colTiles;
    bi = bid / colTiles;
  } else { // each XCD (ids equal modulo 8) a contiguous range of column tiles
    const uint32_t per = (colTiles + 7) / 8, x = bid % 8, local = bid / 8;
    bj = x * per + local % per;
    bi = local / per;
  }
  if (bj >= colTiles || bi >= rowTiles) return;
  const uint32_t i0 = bi * TI, j0 = bj * TJ;
  const uint64_t total = uint64_t(R) * C;
  const int t = threadIdx.x;
  float v[P];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int e = t + p * THREADS;
    const uint32_t row = e / TJ, col = e % TJ;
    const uint64_t r = uint64_t(i0) + row;
    v[p] = (r < R && j0 + col < C) ? in[r * C + j0 + col] : 0.0f;
  }
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int e = t + p * THREADS;
    const uint32_t c = e / TI, l = e % TI;
    const uint64_t j = uint64_t(j0) + c;
    const uint64_t a = ((j * R + i0) & ~31ull) + l;
    if (j < C && a < total) __builtin_nontemporal_store(v[p], &out[a]);
  }
}

template <int TI, int TJ, int THREADS>
void launchPattern(hipStream_t s, hipEvent_t e0, hipEvent_t e1, const float* in, float* out,
                   uint32_t R, uint32_t C, int order) {
  const uint32_t rowTiles = (R + TI - 1) / TI, colTiles = (C + TJ - 1) / TJ;
  const uint32_t grid = order == 2 ? 8 * ((colTiles + 7) / 8) * rowTiles : rowTiles * colTiles;
  hipExtLaunchKernelGGL((transposePatternKernel<TI, TJ, THREADS>), dim3(grid), dim3(THREADS), 0, s,
                        e0, e1, 0, in, out, R, C, rowTiles, colTiles, order);
}

} // namespace

// ---- panels: the memory pattern of a short-contraction matmul with one long
// dimension, without the arithmetic ------------------------------------------
// tall: `longDim` rows of `inShort` floats in (one contiguous array), `longDim`
// rows of `outShort` floats out; a wave takes 32 rows: their input as the
// contiguous piece it is, 16 bytes per lane and load, all loads first; their
// output likewise.
__global__ __launch_bounds__(512) void tallPanelsKernel(const float* in, float* out, uint32_t longDim,
                                                        uint32_t inShort, uint32_t outShort) {
  const uint32_t lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const uint32_t x0 = blockIdx.x * 256 + wave * 32;
  if (x0 >= longDim) return;
  const uint32_t rows = longDim - x0 < 32 ? longDim - x0 : 32;
  const uint32_t inFloats = rows * inShort, outFloats = rows * outShort;
  const float* const piece = in + size_t(x0) * inShort;
  v4f v[16];
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    const uint32_t at = (u * 64 + lane) * 4;
    v[u] = *reinterpret_cast<const v4f*>(piece + (at + 4 <= inFloats ? at : 0));
  }
  v4f acc = v[0];
#pragma unroll
  for (int u = 1; u < 16; ++u)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = v[u][c] > acc[c] ? v[u][c] : acc[c];
  float* const to = out + size_t(x0) * outShort;
  for (uint32_t at = lane * 4; at + 4 <= outFloats; at += 256) *reinterpret_cast<v4f*>(to + at) = acc;
}
// wide: `inShort` rows of `longDim` floats in, `outShort` rows of `longDim`
// floats out; a wave takes 64 columns, a quarter of it one row per instruction:
// four rows of 256 bytes per load and per store, all loads first.
template <int LOADS>
__global__ __launch_bounds__(256) void widePanelsKernel(const float* in, float* out, uint32_t longDim,
                                                        uint32_t inShort, uint32_t outShort) {
  const uint32_t lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const uint32_t x = blockIdx.x * 256 + wave * 64 + 4 * (lane % 16), q = lane / 16;
  if (x + 4 > longDim) return;
  v4f v[LOADS];
#pragma unroll
  for (int u = 0; u < LOADS; ++u) {
    const uint32_t k = 4 * u + q;
    v[u] = *reinterpret_cast<const v4f*>(in + size_t(k < inShort ? k : inShort - 1) * longDim + x);
  }
  v4f acc = v[0];
#pragma unroll
  for (int u = 1; u < LOADS; ++u)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = v[u][c] > acc[c] ? v[u][c] : acc[c];
  for (uint32_t r = q; r < outShort; r += 4) *reinterpret_cast<v4f*>(out + size_t(r) * longDim + x) = acc;
}

extern "C" {

// `reads` input streams of n floats each combined into one output stream of n
// floats (reads in 0..4; n a multiple of 4), every stream an allocation of its
// own; groups of 128 lanes, 256 for reads == 0 (the builtins' shapes).  Bytes
// per launch: 4n(reads + 1).  xcdRanges != 0: each XCD works through a
// contiguous eighth of every stream.  outShiftFloats: the output starts that
// many floats behind a 128-byte boundary, so that a wave's 16-byte stores
// straddle lines (and 16-byte boundaries, if not a multiple of 4).  plainStores:
// ordinary cacheable stores instead of the write-through streaming ones.
int polar_probe_streams(int reads, uint64_t n, int xcdRanges, int outShiftFloats, int plainStores, int sets,
                        int warm, int reps, float* us) {
  if (reads < 0 || reads > 4 || n % 4 != 0 || n == 0 || sets < 1 || reps < 1 || outShiftFloats < 0 ||
      outShiftFloats > 31)
    return hipErrorInvalidValue;
  Buffers mem;
  Stream st;
  PROBE_TRY(hipSetDevice(0));
  PROBE_TRY(st.make());
  std::vector<StreamPointers> ptrs(sets);
  for (int k = 0; k < sets; ++k) {
    for (int s = 0; s < 4; ++s) ptrs[k].in[s] = nullptr;
    for (int s = 0; s < reads; ++s) {
      void* b = nullptr;
      PROBE_TRY(mem.add(n * 4, &b));
      ptrs[k].in[s] = static_cast<const v4f*>(b);
    }
    void* o = nullptr;
    PROBE_TRY(mem.add(n * 4 + 128, &o));
    ptrs[k].out = reinterpret_cast<v4f*>(static_cast<float*>(o) + outShiftFloats);
  }
  const uint64_t n4 = n / 4;
  return timeLaunches(st.s, warm, reps, us, [&](int i, hipEvent_t e0, hipEvent_t e1) {
    const StreamPointers& p = ptrs[i % sets];
    switch (reads) {
    case 0: launchStreams<0, 256>(st.s, e0, e1, p, n4, xcdRanges, plainStores); break;
    case 1: launchStreams<1, 128>(st.s, e0, e1, p, n4, xcdRanges, plainStores); break;
    case 2: launchStreams<2, 128>(st.s, e0, e1, p, n4, xcdRanges, plainStores); break;
    case 3: launchStreams<3, 128>(st.s, e0, e1, p, n4, xcdRanges, plainStores); break;
    default: launchStreams<4, 128>(st.s, e0, e1, p, n4, xcdRanges, plainStores); break;
    }
  });
}

// Read n floats and write next to nothing (one float per wave).  unroll: 16-byte
// loads in flight per lane, one of 2, 4, 8, 16.  Bytes per launch: 4n.
int polar_probe_read(uint64_t n, int unroll, int sets, int warm, int reps, float* us) {
  if (n % 4 != 0 || n == 0 || sets < 1 || reps < 1) return hipErrorInvalidValue;
  if (unroll != 2 && unroll != 4 && unroll != 8 && unroll != 16) return hipErrorInvalidValue;
  Buffers mem;
  Stream st;
  PROBE_TRY(hipSetDevice(0));
  PROBE_TRY(st.make());
  std::vector<v4f*> ins(sets);
  for (int k = 0; k < sets; ++k) PROBE_TRY(mem.add(n * 4, reinterpret_cast<void**>(&ins[k])));
  const uint64_t n4 = n / 4;
  const unsigned grid = static_cast<unsigned>((n4 + 256ull * unroll - 1) / (256ull * unroll));
  float* out = nullptr;
  PROBE_TRY(mem.add(size_t(grid) * 4 * sizeof(float), reinterpret_cast<void**>(&out)));
  return timeLaunches(st.s, warm, reps, us, [&](int i, hipEvent_t e0, hipEvent_t e1) {
    const v4f* in = ins[i % sets];
    switch (unroll) {
    case 2: hipExtLaunchKernelGGL(readKernel<2>, dim3(grid), dim3(256), 0, st.s, e0, e1, 0, in, out, n4); break;
    case 4: hipExtLaunchKernelGGL(readKernel<4>, dim3(grid), dim3(256), 0, st.s, e0, e1, 0, in, out, n4); break;
    case 8: hipExtLaunchKernelGGL(readKernel<8>, dim3(grid), dim3(256), 0, st.s, e0, e1, 0, in, out, n4); break;
    default: hipExtLaunchKernelGGL(readKernel<16>, dim3(grid), dim3(256), 0, st.s, e0, e1, 0, in, out, n4); break;
    }
  });
}

// The memory pattern of a tiled rows x cols fp32 transpose.  variant selects
// the tile: 0 = 32 x 256 (1024 lanes), 1 = 32 x 128 (512 lanes), 2 = 32 x 128
// (256 lanes), 3 = 64 x 256 (1024 lanes), 4 = 32 x 64 (256 lanes), 5 = 128 x 64
// (512 lanes: 512-byte chunks per output row); order: 0 =
// row tiles fastest, 1 = column tiles fastest, 2 = a contiguous range of column
// tiles per XCD.  Bytes per launch: 8 rows cols.
int polar_probe_transpose_pattern(uint32_t rows, uint32_t cols, int variant, int order, int sets,
                                  int warm, int reps, float* us) {
  if (rows == 0 || cols == 0 || variant < 0 || variant > 5 || order < 0 || order > 2 || sets < 1 ||
      reps < 1 || uint64_t(rows) * cols >= (1ull << 31))
    return hipErrorInvalidValue;
  Buffers mem;
  Stream st;
  PROBE_TRY(hipSetDevice(0));
  PROBE_TRY(st.make());
  const size_t bytes = size_t(rows) * cols * 4 + 4096;
  std::vector<float*> ins(sets), outs(sets);
  for (int k = 0; k < sets; ++k) {
    PROBE_TRY(mem.add(bytes, reinterpret_cast<void**>(&ins[k])));
    PROBE_TRY(mem.add(bytes, reinterpret_cast<void**>(&outs[k])));
  }
  return timeLaunches(st.s, warm, reps, us, [&](int i, hipEvent_t e0, hipEvent_t e1) {
    const float* in = ins[i % sets];
    float* out = outs[i % sets];
    switch (variant) {
    case 0: launchPattern<32, 256, 1024>(st.s, e0, e1, in, out, rows, cols, order); break;
    case 1: launchPattern<32, 128, 512>(st.s, e0, e1, in, out, rows, cols, order); break;
    case 2: launchPattern<32, 128, 256>(st.s, e0, e1, in, out, rows, cols, order); break;
    case 3: launchPattern<64, 256, 1024>(st.s, e0, e1, in, out, rows, cols, order); break;
    case 4: launchPattern<32, 64, 256>(st.s, e0, e1, in, out, rows, cols, order); break;
    default: launchPattern<128, 64, 512>(st.s, e0, e1, in, out, rows, cols, order); break;
    }
  });
}

// The memory pattern of C[long x outShort] = A[long x inShort] * B (wide = 0:
// rows of inShort floats in, rows of outShort floats out) or of its mirror
// image C[outShort x long] = A * B[inShort x long] (wide = 1).  inShort <= 128;
// tall needs 32 * inShort <= 4096, both need the long dimension to be a
// multiple of 4.  Bytes per launch: 4 long (inShort + outShort).
int polar_probe_panels(int wide, uint32_t longDim, uint32_t inShort, uint32_t outShort, int sets, int warm,
                       int reps, float* us) {
  if (longDim == 0 || longDim % 4 != 0 || inShort == 0 || inShort > 128 || outShort == 0 || outShort > 128 ||
      sets < 1 || reps < 1)
    return hipErrorInvalidValue;
  Buffers mem;
  Stream st;
  PROBE_TRY(hipSetDevice(0));
  PROBE_TRY(st.make());
  std::vector<float*> ins(sets), outs(sets);
  for (int k = 0; k < sets; ++k) {
    PROBE_TRY(mem.add(size_t(longDim) * inShort * 4 + 4096, reinterpret_cast<void**>(&ins[k])));
    PROBE_TRY(mem.add(size_t(longDim) * outShort * 4 + 4096, reinterpret_cast<void**>(&outs[k])));
  }
  const unsigned grid = (longDim + 255) / 256;
  return timeLaunches(st.s, warm, reps, us, [&](int i, hipEvent_t e0, hipEvent_t e1) {
    const float* in = ins[i % sets];
    float* out = outs[i % sets];
    if (!wide)
      hipExtLaunchKernelGGL(tallPanelsKernel, dim3(grid), dim3(512), 0, st.s, e0, e1, 0, in, out, longDim, inShort,
                            outShort);
    else if (inShort <= 32)
      hipExtLaunchKernelGGL(widePanelsKernel<8>, dim3(grid), dim3(256), 0, st.s, e0, e1, 0, in, out, longDim,
                            inShort, outShort);
    else if (inShort <= 64)
      hipExtLaunchKernelGGL(widePanelsKernel<16>, dim3(grid), dim3(256), 0, st.s, e0, e1, 0, in, out, longDim,
                            inShort, outShort);
    else
      hipExtLaunchKernelGGL(widePanelsKernel<32>, dim3(grid), dim3(256), 0, st.s, e0, e1, 0, in, out, longDim,
                            inShort, outShort);
  });
}

} // extern "C"
