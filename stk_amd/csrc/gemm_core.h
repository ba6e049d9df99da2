// MFMA tile engine shared by the sdd / dsd / dds kernels (gfx950 only).
//
// A workgroup of 4 or 8 wavefronts (WM x WN, or 4 along K) produces one TM x TN
// output tile.  Every wavefront owns a (32 IM) x (32 JN) sub-tile held as IM x JN
// accumulators of v_mfma_f32_32x32x16_{bf16,f16}: 64x64 for 128x128 tiles of four
// wavefronts, 64x128 or 96x64 for the 256x256 and 384x128 tiles of eight that
// read each operand once for two to four blocks.  The contraction dimension is
// consumed in K-tiles of KT (32 or 64) elements that are staged through a ring of
// LDS buffers.  An operand may consist of up to four parts with separate origins
// (sparse blocks that share the other operand); each part is an independent LDS tile.
//
// Operand tiles come in two memory layouts:
//   K-major   element (mn, k) at base + mn * ld + k   (row-major lhs, .t() rhs,
//             sparse block on the lhs, transposed sparse block on the rhs)
//   MN-major  element (mn, k) at base + k * ld + mn   (.t() lhs, row-major rhs,
//             transposed sparse block on the lhs, sparse block on the rhs)
// K-major tiles sit in LDS as [mn][KT k] and feed the MFMA through ds_read_b128;
// MN-major tiles sit as [KT k][mn] and feed it through the gfx950 transposing
// read ds_read_b64_tr_b16, so no layout needs a transposing copy.  Both LDS
// layouts are XOR-swizzled for the 64-bank LDS.
//
// Two pipelines move tiles from global memory to LDS:
//   mainloop_dma  full tiles only.  global_load_lds_dwordx4 writes LDS directly
//                 (no registers, no ds_write); the swizzle is applied by
//                 choosing which global chunk each lane fetches.  STAGES - 1
//                 K-tiles are in flight; completion is awaited with explicit
//                 s_waitcnt vmcnt(n) because the compiler does not see these
//                 loads.  One barrier per K-tile; with three or more stages the
//                 MFMA k-steps are software-pipelined across it.
//   mainloop_reg  ragged tiles (k, m or n tails).  Predicated 16-byte loads to
//                 registers, zero fill, ds_write, double-buffered LDS.
//
// The two MFMA operands are passed swapped (rhs fragment first), which makes
// each lane own 4 consecutive output columns of one output row; the epilogue
// packs them, stages the wave's 64x64 sub-tile in LDS and writes 16 bytes per
// lane in full 128-byte row segments; it can apply an activation to the sums and
// multiply the rounded values by a second array on the way.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace stk {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint16_t elem_t;  // raw 16-bit storage of bf16 / f16

#define STK_LDS __attribute__((address_space(3)))
#define STK_GLOBAL __attribute__((address_space(1)))


template <bool BF16>
__device__ __forceinline__ f32x16_t mfma_32x32x16(u32x4 a, u32x4 b, f32x16_t c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
}

// fp32 -> 16-bit with round-to-nearest-even, two values packed into a dword
// (one hardware conversion instruction per pair).
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
template <bool BF16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  if constexpr (BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  else return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
}

// Two packed 16-bit values -> fp32, and the element-wise product of two packed pairs,
// multiplied in fp32 and rounded once (what a 16-bit multiply of the two arrays gives).
template <bool BF16>
__device__ __forceinline__ f32x2_t unpack2(uint32_t v) {
  if constexpr (BF16) return f32x2_t{__builtin_bit_cast(float, v << 16), __builtin_bit_cast(float, v & 0xffff0000u)};
  else return __builtin_convertvector(__builtin_bit_cast(f16x2_t, v), f32x2_t);
}
template <bool BF16>
__device__ __forceinline__ uint32_t mul_packed(uint32_t a, uint32_t b) {
  const f32x2_t x = unpack2<BF16>(a), y = unpack2<BF16>(b);
  return pack2<BF16>(x.x * y.x, x.y * y.y);
}
// A packed pair times an fp32 factor: the product rounded to fp32, then to 16 bits.
template <bool BF16>
__device__ __forceinline__ uint32_t scale_packed(uint32_t a, float w) {
  const f32x2_t x = unpack2<BF16>(a);
  float lo = w * x.x, hi = w * x.y;
  // (final fp32 values: otherwise the multiplication and the conversion may become one mixed-precision
  // instruction that does not round the product to fp32 first)
  asm volatile("" : "+v"(lo), "+v"(hi));
  return pack2<BF16>(lo, hi);
}

// Activation functions that a product can apply to its fp32 accumulators before they are rounded.
// The second four are the derivatives of the first four: with the incoming gradient as the multiplier, a sampled product
// whose store applies one of them yields the gradient with respect to the sums of a product that applied the function.
enum Activation : int {
  kNoActivation = 0, kRelu = 1, kGeluTanh = 2, kGeluErf = 3, kSilu = 4,
  kReluGrad = 5, kGeluTanhGrad = 6, kGeluErfGrad = 7, kSiluGrad = 8, kActivations = 9
};
template <int KIND>
__device__ __forceinline__ float activate(float x) {
  // exp2 and the reciprocal are the hardware's approximations (1 ulp): the result is rounded to 16 bits
  if constexpr (KIND == kRelu) return x > 0.f ? x : 0.f;
  else if constexpr (KIND == kGeluTanh) {
    // 0.5 x (1 + tanh(u)) = x / (1 + exp(-2 u)), u = sqrt(2 / pi) (x + 0.044715 x^3); -2 u log2(e) = x (k1 + k3 x^2)
    constexpr float k1 = -2.f * 0.7978845608028654f * 1.4426950408889634f, k3 = k1 * 0.044715f;
    return x * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(x * (k1 + k3 * x * x)));
  } else if constexpr (KIND == kGeluErf) return 0.5f * x * (1.f + erff(x * 0.7071067811865476f));
  else if constexpr (KIND == kSilu) return x * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
  else if constexpr (KIND == kReluGrad) return x > 0.f ? 1.f : 0.f;
  else if constexpr (KIND == kGeluTanhGrad) {
    // d/dx [x s], s = 1 / (1 + exp(-2 u)):  s + x s (1 - s) 2 u',  2 u' = 2 sqrt(2 / pi) (1 + 3 * 0.044715 x^2)
    // (x is clamped: beyond +-1e4 the derivative is 1 or 0 to the last bit, and x^2 must stay finite)
    constexpr float c2 = 2.f * 0.7978845608028654f, k1 = -c2 * 1.4426950408889634f, k3 = k1 * 0.044715f;
    x = __builtin_amdgcn_fmed3f(x, -1e4f, 1e4f);
    const float s = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(x * (k1 + k3 * x * x)));
    return s * (1.f + x * (1.f - s) * (c2 + 3.f * 0.044715f * c2 * x * x));
  } else if constexpr (KIND == kGeluErfGrad) {
    // 0.5 (1 + erf(x / sqrt 2)) + x exp(-x^2 / 2) / sqrt(2 pi)
    return 0.5f * (1.f + erff(x * 0.7071067811865476f)) + x * 0.3989422804014327f * __builtin_amdgcn_exp2f(x * x * -0.7213475204444817f);
  } else if constexpr (KIND == kSiluGrad) {
    // s (1 + x (1 - s)), s = 1 / (1 + exp(-x))
    const float s = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
    return s * (1.f + x * (1.f - s));
  } else return x;
}

// v = activation(v) on the 16 values of an accumulator; kind is wave-uniform.
template <int KIND>
__device__ __forceinline__ void activate_16(f32x16_t& v) {
#pragma unroll
  for (int r = 0; r < 16; r++) v[r] = activate<KIND>(v[r]);
}
__device__ __forceinline__ void activate_all(f32x16_t& v, int kind) {
  switch (kind) {
    case kRelu: activate_16<kRelu>(v); break;
    case kGeluTanh: activate_16<kGeluTanh>(v); break;
    case kGeluErf: activate_16<kGeluErf>(v); break;
    case kSilu: activate_16<kSilu>(v); break;
    case kReluGrad: activate_16<kReluGrad>(v); break;
    case kGeluTanhGrad: activate_16<kGeluTanhGrad>(v); break;
    case kGeluErfGrad: activate_16<kGeluErfGrad>(v); break;
    case kSiluGrad: activate_16<kSiluGrad>(v); break;
    default: break;
  }
}

// Wave-uniform pointer into global memory, kept in scalar registers.  The explicit
// address space keeps loads on the global (not flat) path.
typedef const STK_GLOBAL char* gptr_t;
__device__ __forceinline__ gptr_t uniform_global(const void* p) {
  uint64_t v = reinterpret_cast<uint64_t>(p);
  uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (gptr_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// 16 bytes per lane from global memory straight into LDS: lane l of the wave
// writes LDS bytes [lds_base + 16 l, +16).  lds_base is wave-uniform (it travels
// in M0).  The load is tracked by vmcnt only; the caller waits for it.
// STREAM: non-temporal hint for data that is read once, so that it does not
// displace operands and results that are read again from the caches.
template <bool STREAM = false>
__device__ __forceinline__ void dma16(gptr_t base, uint32_t lane_offset, uint32_t lds_base) {
  if constexpr (STREAM)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                 :
                 : "s"(lds_base), "v"(lane_offset), "s"(base)
                 : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_base), "v"(lane_offset), "s"(base)
                 : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// ---------------------------------------------------------------------------
// One operand of a K-tile: ROWS (m or n extent of the workgroup tile) x KT k.
// LDS has 64 banks of 4 bytes: addresses 256 bytes apart share a bank, and wide
// accesses are served 256 bytes (16 lanes x 16 B, or 32 lanes x 8 B) per cycle.
// ---------------------------------------------------------------------------
template <int ROWS, bool KMAJOR, int KT, int NTHREADS>
struct Operand {
  static_assert(KT == 32 || KT == 64, "K-tile of 32 or 64");
  static constexpr int kBytes = ROWS * KT * 2;
  static constexpr int kWaves = NTHREADS / 64;
  static constexpr int kChunks = kBytes / 16 / NTHREADS;  // 16-byte chunks per thread (register path)
  static constexpr int kSlices = kBytes / 1024;           // 1 KiB wave-wide DMA transfers
  static constexpr int kSlicesPerWave = kSlices / kWaves;
  static_assert(kSlices % kWaves == 0 && kChunks >= 1, "tile too small for the workgroup");
  static constexpr int kCR = KT / 8;     // chunks per row (K-major)
  static constexpr int kRB = ROWS * 2;   // bytes per k row (MN-major)
  static constexpr int kCPR = kRB / 16;  // chunks per k row (MN-major)

  // K-major: 16 consecutive rows at one logical chunk must land on 16 distinct
  // 16-byte slots of a 256-byte bank row.
  __device__ __forceinline__ static int kmajor_swizzle(int row) {
    if constexpr (KT == 64) return (row >> 1) & 7;  // 2 rows per bank row
    else return (row >> 2) & 3;                     // 4 rows per bank row
  }
  __device__ __forceinline__ static int kmajor_offset(int row, int chunk) {
    return row * (KT * 2) + ((chunk ^ kmajor_swizzle(row)) << 4);
  }
  // MN-major: a transposing read touches 4 consecutive k rows x 64 bytes per 32
  // lanes; the 64-byte granule is XOR-ed so the 4 rows cover a whole bank row.
  __device__ __forceinline__ static int mnmajor_swizzle(int krow) {
    if constexpr (kRB >= 256) return (krow & 3) << 6;
    else return ((krow >> 1) & 1) << 6;
  }
  __device__ __forceinline__ static int mnmajor_offset(int krow, int col_byte) {
    return krow * kRB + (col_byte ^ mnmajor_swizzle(krow));
  }

  // ---- DMA path -----------------------------------------------------------
  // Global byte offset (from the tile origin) of the chunk that lane `lane`
  // must fetch so that slice `slice` (LDS bytes [1024 slice, +1024)) ends up in
  // the swizzled layout.  Loop invariant.
  __device__ __forceinline__ static uint32_t dma_lane_offset(int slice, int lane, int64_t ld) {
    if constexpr (KMAJOR) {
      int row = slice * (1024 / (KT * 2)) + lane / kCR;
      int chunk = (lane % kCR) ^ kmajor_swizzle(row);
      return (uint32_t)((row * ld + chunk * 8) * 2);
    } else {
      int krow = slice * (1024 / kRB) + lane / kCPR;
      int col_byte = ((lane % kCPR) << 4) ^ mnmajor_swizzle(krow);
      return (uint32_t)(krow * ld * 2 + col_byte);
    }
  }
  __device__ __forceinline__ static void dma_offsets(uint32_t (&off)[kSlicesPerWave], int wave, int lane, int64_t ld) {
#pragma unroll
    for (int i = 0; i < kSlicesPerWave; i++) off[i] = dma_lane_offset(i * kWaves + wave, lane, ld);
  }
  // The same for a K-major operand whose rows are gathered: row `row` of the tile is row source_row(row) of the
  // array at the tile origin (which then is the array's first row at the K-tile's k).
  template <class SourceRow>
  __device__ __forceinline__ static void dma_offsets_gathered(uint32_t (&off)[kSlicesPerWave], int wave, int lane, int64_t ld, SourceRow&& source_row) {
    static_assert(KMAJOR, "rows are gathered, not columns");
#pragma unroll
    for (int i = 0; i < kSlicesPerWave; i++) {
      const int row = (i * kWaves + wave) * (1024 / (KT * 2)) + lane / kCR;
      const int chunk = (lane % kCR) ^ kmajor_swizzle(row);
      off[i] = (uint32_t)(((int64_t)source_row(row) * ld + chunk * 8) * 2);
    }
  }

  // ---- register path --------------------------------------------------------
  __device__ __forceinline__ static void load(u32x4 (&r)[kChunks], const elem_t* base, int64_t ld,
                                              int mn_valid, int k_valid, int tid) {
#pragma unroll
    for (int i = 0; i < kChunks; i++) {
      int c = tid + i * NTHREADS;
      const elem_t* p;
      bool ok;
      if constexpr (KMAJOR) {
        int row = c / kCR, kc = c % kCR;
        ok = (row < mn_valid) && (kc * 8 < k_valid);
        p = base + (int64_t)row * ld + kc * 8;
      } else {
        int krow = c / kCPR, mc = c % kCPR;
        ok = (krow < k_valid) && (mc * 8 < mn_valid);
        p = base + (int64_t)krow * ld + mc * 8;
      }
      u32x4 v = {0u, 0u, 0u, 0u};
      if (ok) v = *reinterpret_cast<const u32x4*>(p);
      r[i] = v;
    }
  }
  __device__ __forceinline__ static void store(const u32x4 (&r)[kChunks], char* s, int tid) {
#pragma unroll
    for (int i = 0; i < kChunks; i++) {
      int c = tid + i * NTHREADS;
      int off;
      if constexpr (KMAJOR) off = kmajor_offset(c / kCR, c % kCR);
      else off = mnmajor_offset(c / kCPR, (c % kCPR) << 4);
      *reinterpret_cast<u32x4*>(s + off) = r[i];
    }
  }

  // ---- MFMA fragment --------------------------------------------------------
  // lane l gets element (mn_base + l % 32, k = 16 ks + 8 (l / 32) + 0..7).
  __device__ __forceinline__ static u32x4 frag(const char* s, int mn_base, int ks, int lane) {
    if constexpr (KMAJOR) {
      int row = mn_base + (lane & 31);
      int ch = ks * 2 + (lane >> 5);
      return *reinterpret_cast<const u32x4*>(s + kmajor_offset(row, ch));
    } else {
      // ds_read_b64_tr_b16: inside each group of 16 lanes, lane i fetches 4 consecutive
      // elements of k row (i / 4) at column chunk (i % 4); lane j receives column j of
      // the 4 rows.  Two reads give the 8 k values of the fragment.
      int krow = ks * 16 + 8 * (lane >> 5) + ((lane & 15) >> 2);
      int mn = mn_base + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
      int off = mnmajor_offset(krow, mn * 2);  // rows krow and krow + 4 share the swizzle term
      s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((STK_LDS s16x4_t*)(s + off));
      s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((STK_LDS s16x4_t*)(s + off + 4 * kRB));
      u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
      u32x4 v = {l2.x, l2.y, h2.x, h2.y};
      return v;
    }
  }
};

// ---------------------------------------------------------------------------
// Workgroup tile configuration.  WM x WN x WK wavefronts (4 or 8); every
// wavefront computes IM x JN MFMA tiles of 32x32.  WK > 1 splits every K-tile
// across wavefronts (used for 64x64 output tiles).  The A / B operand of the
// workgroup tile is made of A_PARTS / B_PARTS equal parts with their own origins.
// ---------------------------------------------------------------------------
template <int WM_, int WN_, int IM_, int JN_, int WK_, int A_PARTS_, int B_PARTS_, bool A_KMAJOR_, bool B_KMAJOR_,
          bool BF16_, int KT_, int STAGES_, bool STREAM_A_ = false, bool STREAM_B_ = false>
struct TileCfg {
  static constexpr int WM = WM_, WN = WN_, IM = IM_, JN = JN_, WK = WK_, KT = KT_, STAGES = STAGES_;
  static constexpr int A_PARTS = A_PARTS_, B_PARTS = B_PARTS_;
  static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_, BF16 = BF16_;
  // The launch reads the operand about once: the direct-to-LDS pipeline loads it non-temporally, so that it
  // does not displace operands and results that are read again from the caches.
  static constexpr bool STREAM_A = STREAM_A_, STREAM_B = STREAM_B_;
  static constexpr int kWaves = WM * WN * WK, kThreads = 64 * kWaves;
  static_assert(kWaves == 4 || kWaves == 8, "four or eight wavefronts per workgroup");
  static_assert(WK == 1 || (KT / 16 == WK && IM == 2 && JN == 2), "split-K: one MFMA k-step per wavefront, 64x64 tile");
  static_assert(JN % 2 == 0, "wave tile is made of 64-column strips");
  static constexpr int TM = 32 * IM * WM, TN = 32 * JN * WN;
  static constexpr int PM = TM / A_PARTS, PN = TN / B_PARTS;  // rows / columns per operand part
  static_assert(PM % 32 == 0 && PN % 32 == 0, "an MFMA tile lies inside one A part and one B part");
  using OpA = Operand<PM, A_KMAJOR, KT, kThreads>;
  using OpB = Operand<PN, B_KMAJOR, KT, kThreads>;
  static constexpr int kStageBytes = A_PARTS * OpA::kBytes + B_PARTS * OpB::kBytes;
  static constexpr int kEpilogueBytes = (WK > 1) ? 4 * 3 * 32 * 32 * 4 : kWaves * 8192;
  static constexpr int kSmemBytes = (STAGES * kStageBytes > kEpilogueBytes) ? STAGES * kStageBytes : kEpilogueBytes;
  static constexpr int kAccRegs = IM * JN;
};

constexpr int kMaxSegments = 64;  // walk entries of a sparse line held at a time, one per lane of every wavefront

struct TilePtrs {
  const elem_t* a[4];  // element (m = 0, k = 0) of each part of the A tile
  const elem_t* b[4];  // element (k = 0, n = 0) of each part of the B tile
  int k_valid;         // valid k extent of this K-tile (register path only)
};

// Operand fragments of one MFMA k-step (16 k) of a wavefront's sub-tile.
template <class Cfg>
struct Frags {
  u32x4 a[Cfg::IM], b[Cfg::JN];
};
// Reads the fragments of k-step ks of the K-tile held in LDS at `stage` (the A parts followed by
// the B parts); (wm, wn) select the wavefront's rows / columns.
template <class Cfg>
__device__ __forceinline__ void load_frags(Frags<Cfg>& f, const char* stage, int wm, int wn, int ks, int lane) {
  using OpA = typename Cfg::OpA;
  using OpB = typename Cfg::OpB;
  const int m0 = wm * 32 * Cfg::IM, n0 = wn * 32 * Cfg::JN;  // within the workgroup tile
  const char* sb = stage + Cfg::A_PARTS * OpA::kBytes;
#pragma unroll
  for (int i = 0; i < Cfg::IM; i++) {
    const int m = m0 + i * 32;  // a wave tile may straddle parts; a 32-wide MFMA tile does not
    f.a[i] = OpA::frag(stage + (m / Cfg::PM) * OpA::kBytes, m % Cfg::PM, ks, lane);
  }
#pragma unroll
  for (int j = 0; j < Cfg::JN; j++) {
    const int n = n0 + j * 32;
    f.b[j] = OpB::frag(sb + (n / Cfg::PN) * OpB::kBytes, n % Cfg::PN, ks, lane);
  }
}
template <class Cfg>
__device__ __forceinline__ void mfma_frags(f32x16_t (&acc)[Cfg::IM][Cfg::JN], const Frags<Cfg>& f) {
#pragma unroll
  for (int i = 0; i < Cfg::IM; i++)
#pragma unroll
    for (int j = 0; j < Cfg::JN; j++) acc[i][j] = mfma_32x32x16<Cfg::BF16>(f.b[j], f.a[i], acc[i][j]);
}

// Scheduling of one k-step of the software pipeline: the fragment reads of the next k-step are spread between
// the MFMAs of the current one (an MFMA keeps its pipe busy for 32 cycles but the wavefront's issue only for a
// few: LDS reads issued in between cost nothing, issued as a block in front they leave the pipe idle).
template <class Cfg, int I = 0>
__device__ __forceinline__ void interleave_reads_with_mfmas() {
  constexpr int kMfmas = Cfg::IM * Cfg::JN;
  constexpr int kReads = (Cfg::A_KMAJOR ? 1 : 2) * Cfg::IM + (Cfg::B_KMAJOR ? 1 : 2) * Cfg::JN;
  constexpr int kPer = (kReads + kMfmas - 2) / (kMfmas - 1);  // reads behind each MFMA but the last
  if constexpr (I < kMfmas) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
    constexpr int kLeft = kReads - I * kPer;
    if constexpr (kLeft > 0) __builtin_amdgcn_sched_group_barrier(0x100, kLeft < kPer ? kLeft : kPer, 0);  // LDS reads
    interleave_reads_with_mfmas<Cfg, I + 1>();
  }
}

// acc += A_tile * B_tile for one K-tile held in LDS at `stage`.  The fragments of the next k-step are read
// while the MFMAs of the current one run (only the reads of the first k-step are exposed).
template <class Cfg>
__device__ __forceinline__ void compute_stage(f32x16_t (&acc)[Cfg::IM][Cfg::JN], const char* stage, int wm, int wn, int wk, int lane) {
  if constexpr (Cfg::WK > 1) {
    // split-K: this wavefront's only k-step
    Frags<Cfg> f;
    load_frags<Cfg>(f, stage, wm, wn, wk, lane);
    mfma_frags<Cfg>(acc, f);
  } else {
    constexpr int NKS = Cfg::KT / 16;
    Frags<Cfg> f[2];
    load_frags<Cfg>(f[0], stage, wm, wn, 0, lane);
#pragma unroll
    for (int ks = 0; ks < NKS; ks++) {
      __builtin_amdgcn_sched_barrier(0);
      if (ks + 1 < NKS) load_frags<Cfg>(f[(ks + 1) & 1], stage, wm, wn, ks + 1, lane);
      mfma_frags<Cfg>(acc, f[ks & 1]);
      if (ks + 1 < NKS) interleave_reads_with_mfmas<Cfg>();
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

struct WaveCoords {
  int lane, wave, wm, wn, wk;
};
template <class Cfg>
__device__ __forceinline__ WaveCoords wave_coords() {
  WaveCoords w;
  w.lane = threadIdx.x & 63;
  w.wave = uniform(threadIdx.x >> 6);
  w.wk = (Cfg::WK > 1) ? w.wave : 0;
  w.wm = (Cfg::WK > 1) ? 0 : w.wave % Cfg::WM;
  w.wn = (Cfg::WK > 1) ? 0 : w.wave / Cfg::WM;
  return w;
}

// Origin of the wavefront's sub-tile inside the workgroup tile.
template <class Cfg>
__device__ __forceinline__ int wave_m0(const WaveCoords& w) { return w.wm * 32 * Cfg::IM; }
template <class Cfg>
__device__ __forceinline__ int wave_n0(const WaveCoords& w) { return w.wn * 32 * Cfg::JN; }

// Compile-time loop: fn(Index<0>{}), ..., fn(Index<N - 1>{}).
template <int I>
struct Index {
  static constexpr int value = I;
};
template <int N, int I = 0, class Fn>
__device__ __forceinline__ void static_for(Fn&& fn) {
  if constexpr (I < N) {
    fn(Index<I>{});
    static_for<N, I + 1>(fn);
  }
}

// Full tiles: direct-to-LDS pipeline.  tile_fn(t) gives the operand origins of
// K-tile t; it is called exactly once per t, in increasing order.
// after_prologue() runs once, behind the transfers of the first STAGES - 1 K-tiles and in front of the first wait: work
// that does not depend on the tile (the caller's look-ahead) sits there in the shadow of the first transfers' latency.
// rows_a(q, row): the row of the array at part q's origin that holds row `row` of that part of the A tile
// (ConsecutiveRows: the rows follow each other from the origin; anything else needs a K-major A operand and offsets
// of less than 4 GiB from the origin).
struct ConsecutiveRows {};
template <class Cfg, class TileFn, class Hook, class RowsA>
__device__ __forceinline__ void mainloop_dma(f32x16_t (&acc)[Cfg::IM][Cfg::JN], int ntiles, TileFn&& tile_fn,
                                             int64_t lda, int64_t ldb, char* smem, Hook&& after_prologue, RowsA&& rows_a) {
  using OpA = typename Cfg::OpA;
  using OpB = typename Cfg::OpB;
  constexpr int S = Cfg::STAGES;
  constexpr int kLoadsA = Cfg::A_PARTS * OpA::kSlicesPerWave;
  constexpr int kLoadsPerTile = kLoadsA + Cfg::B_PARTS * OpB::kSlicesPerWave;  // per wavefront
  static_assert(S >= 2 && S <= 5 && (S - 2) * kLoadsPerTile < 64, "vmcnt is a 6-bit counter");
  const WaveCoords w = wave_coords<Cfg>();
  const uint32_t lds0 = (uint32_t)(uintptr_t)((STK_LDS char*)smem);

  constexpr bool kGathered = !std::is_same<typename std::decay<RowsA>::type, ConsecutiveRows>::value;
  uint32_t offa[kGathered ? Cfg::A_PARTS : 1][OpA::kSlicesPerWave], offb[OpB::kSlicesPerWave];
  if constexpr (kGathered) {
#pragma unroll
    for (int q = 0; q < Cfg::A_PARTS; q++) OpA::dma_offsets_gathered(offa[q], w.wave, w.lane, lda, [&](int row) { return rows_a(q, row); });
  } else {
    OpA::dma_offsets(offa[0], w.wave, w.lane, lda);
  }
  OpB::dma_offsets(offb, w.wave, w.lane, ldb);
  // The loads of K-tile t in two steps: the operand origins as scalar pointers (address arithmetic that can
  // run in the shadow of MFMAs), then the transfers themselves, one 1 KiB piece per call.
  struct Origins {
    gptr_t a[Cfg::A_PARTS], b[Cfg::B_PARTS];
  };
  auto prepare = [&](int t) {
    TilePtrs p = tile_fn(t);
    Origins o;
#pragma unroll
    for (int q = 0; q < Cfg::A_PARTS; q++) o.a[q] = uniform_global(p.a[q]);
#pragma unroll
    for (int q = 0; q < Cfg::B_PARTS; q++) o.b[q] = uniform_global(p.b[q]);
    return o;
  };
  auto stage_of = [&](int t) { return lds0 + (uint32_t)(t % S) * Cfg::kStageBytes; };
  auto fire_piece = [&](const Origins& o, uint32_t stage, auto piece) {
    constexpr int P = decltype(piece)::value;
    if constexpr (P < kLoadsA) {
      constexpr int q = P / OpA::kSlicesPerWave, i = P % OpA::kSlicesPerWave;
      dma16<Cfg::STREAM_A>(o.a[q], offa[kGathered ? q : 0][i], stage + q * OpA::kBytes + (i * OpA::kWaves + w.wave) * 1024);
    } else if constexpr (P < kLoadsPerTile) {
      constexpr int q = (P - kLoadsA) / OpB::kSlicesPerWave, i = (P - kLoadsA) % OpB::kSlicesPerWave;
      dma16<Cfg::STREAM_B>(o.b[q], offb[i], stage + Cfg::A_PARTS * OpA::kBytes + q * OpB::kBytes + (i * OpB::kWaves + w.wave) * 1024);
    }
  };
  auto issue = [&](int t) {
    const Origins o = prepare(t);
    const uint32_t stage = stage_of(t);
    static_for<kLoadsPerTile>([&](auto piece) { fire_piece(o, stage, piece); });
  };
#pragma unroll
  for (int s = 0; s < S - 1; s++)
    if (s < ntiles) issue(s);
  after_prologue();

  if constexpr (Cfg::WK == 1 && S >= 3) {
    // Software pipeline over the MFMA k-steps: the fragments of the next k-step are read
    // from LDS while the MFMAs of the current one run, also across K-tiles.  The wait and
    // the barrier for K-tile t + 1 therefore sit before the last k-step of K-tile t; the
    // stage refilled after that barrier is the one of K-tile t - 1, which every wavefront
    // has left.  K-tile t + 1 must have landed one k-step early, which leaves S - 3 younger
    // K-tiles in flight at the wait.
    constexpr int NKS = Cfg::KT / 16;
    constexpr int kMfmas = Cfg::IM * Cfg::JN;
    constexpr int kPiecesPerMfma = (kLoadsPerTile + kMfmas - 1) / kMfmas;
    static_assert(NKS % 2 == 0 && S <= 5, "fragment buffers alternate per k-step; the waits below cover three to five stages");
    if (ntiles > 0) {
      // K-tile 0 must have landed; the younger ones of the first S - 1 may stay in flight
      if (S >= 5 && ntiles >= 4) wait_vmcnt<3 * kLoadsPerTile>();
      else if (S >= 4 && ntiles >= 3) wait_vmcnt<2 * kLoadsPerTile>();
      else if (ntiles >= 2) wait_vmcnt<1 * kLoadsPerTile>();
      else wait_vmcnt<0>();
      __syncthreads();
      Frags<Cfg> f[2];
      load_frags<Cfg>(f[0], smem, w.wm, w.wn, 0, w.lane);
      // One k-step that is not the last of its K-tile: the MFMAs on `cur`, the reads of `next` in between.
      auto inner_step = [&](const Frags<Cfg>& cur, Frags<Cfg>& next, const char* stage, int ks_next) {
        load_frags<Cfg>(next, stage, w.wm, w.wn, ks_next, w.lane);
        mfma_frags<Cfg>(acc, cur);
        interleave_reads_with_mfmas<Cfg>();
      };
      // K-tile t, not the last one.  REFILL: K-tile t + S - 1 exists (it then also follows that K-tile t + 2
      // does); it is loaded behind the barrier, piece by piece between the MFMAs of the last k-step, after
      // the fragment read that goes with each MFMA.
      auto ktile = [&](int t, auto refill_tag) {
        constexpr bool REFILL = decltype(refill_tag)::value != 0;
        const char* stage = smem + (t % S) * Cfg::kStageBytes;
        Origins refill = {};
#pragma unroll
        for (int ks = 0; ks + 1 < NKS; ks++) {
          __builtin_amdgcn_sched_barrier(0);
          // (the origins of the refill, worked out in the shadow of this k-step's MFMAs)
          if (REFILL && ks + 2 == NKS) refill = prepare(t + S - 1);
          inner_step(f[ks & 1], f[(ks + 1) & 1], stage, ks + 1);
          __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (REFILL) {
          wait_vmcnt<(S - 3) * kLoadsPerTile>();
        } else {
          // no refill any more: K-tiles t + 2 .. ntiles - 1 (at most S - 3 of them) are still in flight
          if (S >= 5 && t + 3 < ntiles) wait_vmcnt<2 * kLoadsPerTile>();
          else if (S >= 4 && t + 2 < ntiles) wait_vmcnt<1 * kLoadsPerTile>();
          else wait_vmcnt<0>();
        }
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        const char* next_stage = smem + ((t + 1) % S) * Cfg::kStageBytes;
        const Frags<Cfg>& cur = f[(NKS - 1) & 1];
        if constexpr (REFILL) {
          const uint32_t target = stage_of(t + S - 1);
          const int m0 = w.wm * 32 * Cfg::IM, n0 = w.wn * 32 * Cfg::JN;
          const char* sb = next_stage + Cfg::A_PARTS * OpA::kBytes;
          static_for<kMfmas>([&](auto q_) {
            constexpr int q = decltype(q_)::value, i = q / Cfg::JN, j = q % Cfg::JN;
            acc[i][j] = mfma_32x32x16<Cfg::BF16>(cur.b[j], cur.a[i], acc[i][j]);
            if constexpr (q < Cfg::IM) {
              const int m = m0 + q * 32;
              f[0].a[q] = OpA::frag(next_stage + (m / Cfg::PM) * OpA::kBytes, m % Cfg::PM, 0, w.lane);
            } else if constexpr (q < Cfg::IM + Cfg::JN) {
              const int n = n0 + (q - Cfg::IM) * 32;
              f[0].b[q - Cfg::IM] = OpB::frag(sb + (n / Cfg::PN) * OpB::kBytes, n % Cfg::PN, 0, w.lane);
            }
            static_for<kPiecesPerMfma>([&](auto r_) { fire_piece(refill, target, Index<q * kPiecesPerMfma + decltype(r_)::value>{}); });
            __builtin_amdgcn_sched_barrier(0);
          });
        } else {
          inner_step(cur, f[0], next_stage, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
      };
      // All K-tiles but the last (kept apart so that the reads of the next K-tile's first
      // fragments are in flight on every path through the loop body, and the wait before
      // the MFMAs can leave them in flight): first those that refill a stage, then the rest.
      int t = 0;
      for (; t + S - 1 < ntiles; t++) ktile(t, Index<1>{});
      for (; t + 1 < ntiles; t++) ktile(t, Index<0>{});
      const char* stage = smem + ((ntiles - 1) % S) * Cfg::kStageBytes;
#pragma unroll
      for (int ks = 0; ks < NKS; ks++) {
        __builtin_amdgcn_sched_barrier(0);
        if (ks + 1 < NKS) load_frags<Cfg>(f[(ks + 1) & 1], stage, w.wm, w.wn, ks + 1, w.lane);
        mfma_frags<Cfg>(acc, f[ks & 1]);
        if (ks + 1 < NKS) interleave_reads_with_mfmas<Cfg>();
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  } else {
    for (int t = 0; t < ntiles; t++) {
      // Tile t must have landed; up to S - 2 younger tiles may stay in flight.
      const int younger = ntiles - 1 - t;
      if (S >= 5 && younger >= 3) wait_vmcnt<3 * kLoadsPerTile>();
      else if (S >= 4 && younger >= 2) wait_vmcnt<2 * kLoadsPerTile>();
      else if (S >= 3 && younger >= 1) wait_vmcnt<1 * kLoadsPerTile>();
      else wait_vmcnt<0>();
      // Barrier: (a) every wavefront's part of tile t is visible, (b) every wavefront
      // has finished the MFMAs of tile t - 1, whose stage is the one refilled below.
      __syncthreads();
      if (t + S - 1 < ntiles) issue(t + S - 1);
      compute_stage<Cfg>(acc, smem + (t % S) * Cfg::kStageBytes, w.wm, w.wn, w.wk, w.lane);
    }
  }
  __syncthreads();  // operand reads done before the epilogue reuses LDS
}
template <class Cfg, class TileFn, class Hook>
__device__ __forceinline__ void mainloop_dma(f32x16_t (&acc)[Cfg::IM][Cfg::JN], int ntiles, TileFn&& tile_fn,
                                             int64_t lda, int64_t ldb, char* smem, Hook&& after_prologue) {
  mainloop_dma<Cfg>(acc, ntiles, tile_fn, lda, ldb, smem, after_prologue, ConsecutiveRows{});
}
template <class Cfg, class TileFn>
__device__ __forceinline__ void mainloop_dma(f32x16_t (&acc)[Cfg::IM][Cfg::JN], int ntiles, TileFn&& tile_fn,
                                             int64_t lda, int64_t ldb, char* smem) {
  mainloop_dma<Cfg>(acc, ntiles, tile_fn, lda, ldb, smem, [] {}, ConsecutiveRows{});
}

// Ragged tiles: predicated register staging, two LDS stages.
template <class Cfg, class TileFn>
__device__ __forceinline__ void mainloop_reg(f32x16_t (&acc)[Cfg::IM][Cfg::JN], int ntiles, TileFn&& tile_fn,
                                             int64_t lda, int64_t ldb, int m_valid, int n_valid, char* smem) {
  using OpA = typename Cfg::OpA;
  using OpB = typename Cfg::OpB;
  const int tid = threadIdx.x;
  const WaveCoords w = wave_coords<Cfg>();
  static_assert(Cfg::A_PARTS == 1 && Cfg::B_PARTS == 1, "the register path handles single-part operands");
  u32x4 ra[OpA::kChunks], rb[OpB::kChunks];
  if (ntiles > 0) {
    TilePtrs p = tile_fn(0);
    OpA::load(ra, p.a[0], lda, m_valid, p.k_valid, tid);
    OpB::load(rb, p.b[0], ldb, n_valid, p.k_valid, tid);
    OpA::store(ra, smem, tid);
    OpB::store(rb, smem + OpA::kBytes, tid);
  }
  __syncthreads();
  for (int t = 0; t < ntiles; t++) {
    char* cur = smem + (t & 1) * Cfg::kStageBytes;
    char* nxt = smem + ((t + 1) & 1) * Cfg::kStageBytes;
    const bool more = t + 1 < ntiles;
    if (more) {
      TilePtrs p = tile_fn(t + 1);
      OpA::load(ra, p.a[0], lda, m_valid, p.k_valid, tid);
      OpB::load(rb, p.b[0], ldb, n_valid, p.k_valid, tid);
    }
    compute_stage<Cfg>(acc, cur, w.wm, w.wn, w.wk, w.lane);
    if (more) {
      OpA::store(ra, nxt, tid);
      OpB::store(rb, nxt + OpA::kBytes, tid);
    }
    __syncthreads();
  }
}

// Where row m of a 64-row staging quadrant (rows of 128 bytes) keeps its pieces: bits 0-2 are XOR-ed into the index of
// the 16-byte piece, bit 3 swaps the two 8-byte halves of a piece.  A staging write (64 lanes x 8 bytes: rows m ..
// m + 31 of one piece column, both halves) then touches every bank once per 16 lanes whether the banks repeat every 128
// or every 256 bytes: 16 consecutive rows get 16 different (piece, half) places, and the rows 16 apart, which share
// a place, differ in the parity that selects the upper or lower 128 bytes of a 256-byte bank row.
__device__ __forceinline__ int staging_swizzle(int m) { return (m ^ ((m >> 4) & 1)) & 15; }

// Writes the wavefront's part of the workgroup tile.  `out` points at element
// (0, 0) of the wavefront's sub-tile, ldc in elements; rows >= m_valid and
// columns >= n_valid (both relative to `out`, n_valid a multiple of 8) are
// skipped.  Lane l holds, in acc[i][j][4 g + q], the element
// (m = 32 i + l % 32, n = 32 j + 8 g + 4 (l / 32) + q) of the sub-tile.  Each
// 64x64 quadrant is packed to 16 bits, staged in the wavefront's own 8 KiB of
// LDS and written as 16 bytes per lane in 128-byte row segments; the wavefronts
// run through it independently of each other.
// The caller guarantees that no wavefront still reads operand tiles from LDS.
// STREAM: the output is not read again soon (large dense results); it is written
// with non-temporal stores so that it does not displace the operands from the caches.
// quadrant_stride: elements from one 64-column quadrant of the sub-tile to the next (64: they are neighbours in
// the rows of `out`; a block size: every quadrant is a 64-block of its own).
// row_jump: extra elements between row 128 k - 1 and row 128 k of the workgroup tile (whose row row_base is
// the sub-tile's first), for outputs made of 128-row blocks that do not follow each other in memory.
// activation (wave-uniform): applied to the fp32 sums before they are rounded.
// mul (wave-uniform, or null): an array laid out like `out`, pointing at the same element; the rounded
// values are multiplied by its elements and rounded again.  With the derivative of an activation the product is a
// gradient, not the product of two stored matrices: the fp32 derivative is multiplied by the element and the product
// is rounded once.
// SCATTER: row gm of the sub-tile goes to row row_map[gm] of the array whose row 0 `out` then points into (at the
// sub-tile's first column); rows whose entry is negative or not below out_rows are dropped.  row_scale (or null):
// fp32 factors by destination row; the rounded values are multiplied by them and rounded again.
// sums (wave-uniform, or null): an array laid out like `out`, pointing at the same element; it receives the sums
// rounded to 16 bits as they are, before the activation and the multiplier.
template <class Cfg, bool STREAM, bool SCATTER = false>
__device__ __forceinline__ void epilogue(f32x16_t (&acc)[Cfg::IM][Cfg::JN], elem_t* out, int64_t ldc,
                                         int m_valid, int n_valid, char* smem, int64_t quadrant_stride = 64,
                                         int activation = kNoActivation, const elem_t* mul = nullptr,
                                         int row_base = 0, int64_t row_jump = 0, const int32_t* row_map = nullptr,
                                         const float* row_scale = nullptr, int out_rows = 0, elem_t* sums = nullptr) {
  static_assert(!SCATTER || Cfg::WK == 1, "scattered rows: whole-K wavefront tiles only");
  // (the thread's id through an opaque statement: in a workgroup that loops over tiles the store addresses below would
  // otherwise be computed once in front of the loop and held in registers through every K loop)
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if constexpr (Cfg::WK == 1) {
    char* s = smem + wave * 8192;  // [64 m][64 n] 16-bit, rows of 128 bytes, 8-byte units swizzled by the row (staging_swizzle)
#pragma unroll
    for (int qi = 0; qi < (Cfg::IM + 1) / 2; qi++)
#pragma unroll
      for (int qj = 0; qj < Cfg::JN / 2; qj++) {
        constexpr int kOdd = Cfg::IM & 1;
        const int strips = (kOdd && qi == Cfg::IM / 2) ? 1 : 2;  // 32-row strips in this pass (the last one of an odd IM has one)
        // where piece `it` of this pass goes: row gm, eight columns from gn, element offset `at` in out (and mul)
        auto place = [&](int it, int& gm, int& gn) {
          const int m = it * 8 + (lane >> 3), ch = lane & 7;
          gm = qi * 64 + m, gn = qj * 64 + ch * 8;
          return (int64_t)gm * ldc + qj * quadrant_stride + ch * 8 + (int64_t)((row_base + gm) >> 7) * row_jump;
        };
        // scattered rows: where this pass's rows go and what they are scaled by, read once
        int dest[SCATTER ? 8 : 1];
        float scale[SCATTER ? 8 : 1];
        if constexpr (SCATTER) {
#pragma unroll
          for (int it = 0; it < 8; it++) {
            const int gm = qi * 64 + it * 8 + (lane >> 3);
            int d = -1;
            if (it < 4 * strips && gm < m_valid) d = row_map[gm];
            dest[it] = d < out_rows ? d : -1;
          }
#pragma unroll
          for (int it = 0; it < 8; it++) scale[it] = (row_scale && dest[it] >= 0) ? row_scale[dest[it]] : 1.0f;
        }
        // the multiplier's values of this pass, read once: on their way while the sums are rounded and staged
        const bool one_rounding = mul && activation >= kReluGrad;
        u32x4 factor[8];
        if (mul && !one_rounding) {
#pragma unroll
          for (int it = 0; it < 8; it++) {
            int gm, gn;
            const int64_t at = place(it, gm, gn);
            factor[it] = u32x4{0u, 0u, 0u, 0u};
            if (it < 4 * strips && gm < m_valid && gn < n_valid) factor[it] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(mul + at));
          }
        }
        // rounds this pass's sums to 16 bits and puts them into the staging buffer, element (m, n) of the pass's 64 x 64
        // quadrant at row m, 8-byte unit swizzled by the row
        auto stage = [&]() {
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
              for (int g = 0; g < 4; g++) {
                if (i >= strips) continue;
                const f32x16_t& c = acc[(2 * qi + i) < Cfg::IM ? 2 * qi + i : 0][2 * qj + j];
                int m = i * 32 + (lane & 31);
                int ch = 4 * j + g;
                u32x2 v = {pack2<Cfg::BF16>(c[4 * g], c[4 * g + 1]), pack2<Cfg::BF16>(c[4 * g + 2], c[4 * g + 3])};
                const int sw = staging_swizzle(m);
                *reinterpret_cast<u32x2*>(s + m * 128 + ((ch ^ (sw & 7)) << 4) + ((((lane >> 5) ^ (sw >> 3)) & 1) << 3)) = v;
              }
        };
        // piece `it` of the staged pass: eight consecutive elements of a row
        // (no barrier: the staging buffer is private to the wavefront and LDS serves a wavefront's accesses in order)
        auto staged = [&](int it) {
          int m = it * 8 + (lane >> 3);
          int ch = lane & 7;
          const int sw = staging_swizzle(m);
          u32x4 v = *reinterpret_cast<const u32x4*>(s + m * 128 + ((ch ^ (sw & 7)) << 4));
          if (sw >> 3) v = u32x4{v.z, v.w, v.x, v.y};  // the two 8-byte halves were stored swapped
          return v;
        };
        if (sums) {
          // the sums themselves, rounded, before anything is applied to them
          stage();
#pragma unroll
          for (int it = 0; it < 8; it++) {
            if (it >= 4 * strips) continue;
            const u32x4 v = staged(it);
            int gm, gn;
            const int64_t at = place(it, gm, gn);
            if (gm < m_valid && gn < n_valid) *reinterpret_cast<u32x4*>(sums + at) = v;
          }
        }
        // (the activation of this pass's sums: arithmetic for the loads above to hide behind)
        if (activation != kNoActivation) {
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
              if (2 * qi + i < Cfg::IM) activate_all(acc[2 * qi + i][2 * qj + j], activation);
        }
        if (one_rounding) {
          // the multiplier's elements where the accumulators hold theirs: lane l has row 32 i + l % 32 and the four
          // columns from 32 j + 8 g + 4 (l / 32) of this pass's quadrant in values 4 g .. 4 g + 3
          u32x2 f[2][2][4];
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
              for (int g = 0; g < 4; g++) {
                const int gm = qi * 64 + i * 32 + (lane & 31), n = j * 32 + 8 * g + 4 * (lane >> 5);
                f[i][j][g] = u32x2{0u, 0u};
                if (i < strips && gm < m_valid && qj * 64 + n < n_valid)
                  f[i][j][g] = *reinterpret_cast<const u32x2*>(mul + (int64_t)gm * ldc + qj * quadrant_stride + n +
                                                               (int64_t)((row_base + gm) >> 7) * row_jump);
              }
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
              for (int g = 0; g < 4; g++) {
                if (i >= strips) continue;
                f32x16_t& c = acc[(2 * qi + i) < Cfg::IM ? 2 * qi + i : 0][2 * qj + j];
                const f32x2_t lo = unpack2<Cfg::BF16>(f[i][j][g].x), hi = unpack2<Cfg::BF16>(f[i][j][g].y);
                c[4 * g] *= lo.x, c[4 * g + 1] *= lo.y, c[4 * g + 2] *= hi.x, c[4 * g + 3] *= hi.y;
              }
        }
        stage();
#pragma unroll
        for (int it = 0; it < 8; it++) {
          if (it >= 4 * strips) continue;
          u32x4 v = staged(it);
          int gm, gn;
          int64_t at = place(it, gm, gn);
          bool wanted = gm < m_valid && gn < n_valid;
          if constexpr (SCATTER) {
            wanted = wanted && dest[it] >= 0;
            at = (int64_t)dest[it] * ldc + gn;
          }
          if (wanted) {
            if (mul && !one_rounding) {
              const u32x4 f = factor[it];
              v = u32x4{mul_packed<Cfg::BF16>(v.x, f.x), mul_packed<Cfg::BF16>(v.y, f.y), mul_packed<Cfg::BF16>(v.z, f.z), mul_packed<Cfg::BF16>(v.w, f.w)};
            }
            if constexpr (SCATTER) {
              if (row_scale) {
                const float f = scale[it];
                v = u32x4{scale_packed<Cfg::BF16>(v.x, f), scale_packed<Cfg::BF16>(v.y, f), scale_packed<Cfg::BF16>(v.z, f), scale_packed<Cfg::BF16>(v.w, f)};
              }
            }
            u32x4* dst = reinterpret_cast<u32x4*>(out + at);
            if constexpr (STREAM) __builtin_nontemporal_store(v, dst);
            else *dst = v;
          }
        }
      }
  } else {
    // Split-K across the four wavefronts of a 64x64 tile: wavefront w finishes the
    // 32x32 quadrant w.  Partials of the other three quadrants go through LDS as
    // [dst quadrant][slot][16 values][64 lanes] fp32.
    float* red = reinterpret_cast<float*>(smem);
#pragma unroll
    for (int q = 0; q < 4; q++) {
      if (q == wave) continue;
      int slot = (wave > q) ? wave - 1 : wave;  // 0..2 among the writers of quadrant q
#pragma unroll
      for (int r = 0; r < 16; r++) red[((q * 3 + slot) * 16 + r) * 64 + lane] = acc[q >> 1][q & 1][r];
    }
    __syncthreads();
    const int qi = wave >> 1, qj = wave & 1;
    f32x16_t sum = acc[0][0];
    if (wave == 1) sum = acc[0][1];
    if (wave == 2) sum = acc[1][0];
    if (wave == 3) sum = acc[1][1];
#pragma unroll
    for (int slot = 0; slot < 3; slot++)
#pragma unroll
      for (int r = 0; r < 16; r++) sum[r] += red[((wave * 3 + slot) * 16 + r) * 64 + lane];
    int gm = qi * 32 + (lane & 31);
    if (sums) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        int gn = qj * 32 + 8 * g + 4 * (lane >> 5);
        u32x2 v = {pack2<Cfg::BF16>(sum[4 * g], sum[4 * g + 1]), pack2<Cfg::BF16>(sum[4 * g + 2], sum[4 * g + 3])};
        if (gm < m_valid && gn < n_valid) *reinterpret_cast<u32x2*>(sums + (int64_t)gm * ldc + gn) = v;
      }
    }
    if (activation != kNoActivation) activate_all(sum, activation);
#pragma unroll
    for (int g = 0; g < 4; g++) {
      int gn = qj * 32 + 8 * g + 4 * (lane >> 5);
      u32x2 v = {pack2<Cfg::BF16>(sum[4 * g], sum[4 * g + 1]), pack2<Cfg::BF16>(sum[4 * g + 2], sum[4 * g + 3])};
      if (gm < m_valid && gn < n_valid) {
        if (mul) {
          const u32x2 f = *reinterpret_cast<const u32x2*>(mul + (int64_t)gm * ldc + gn);
          if (activation >= kReluGrad) {
            const f32x2_t lo = unpack2<Cfg::BF16>(f.x), hi = unpack2<Cfg::BF16>(f.y);
            v = u32x2{pack2<Cfg::BF16>(sum[4 * g] * lo.x, sum[4 * g + 1] * lo.y), pack2<Cfg::BF16>(sum[4 * g + 2] * hi.x, sum[4 * g + 3] * hi.y)};
          } else {
            v = u32x2{mul_packed<Cfg::BF16>(v.x, f.x), mul_packed<Cfg::BF16>(v.y, f.y)};
          }
        }
        *reinterpret_cast<u32x2*>(out + (int64_t)gm * ldc + gn) = v;
      }
    }
  }
}

// Workgroup id -> work item, so that each of the 8 XCDs (which take workgroup
// ids round-robin and own a private L2) receives a contiguous range of items.
__device__ __forceinline__ int xcd_chunked(int bid, int n) {
  int q = n >> 3, r = n & 7;
  int x = bid & 7;
  return x * q + (x < r ? x : r) + (bid >> 3);
}


// The same in small portions: the list is cut into groups of GROUP consecutive items, and each
// stretch of eight groups is spread over the eight XCDs, so that all of them move through the
// list at the same pace - whatever the cost of the items does along the list (walks of very
// different lengths in a skewed topology), and with the eight dies reading the same stretch of the
// operands from memory at about the same time - while the items of a group, neighbours that share
// operand tiles, still meet in one L2.  The tail that does not fill eight groups is taken in order.
constexpr int kXcdGroup = 32;
template <int GROUP = kXcdGroup>
__device__ __forceinline__ int xcd_grouped(int bid, int n) {
  constexpr int kStretch = 8 * GROUP;
  const int base = bid / kStretch * kStretch;
  if (base + kStretch > n) return bid;
  const int r = bid - base;
  return base + (r & 7) * GROUP + (r >> 3);
}
// Tiles of a plan's list of grouped lines: `entries` consecutive list entries (with the `per` tiles of each) go to one
// compute die at a time, eight such groups to the eight dies.  Tiles of neighbouring entries share operand panels - in a
// dMoE topology the lines of an expert are neighbours - so a large group keeps a panel in one L2 instead of having
// every die fetch it; but the first group of a list sorted by length is its heaviest, and once it outweighs a die's
// fair share of the launch that die holds everything up.  The plan therefore sets `entries` per list (plan_roles_kernel:
// a quarter of a die's share of the list's blocks, at most 32).  Measured inside a forward + backward chain of
// products, where the operands come from memory: dds on the benchmark topology 267 -> 252 us with 32 entries instead
// of 4, while on the Zipf-skewed top-2 topology of BASELINE's configuration 4 groups of 16 or 32 entries cost
// 25 - 70 % (one die would get the whole of the most popular expert) and the plan picks 2 - 4 there.
__device__ __forceinline__ int xcd_item(int bid, int n, int per, int entries) {
  const int group = entries * per, stretch = 8 * group;
  const int base = bid / stretch * stretch;
  if (base + stretch > n) return bid;
  const int r = bid - base;
  return base + (r & 7) * group + (r >> 3);
}
// Tiles of a list of single lines, `per` tiles of the dense operand for each line (item = line index * per + dense
// tile); bid counts from the list's first tile and id is the workgroup's id in the whole launch (for a workgroup
// that walks several tiles: the id a launch of one workgroup per tile would give this tile).  From `stripe_from` dense tiles on (0: never; the plan's hint) and
// when they divide by the eight dies, die d takes the dense tiles [d per / 8, (d + 1) per / 8) of every line, in the
// order of the lines: it then fetches its stripe of the dense operand once, whichever lines need it.  Otherwise
// groups of neighbouring items.
__device__ __forceinline__ int xcd_lines(int bid, int id, int n, int per, int stripe_from) {
  if (stripe_from == 0 || per < stripe_from || (per & 7)) return xcd_grouped(bid, n);
  // the workgroup's die, and how many of the list's tiles the die has taken before this one
  const int first = id - bid, die = id & 7;
  const int local = (id >> 3) - ((first + 7 - die) >> 3);
  const int share = per >> 3;
  return (local / share) * per + die * share + local % share;
}
__device__ __forceinline__ int xcd_lines(int bid, int n, int per, int stripe_from) { return xcd_lines(bid, blockIdx.x, n, per, stripe_from); }
// The tiles of stk_sdd: groups of eight.  Measured against eight contiguous shares of the tile list: the same or up
// to 6 % faster (equal shares of a list are unequal shares of the work when the experts differ in size).
#ifndef STK_XCD_SDD_GROUP
#define STK_XCD_SDD_GROUP 8
#endif
__device__ __forceinline__ int xcd_tile(int bid, int n) { return xcd_grouped<STK_XCD_SDD_GROUP>(bid, n); }
// spread (wave-uniform, a hint of the plan: the lines' lengths drift along the list): groups of kXcdGroup;
// otherwise eight contiguous shares.
__device__ __forceinline__ int xcd_share(int bid, int n, bool spread) { return spread ? xcd_grouped(bid, n) : xcd_chunked(bid, n); }

}  // namespace stk
