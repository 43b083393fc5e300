// 3x3, pad 1, stride 1 NHWC convolution whose input tile stays in LDS.
//
// The generic implicit-GEMM path (gemm_kernel_dma.h, kAConv) fetches every
// input pixel once per filter tap: nine trips through the vector memory path
// for data that is used nine times.  With stride 1 and pad 1 the output has the
// input's height and width, so in the flattened (n, h, w) pixel index the nine
// taps of output pixel m are input pixels m + (r-1)*W + (s-1): the 128 output
// pixels of a tile need the contiguous run of 128 + 2W + 2 input pixels around
// them.  That run (the tile plus its halo) is loaded into LDS once; the A
// fragment of tap (r, s) is then an LDS read at a shifted pixel index.  A lane
// whose tap falls outside the image (the flat neighbour would be a pixel of the
// next row or the next image) reads a pixel of zeros kept behind the run
// instead: one select on the address per tap, none on the fragments.  Only the
// filter is streamed, one 64-channel chunk of one tap per step, through a ring
// of stages as in the GEMM kernel; it is small and comes from L2 (a deeper ring
// measured the same: four and five stages against three on 28x28x128).
//
// LDS: [filter stages of BN x 64 halfs][halo: (BM + 2W + 2) pixels x C halfs][one pixel of zeros].
// A pixel's 16-byte channel chunks are stored at chunk ^ (pixel & (C/8 - 1)),
// so the 32 consecutive pixels an MFMA fragment reads fall on distinct banks.
//
// Every wavefront owns a 64 x 64 piece of the tile (two by two MFMA tiles): with
// 64 x 32 the kernel spent its time on LDS reads, three 16-byte reads per two
// MFMAs (measured: 0.54 us per 64-channel step against 0.1 us of MFMA work).
#pragma once

#include "gemm_kernel_dma.h"

namespace cusync {
namespace gemm {

// How many 16-channel products ahead of their use the fragments are read from LDS.  Measured on the ResNet pairs
// (56x56x64 / 28x28x128 / 14x14x256, stream-ordered, us): the compiler's own order 41.0 / 51.1 / 68.3; one ahead
// 39.9 / 48.6 / 63.8; two 39.7 / 49.4 / 65.2; the whole step up front 39.9 / 52.3 / 71.6.
constexpr int kFragsAhead = 1;

template<int BM_, int BN_, int WM_, int WN_, int STAGES_, int OCC_>
struct Halo3x3Cfg {
  static constexpr int BM = BM_, BN = BN_, BK = 64, WM = WM_, WN = WN_, STAGES = STAGES_, OCC = OCC_;
  static constexpr int THREADS = kThreads;
  static constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32, KS = BK / 16;
  static constexpr int B_ROW_BYTES = BK * 2, B_CPR = B_ROW_BYTES / 16;
  static constexpr int B_STAGE = BN * B_ROW_BYTES, B_LOADS = B_STAGE / 1024 / 4;
  static constexpr int B_BYTES = STAGES * B_STAGE;
  static constexpr int LDS_BYTES = B_BYTES;        // what the epilogue may use (finishTile)
  static_assert(WM * WN == 4 && B_CPR == 8 && B_LOADS >= 1, "four wavefronts, 64-channel filter chunks");
  // Bytes of LDS a launch needs for images of width W with C channels.
  static uint32_t ldsBytes(uint32_t W, uint32_t C) {
    const uint32_t haloBytes = (BM + 2 * W + 3) * C * 2;      // the run of input pixels and one pixel of zeros behind it
    return B_BYTES + (haloBytes + 1023) / 1024 * 1024;
  }
};

// One layer: all tiles of stage p.stage that this workgroup draws.  SPLIT: the launch may cut the 9 * C/64 steps of
// a tile into p.splitK runs (grid z), each a workgroup's, whose partial sums are put together as the GEMM's k-slices
// are (finishTile); the layers whose tiles are fewer than half the CUs are run that way.  A kernel without it does
// not carry the exchange's code.
template<class C, bool SPLIT>
__device__ __forceinline__ void convHalo3x3Layer(const GemmParams& p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  __shared__ uint32_t sTicket, sLast;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / C::WN, wn = wave % C::WN;
  const uint32_t hi = lane >> 5;
  const cusync::DynStage& stage = p.stage;

  const uint32_t Cc = p.cvC, W = p.cvW, H = p.cvH;
  const uint32_t pixBytes = Cc * 2, cprMask = Cc / 8 - 1;             // C is a power of two
  const uint32_t pixShift = 31 - __builtin_clz(pixBytes);
  const uint32_t haloPix = C::BM + 2 * W + 2;
  const uint32_t haloLoads = ((haloPix + 1) * pixBytes + 1023) / 1024;       // 1 KiB pieces; pixel haloPix is the pixel of zeros
  const uint32_t zeroPixel = haloPix << pixShift;
  const uint32_t chunksPerTap = Cc / C::BK, steps = 9 * chunksPerTap;
  const uint4v rA = rawRsrc(p.A, p.M * Cc * 2);
  const uint4v rB = rawRsrc(p.B, p.N * p.ldb * 2);
  const uint32_t ldsBase = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
  const uint32_t ldsHalo = ldsBase + C::B_BYTES;
  const char* halo = smem + C::B_BYTES;

  // Filter stage: [BN rows = output channels][BK halfs], chunk c of row n at slot c ^ (n & 7).
  uint32_t bLoadRow[C::B_LOADS], bLoadChunk[C::B_LOADS];
#pragma unroll
  for (int q = 0; q < C::B_LOADS; q++) {
    const uint32_t slot = (wave * C::B_LOADS + q) * 64 + lane;
    bLoadRow[q] = slot / C::B_CPR;
    bLoadChunk[q] = (slot % C::B_CPR) ^ (bLoadRow[q] & 7);
  }
  // fragment of MFMA tile j, k-step kk: row wn*WTN + 32j + lane%32 (a multiple of 32 more does not change
  // row & 7), chunk 2kk + hi
  uint32_t bFrag[C::KS];
  {
    const uint32_t row = wn * C::WTN + (lane & 31);
#pragma unroll
    for (int kk = 0; kk < C::KS; kk++) bFrag[kk] = row * C::B_ROW_BYTES + (((2 * kk + hi) ^ (row & 7)) * 16);
  }

  const uint32_t numTiles = stage.numTiles();
  const bool consumer = stage.isConsumer();
  const uint32_t tmq = consumer ? stage.d.in.tileM : 1, tnq = consumer ? stage.d.in.tileN : 1;

  uint32_t dryXcds = 0, nextRaw = 0;
  const unsigned long long tlEntry = p.timeline ? wall_clock64() : 0;
  const uint32_t startToken = tid == 0 ? stage.beginStart() : 0;
  const bool noDraws = stage.noDraws;     // every tile is some workgroup's static first tile
  for (uint32_t round = 0;; round++) {
    if (tid == 0) sTicket = round == 0 ? stage.firstTicket(p.launched, dryXcds, noDraws) : stage.drawFinish(nextRaw, p.launched, round, dryXcds, noDraws);
    __syncthreads();
    const uint32_t ticket = sTicket;
    if (ticket >= numTiles) {
      if (tid == 0 && round == 0) stage.finishStart(startToken, p.launched);
      break;
    }
    const cusync_dim3 t = stage.ticketToTile(ticket);
    const unsigned long long tl0 = p.timeline ? wall_clock64() : 0;
    const uint32_t m0 = t.y * C::BM, n0 = t.x * C::BN;
    // this workgroup's steps of the tile: all of them, or run t.z of p.kPerSlice / 64 steps
    const uint32_t itBegin = SPLIT ? min(steps, t.z * (p.kPerSlice / C::BK)) : 0;
    const uint32_t itEnd = SPLIT ? min(steps, itBegin + p.kPerSlice / C::BK) : steps;

    // Which of the nine taps of this lane's output pixels lie inside the image: bit 3r + s.
    uint32_t tapMask[C::TM];
#pragma unroll
    for (int i = 0; i < C::TM; i++) {
      const uint32_t m = m0 + wm * C::WTM + i * 32 + (lane & 31);
      const uint32_t ow = m % W, oh = (m / W) % H;
      uint32_t bits = 0;
#pragma unroll
      for (uint32_t r = 0; r < 3; r++)
#pragma unroll
        for (uint32_t s = 0; s < 3; s++)
          if (oh + r >= 1 && oh + r <= H && ow + s >= 1 && ow + s <= W) bits |= 1u << (3 * r + s);
      tapMask[i] = m < p.M ? bits : 0;
    }

    // A consumer waits for every producer row block the halo reaches, once per producer channel tile
    // (every wave for itself: each one fetches part of the halo).
    if (consumer) {
      const uint32_t lo = m0 > W + 1 ? m0 - (W + 1) : 0, hiRow = min(m0 + C::BM + W, p.M - 1);
      if (stage.d.in.kind == CUSYNC_POLICY_ROWSYNC) {
        stage.waitWaveRows(lo, hiRow, tmq, 0, 1);
      } else {
        const uint32_t perTile = stage.d.in.kind == CUSYNC_POLICY_CONV2DTILESYNC ? 9 * tnq : tnq;
        for (uint32_t ct = 0; ct < Cc / tnq; ct++)
          stage.waitWaveRows(lo, hiRow, tmq, ct * perTile, 0);
      }
    }

    // Halo: input pixels m0 - (W+1) .. m0 + BM + W, 1 KiB per load; pixels before the first or after the
    // last image are sent out of range and arrive as zeros.
    for (uint32_t q = wave; q < haloLoads; q += 4) {
      const uint32_t byteOff = q * 1024 + lane * 16;
      const uint32_t pl = byteOff >> pixShift, slot = (byteOff & (pixBytes - 1)) >> 4;
      const uint32_t chunk = slot ^ (pl & cprMask);
      const uint32_t flat = m0 + pl - (W + 1);                       // wraps below zero for the first tile
      const bool inside = m0 + pl >= W + 1 && flat < p.M && pl < haloPix;
      loadToLds(rA, __builtin_amdgcn_readfirstlane(ldsHalo + q * 1024), inside ? (flat * Cc + chunk * 8) * 2 : kOutOfRange);
    }
    // Filter chunk `it` (tap it / chunksPerTap, channels (it % chunksPerTap) * 64 ..) into stage (it - itBegin) % STAGES.
    auto issueB = [&](uint32_t it) {
      const uint32_t lds = ldsBase + ((it - itBegin) % C::STAGES) * C::B_STAGE + wave * C::B_LOADS * 1024;
#pragma unroll
      for (int q = 0; q < C::B_LOADS; q++) {
        const bool live = it < itEnd && n0 + bLoadRow[q] < p.N;
        loadToLds(rB, __builtin_amdgcn_readfirstlane(lds + q * 1024),
                  live ? ((n0 + bLoadRow[q]) * p.ldb + it * C::BK + bLoadChunk[q] * 8) * 2 : kOutOfRange);
      }
    };
#pragma unroll
    for (uint32_t it = 0; it < C::STAGES - 1; it++) issueB(itBegin + it);
    if (tid == 0 && round == 0) stage.finishStart(startToken, p.launched);
    const unsigned long long tl1 = p.timeline ? wall_clock64() : 0;

    floatx16 acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; i++)
#pragma unroll
      for (int j = 0; j < C::TN; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    const uint32_t aPixel0 = wm * C::WTM + (lane & 31) + W + 1;       // this lane's first output pixel inside the halo
    for (uint32_t it = itBegin; it < itEnd; it++) {
      waitVmcnt<(C::STAGES - 2) * C::B_LOADS>();     // chunk `it` (and, the first time, the halo) has landed
      __builtin_amdgcn_s_barrier();                   // ... for everyone; everyone is done with chunk it-1
      asm volatile("" ::: "memory");
      issueB(it + C::STAGES - 1);
      const uint32_t tap = it / chunksPerTap, cc = it % chunksPerTap;
      const int32_t shift = ((int32_t)(tap / 3) - 1) * (int32_t)W + (int32_t)(tap % 3) - 1;
      const char* sb = smem + ((it - itBegin) % C::STAGES) * C::B_STAGE;
      uint32_t aBase[C::TM], aSwz[C::TM];
#pragma unroll
      for (int i = 0; i < C::TM; i++) {
        const uint32_t pl = (uint32_t)((int32_t)(aPixel0 + i * 32) + shift);
        aBase[i] = (tapMask[i] >> tap) & 1 ? pl << pixShift : zeroPixel;
        aSwz[i] = pl & cprMask;      // any slot of the pixel of zeros will do
      }
      // The fragments of 16 channels are requested kFragsAhead products of 16 channels before they are used.
      half8 fb[C::KS][C::TN], fa[C::KS][C::TM];
      auto readFrags = [&](int kk) {
#pragma unroll
        for (int j = 0; j < C::TN; j++) fb[kk][j] = *reinterpret_cast<const half8*>(sb + bFrag[kk] + j * 32 * C::B_ROW_BYTES);
#pragma unroll
        for (int i = 0; i < C::TM; i++) {
          const uint32_t chunk = cc * (C::BK / 8) + 2 * kk + hi;
          fa[kk][i] = *reinterpret_cast<const half8*>(halo + aBase[i] + ((chunk ^ aSwz[i]) << 4));
        }
      };
#pragma unroll
      for (int kk = 0; kk < kFragsAhead && kk < C::KS; kk++) readFrags(kk);
#pragma unroll
      for (int kk = 0; kk < C::KS; kk++) {
        __builtin_amdgcn_sched_barrier(0);      // left alone, the compiler issues each read two MFMAs before its use
        if (kk + kFragsAhead < C::KS) readFrags(kk + kFragsAhead);
#pragma unroll
        for (int i = 0; i < C::TM; i++)
#pragma unroll
          for (int j = 0; j < C::TN; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[kk][j], fa[kk][i], acc[i][j], 0, 0, 0);
      }
    }

    // The loads issued for chunks past the last one (zeros) may still be on their way into LDS, which the
    // epilogue is about to reuse.
    waitVmcnt<0>();
    const unsigned long long tl2 = p.timeline ? wall_clock64() : 0;
    if (tid == 0) nextRaw = stage.drawBegin(dryXcds, noDraws);     // settled after the epilogue
    const bool completed = finishTile<C, SPLIT>(p, acc, t, wm, wn, lane, &sLast, smem);
    cusync_dim3 done = {m0, n0, 0};
    if (completed && stage.isProducer()) stage.post(done, 1, stage.storesThrough());
    else __syncthreads();
    if (tid == 0) recordTile(p, t, round, tlEntry, tl0, tl1, tl2, p.timeline ? wall_clock64() : 0);
  }
}

template<class C, bool SPLIT = false>
__global__ __launch_bounds__(kThreads, C::OCC) void convHalo3x3Kernel(GemmParams p) {
  convHalo3x3Layer<C, SPLIT>(p);
}

// A chain of layers in ONE launch: every workgroup works through the tiles of layer 0 it can draw, then those
// of layer 1, and so on; a tile of layer l+1 waits on the semaphores of layer l exactly as it does when the
// layers are separate launches.  No wait kernel and no second launch sit between a producer and its consumer
// (on this device the first dispatch on another stream starts 15-20 us after the producer did, about as long
// as a whole 3x3 layer of the ResNet shapes takes).  Forward progress: the launch has no more workgroups than
// stay resident, and a workgroup only moves on to layer l+1 when layer l has no tile left to hand out, so every
// tile a consumer tile waits for is already in the hands of a running workgroup.
constexpr int kMaxFusedLayers = 8;
struct ConvChainParams {
  GemmParams layer[kMaxFusedLayers];
  uint32_t layers;
};

template<class C>
__global__ __launch_bounds__(kThreads, C::OCC) void convHalo3x3ChainKernel(ConvChainParams cp) {
  for (uint32_t l = 0; l < cp.layers; l++) {
    convHalo3x3Layer<C, false>(cp.layer[l]);
    __syncthreads();        // everyone has read the last ticket of this layer before the next one's is written
  }
}

}  // namespace gemm
}  // namespace cusync
