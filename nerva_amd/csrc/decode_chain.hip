// Persistent layer-chain kernel (see decode_chain.cuh).
//
// Roles inside a workgroup (one workgroup per CU, 256 in all):
//   * eight streaming waves. Each owns a fixed slice of the rows of every phase and walks one
//     flat list of 4 KiB weight batches that spans all phases of the launch, four batches in
//     flight in four register buffers (refilled as they are consumed, fully unrolled). The list
//     does not stop at a phase boundary: while a barrier is pending the wave already holds the
//     first batches of the next phase.
//   * one activation wave. It never requests weights, so its memory operations are not queued
//     behind a weight stream: it turns the workgroup's row results into the phase output
//     (bias, residual, rounding), publishes them with device-coherent stores, signals arrival
//     and waits for all 256 workgroups.
// Workgroup barriers connect the roles in every phase: B1 (the grid barrier has been passed),
// then the streaming waves stage the phase's input vector into LDS together (RMSNorm included;
// their own earlier weight requests have long landed by then), B2 (input vector ready), the
// rows, and A (row results ready). The grid barrier is a flag array: every workgroup writes its
// own 64-byte-spaced flag and reads everybody's; no read-modify-write, no cache flush. Flags
// hold monotonically growing epochs derived from the sequence position, so they are never
// reset inside a step.
// Every wait is bounded: when it runs out the kernel raises abort_flag and every workgroup exits.
#include "decode_chain.cuh"

#include "gemv_stream.cuh"

namespace nv {

namespace {

constexpr uint32_t kChainWaveCount = kChainGrid * kChainWaves;  // streaming waves in the grid
constexpr uint32_t kRing = 4;                                   // 4 KiB weight batches in flight per wave
constexpr uint32_t kSpinLimit = 1u << 20;                       // polls before a wait gives up
constexpr uint32_t kMaxRowsPerCu = 64;                          // one activation-wave lane per row
constexpr uint32_t kChainLdsBytes = 96u * 1024u;                // > half a CU's LDS: one workgroup per CU

enum : int { kPhO = 0, kPhGateUp = 1, kPhDown = 2, kPhQkv = 3 };

struct Phase {
  const uint16_t *w;
  uint32_t units;  // output rows (gate/up: pairs)
  uint32_t cols;
  uint32_t rpw;    // rows per streaming wave
  uint32_t bpr;    // 4 KiB batches per row (pair)
};

__device__ __forceinline__ Phase phase_of(const ChainParams &p, int ph) {
  Phase f;
  if (ph == kPhO) {
    f.w = p.wo;
    f.units = p.hidden;
    f.cols = p.attn_dim;
  } else if (ph == kPhGateUp) {
    f.w = p.wgu;
    f.units = p.inter;
    f.cols = p.hidden;
  } else if (ph == kPhDown) {
    f.w = p.wdown;
    f.units = p.hidden;
    f.cols = p.inter;
  } else {
    f.w = p.wqkv_next;
    f.units = p.qkv_rows;
    f.cols = p.hidden;
  }
  f.rpw = (f.units + kChainWaveCount - 1) / kChainWaveCount;
  f.bpr = ph == kPhGateUp ? f.cols / 1024u : f.cols / 2048u;
  return f;
}
#ifndef NV_CHAIN_INTERLEAVE
#define NV_CHAIN_INTERLEAVE 1
#endif
// Row i of streaming wave gw (grid-wide index). Interleaved: consecutive waves stream consecutive
// rows, so at any moment the 2048 waves cover one contiguous 16 MiB window of the matrix.
constexpr bool kInterleave = NV_CHAIN_INTERLEAVE != 0;
__device__ __forceinline__ uint32_t wave_nrows(const Phase &f, uint32_t gw) {
  if (kInterleave) return gw >= f.units ? 0u : (f.units - gw + kChainWaveCount - 1) / kChainWaveCount;
  const uint32_t first = gw * f.rpw;
  return first >= f.units ? 0u : min(f.rpw, f.units - first);
}
__device__ __forceinline__ uint32_t wave_row(const Phase &f, uint32_t gw, uint32_t i) {
  return kInterleave ? gw + i * kChainWaveCount : gw * f.rpw + i;
}

// Device-scope coherent accesses (written through / read around the XCD-local L2).
__device__ __forceinline__ void st_coherent(float *ptr, float v) {
  __hip_atomic_store(ptr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_coherent(uint16_t *ptr, uint16_t v) {
  __hip_atomic_store(ptr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_coherent(uint32_t *ptr, uint32_t v) {
  __hip_atomic_store(ptr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_coherent(const float *ptr) {
  return __hip_atomic_load(ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_coherent(const uint32_t *ptr) {
  return __hip_atomic_load(ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t ld_coherent(const uint64_t *ptr) {
  return __hip_atomic_load(ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void wait_own_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Activation wave: waits until every workgroup's flag has reached `epoch`.
__device__ __forceinline__ bool wait_all_arrived(const ChainParams &p, uint32_t epoch, int lane) {
  uint32_t spins = 0;
  for (;;) {
    bool mine = true;
#pragma unroll
    for (uint32_t j = 0; j < kChainGrid / kWave; ++j)
      mine = mine && ld_coherent(p.flags + (j * kWave + lane) * kChainFlagStride) >= epoch;
    const bool stop = ld_coherent(p.abort_flag) != 0u;  // raised by another workgroup, or by the host
    if (!stop && __all(mine)) return true;
    if (stop || ++spins > kSpinLimit) {
      if (lane == 0) st_coherent(p.abort_flag, 1u);
      return false;
    }
  }
}

constexpr int kStreamThreads = kChainWaves * kWave;  // the streaming waves stage the input vector together

// Streaming waves: 16-bit vector (device-coherent source) -> LDS. count % 2048 == 0, so every
// thread copies the same number of 8-byte pieces.
__device__ __forceinline__ void stage_x16(const uint16_t *src, uint32_t count, uint16_t *xs) {
  const uint64_t *s8 = reinterpret_cast<const uint64_t *>(src);
  uint64_t *d8 = reinterpret_cast<uint64_t *>(xs);
  const uint32_t per_thread = count / (4 * kStreamThreads);  // 1 .. 6
  uint32_t tid = threadIdx.x;
  asm volatile("" : "+v"(tid));  // addresses are formed here, per phase, not kept live across phases
  uint64_t v[6];
#pragma unroll
  for (int j = 0; j < 6; ++j)
    if (static_cast<uint32_t>(j) < per_thread) v[j] = ld_coherent(s8 + tid + j * kStreamThreads);
#pragma unroll
  for (int j = 0; j < 6; ++j)
    if (static_cast<uint32_t>(j) < per_thread) d8[tid + j * kStreamThreads] = v[j];
}

// Streaming waves: x = round16(v * rsqrt(mean(v^2) + eps) * gamma) of an f32 vector -> LDS.
// count % 2048 == 0 and count <= 4096: a thread holds 2 or 4 pairs. Contains one workgroup
// barrier (the activation wave takes part in it).
template <uint32_t DT>
__device__ __forceinline__ void stage_rmsnorm(const float *src, const uint16_t *gamma, uint32_t count, float eps,
                                              uint16_t *xs, float *red, int lane, int wave) {
  const uint64_t *s8 = reinterpret_cast<const uint64_t *>(src);
  const uint32_t *g4 = reinterpret_cast<const uint32_t *>(gamma);
  uint32_t *d4 = reinterpret_cast<uint32_t *>(xs);
  const uint32_t per_thread = count / (2 * kStreamThreads);  // 2 or 4
  uint32_t tid = threadIdx.x;
  asm volatile("" : "+v"(tid));  // addresses are formed here, per phase, not kept live across phases
  float va[4], vb[4];
  uint32_t gw[4];
  float ss = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const bool on = static_cast<uint32_t>(j) < per_thread;
    const uint64_t raw = on ? ld_coherent(s8 + tid + j * kStreamThreads) : 0ull;
    gw[j] = on ? g4[tid + j * kStreamThreads] : 0u;
    va[j] = __uint_as_float(static_cast<uint32_t>(raw));
    vb[j] = __uint_as_float(static_cast<uint32_t>(raw >> 32));
    ss += va[j] * va[j] + vb[j] * vb[j];
  }
  ss = wave_sum(ss);
  if (lane == 0) red[wave] = ss;
  __syncthreads();
  float total = 0.0f;
#pragma unroll
  for (int w = 0; w < kChainWaves; ++w) total += red[w];
  const float scale = 1.0f / sqrtf(total / static_cast<float>(count) + eps);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float g0, g1;
    unpack2<DT>(gw[j], g0, g1);
    if (static_cast<uint32_t>(j) < per_thread)
      d4[tid + j * kStreamThreads] =
          enc16<DT>(va[j] * scale * g0) | (static_cast<uint32_t>(enc16<DT>(vb[j] * scale * g1)) << 16);
  }
}

template <uint32_t DT>
__global__ __launch_bounds__(kChainThreads) void decode_chain_kernel(ChainParams p) {
  extern __shared__ __align__(16) uint16_t xs[];  // input vector of the current phase, 16-bit
  __shared__ float res[kMaxRowsPerCu];             // this workgroup's row results of the current phase
  __shared__ float red[kChainWaves];
  __shared__ uint32_t lds_abort;

  const uint32_t pos = *p.cursor;
  if (pos >= p.max_steps) return;  // same decision in every workgroup
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // uniform: keep it scalar
  const int nph = p.wqkv_next != nullptr ? 4 : 3;
  if (threadIdx.x == 0) lds_abort = 0u;

  if (wave == kChainWaves) {
    // ------------------------------------------------------------ activation wave
#pragma unroll 1
    for (int ph = 0; ph < nph; ++ph) {
      const Phase f = phase_of(p, ph);
      if (ph > 0) {
        const uint32_t epoch = pos * p.barriers_per_step + p.barrier_base + static_cast<uint32_t>(ph);
        if (!wait_all_arrived(p, epoch, lane) && lane == 0) lds_abort = 1u;
      }
      if (p.trace != nullptr && blockIdx.x == 0 && lane == 0) p.trace[ph * 4 + 0] = wall_clock64();
      __syncthreads();  // B1: the grid barrier has been passed (or given up)
      if (lds_abort != 0u) return;
      if (ph == kPhGateUp || ph == kPhQkv) __syncthreads();  // the RMSNorm staging's own barrier
      __syncthreads();  // B2: the streaming waves have staged the input vector
      if (p.trace != nullptr && blockIdx.x == 0 && lane == 0) p.trace[ph * 4 + 1] = wall_clock64();
      // operands of this phase's epilogue, requested while the rows are being computed
      // lane = (streaming wave, its i-th row): the slot the wave wrote in res[]
      const uint32_t lw = static_cast<uint32_t>(lane) / f.rpw, li = static_cast<uint32_t>(lane) % f.rpw;
      const uint32_t row = wave_row(f, blockIdx.x * kChainWaves + lw, li);
      const bool live = lw < static_cast<uint32_t>(kChainWaves) && row < f.units;
      float resid = 0.0f, bias = 0.0f;
      if (live && ph == kPhO) {
        resid = ld_coherent(p.x + row);
        if (p.o_bias != nullptr) bias = dec16<DT>(p.o_bias[row]);
      } else if (live && ph == kPhDown) {
        resid = ld_coherent(p.r + row);
      }
      __syncthreads();  // A
      if (p.trace != nullptr && blockIdx.x == 0 && lane == 0) p.trace[ph * 4 + 2] = wall_clock64();
      float y = live ? res[lane] : 0.0f;
      if (ph == kPhGateUp) {
        if (live) st_coherent(p.ff16 + row, enc16<DT>(y));
      } else if (live) {
        if (ph == kPhO) {
          y += bias;
          y += resid;
          st_coherent(p.r + row, y);
        } else if (ph == kPhDown) {
          y += resid;
          if (p.round_out) y = round16<DT>(y);
          st_coherent(p.x + row, y);
        } else {
          st_coherent(p.qkv + row, y);
        }
      }
      if (ph + 1 < nph) {
        wait_own_stores();
        if (lane == 0)
          st_coherent(p.flags + blockIdx.x * kChainFlagStride,
                      pos * p.barriers_per_step + p.barrier_base + static_cast<uint32_t>(ph) + 1u);
      }
      if (p.trace != nullptr && blockIdx.x == 0 && lane == 0) p.trace[ph * 4 + 3] = wall_clock64();
    }
    return;
  }

  // -------------------------------------------------------------- streaming waves
  // The wave's work is a list of 4 KiB weight batches: phase after phase, row after row. Each
  // phase's share is padded to a multiple of kRing, so that a phase always starts in register
  // buffer `a`: the steps below are straight-line code with fixed buffers, which lets the
  // compiler count outstanding requests exactly (the pad positions request and consume nothing).
  // The request side runs kRing positions ahead of the consuming side and does not stop at a
  // phase boundary.
  const uint32_t gw = blockIdx.x * kChainWaves + wave;  // `wave` is uniform: held in a scalar register
  const bool tracer = p.trace != nullptr && blockIdx.x == 0 && threadIdx.x == 0;
  if (tracer) p.trace[16] = wall_clock64();

  // request side: phase, position inside the padded phase, row and batch inside the row
  int ip = 0;
  Phase fi = phase_of(p, 0);
  uint32_t inb = wave_nrows(fi, gw) * fi.bpr;           // real batches of the phase
  uint32_t inbp = (inb + kRing - 1) / kRing * kRing;    // padded
  uint32_t iq = 0, ii = 0, ib = 0;
  const uint16_t *wp0 = nullptr, *wp1 = nullptr;
  // The weight requests are asynchronous loads issued by hand, and each batch is awaited with an
  // explicit outstanding-request count just before its use: the compiler's own bookkeeping
  // treats every conditional request as possibly outstanding and would wait for the whole ring
  // at every batch. Requests return in issue order, so "at most 4 * n outstanding" means the
  // batch is complete once n newer batches have been requested; requests the compiler issues in
  // between (input staging) only make that wait stricter. `hist` remembers which of the last
  // positions really requested something (pads do not).
  u32x4_t a0, a1, a2, a3, b0, b1, b2, b3, c0, c1, c2, c3, d0, d1, d2, d3;
  uint32_t hist = 0;
#define NV_CH_LOAD4(B, P0, P1, ONE_ROW)                                                              \
  do {                                                                                               \
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(B##0) : "v"(P0) : "memory");            \
    asm volatile("global_load_dwordx4 %0, %1, off offset:1024 nt" : "=v"(B##1) : "v"(P0) : "memory"); \
    if (ONE_ROW) {                                                                                   \
      asm volatile("global_load_dwordx4 %0, %1, off offset:2048 nt" : "=v"(B##2) : "v"(P0) : "memory"); \
      asm volatile("global_load_dwordx4 %0, %1, off offset:3072 nt" : "=v"(B##3) : "v"(P0) : "memory"); \
    } else {                                                                                         \
      asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(B##2) : "v"(P1) : "memory");          \
      asm volatile("global_load_dwordx4 %0, %1, off offset:1024 nt" : "=v"(B##3) : "v"(P1) : "memory"); \
    }                                                                                                \
  } while (0)
#define NV_CH_AWAIT(B, NEWER)                                                                              \
  do {                                                                                                     \
    switch (NEWER) {                                                                                       \
      case 0u: asm volatile("s_waitcnt vmcnt(0)" : "+v"(B##0), "+v"(B##1), "+v"(B##2), "+v"(B##3)); break;  \
      case 1u: asm volatile("s_waitcnt vmcnt(4)" : "+v"(B##0), "+v"(B##1), "+v"(B##2), "+v"(B##3)); break;  \
      case 2u: asm volatile("s_waitcnt vmcnt(8)" : "+v"(B##0), "+v"(B##1), "+v"(B##2), "+v"(B##3)); break;  \
      default: asm volatile("s_waitcnt vmcnt(12)" : "+v"(B##0), "+v"(B##1), "+v"(B##2), "+v"(B##3)); break; \
    }                                                                                                      \
  } while (0)
#define NV_CH_U4(V) make_uint4((V).x, (V).y, (V).z, (V).w)
#define NV_CH_ISSUE(B)                                                                      \
  do {                                                                                      \
    uint32_t requested_ = 0u;                                                               \
    if (ip < nph) {                                                                         \
      if (iq < inb) {                                                                       \
        if (ib == 0u) {                                                                     \
          const uint64_t row_ = wave_row(fi, gw, ii);                                       \
          wp0 = fi.w + row_ * fi.cols + lane * 8;                                           \
          wp1 = fi.w + (row_ + fi.units) * fi.cols + lane * 8;                              \
        }                                                                                   \
        if (ip == kPhGateUp) {                                                              \
          const uint16_t *q0_ = wp0 + ib * 1024u, *q1_ = wp1 + ib * 1024u;                  \
          NV_CH_LOAD4(B, q0_, q1_, false); /* two chunks of the gate row, two of the up row */ \
        } else {                                                                            \
          const uint16_t *q0_ = wp0 + ib * 2048u;                                           \
          NV_CH_LOAD4(B, q0_, q0_, true); /* four consecutive chunks of one row */          \
        }                                                                                   \
        requested_ = 1u;                                                                    \
        if (++ib == fi.bpr) {                                                               \
          ib = 0u;                                                                          \
          ++ii;                                                                             \
        }                                                                                   \
      }                                                                                     \
      if (++iq == inbp) {                                                                   \
        iq = 0u;                                                                            \
        ii = 0u;                                                                            \
        ++ip;                                                                               \
        if (ip < nph) {                                                                     \
          fi = phase_of(p, ip);                                                             \
          inb = wave_nrows(fi, gw) * fi.bpr;                                                \
          inbp = (inb + kRing - 1) / kRing * kRing;                                         \
        }                                                                                   \
      }                                                                                     \
    }                                                                                       \
    hist = (hist << 1) | requested_;                                                        \
  } while (0)
  // consuming side: one position of the padded phase
#define NV_CH_STEP(B)                                                                       \
  do {                                                                                      \
    if (cq < nb) {                                                                          \
      /* the three positions requested after this one: how many of them were real */       \
      const uint32_t newer_ = static_cast<uint32_t>(__builtin_popcount(hist & 7u));         \
      NV_CH_AWAIT(B, newer_);                                                               \
      if (ph == kPhGateUp) {                                                                \
        const uint32_t col_ = cb * 1024u + lane * 8;                                        \
        const uint4 x0_ = *reinterpret_cast<const uint4 *>(xs + col_);                      \
        const uint4 x1_ = *reinterpret_cast<const uint4 *>(xs + col_ + 512u);               \
        acc0 = dot8<DT, false>(NV_CH_U4(B##0), x0_, acc0);                                            \
        acc1 = dot8<DT, false>(NV_CH_U4(B##2), x0_, acc1);                                            \
        acc0 = dot8<DT, false>(NV_CH_U4(B##1), x1_, acc0);                                            \
        acc1 = dot8<DT, false>(NV_CH_U4(B##3), x1_, acc1);                                            \
      } else {                                                                              \
        const uint32_t col_ = cb * 2048u + lane * 8;                                        \
        acc0 = dot8<DT, false>(NV_CH_U4(B##0), *reinterpret_cast<const uint4 *>(xs + col_), acc0);    \
        acc0 = dot8<DT, false>(NV_CH_U4(B##1), *reinterpret_cast<const uint4 *>(xs + col_ + 512u), acc0);   \
        acc0 = dot8<DT, false>(NV_CH_U4(B##2), *reinterpret_cast<const uint4 *>(xs + col_ + 1024u), acc0);  \
        acc0 = dot8<DT, false>(NV_CH_U4(B##3), *reinterpret_cast<const uint4 *>(xs + col_ + 1536u), acc0);  \
      }                                                                                     \
      if (++cb == f.bpr) {                                                                  \
        cb = 0u;                                                                            \
        acc0 = wave_sum(acc0);                                                              \
        if (ph == kPhGateUp) acc1 = wave_sum(acc1);                                         \
        if (lane == 0) res[wave * f.rpw + ci] = ph == kPhGateUp ? silu(acc0) * acc1 : acc0; \
        acc0 = 0.0f;                                                                        \
        acc1 = 0.0f;                                                                        \
        ++ci;                                                                               \
      }                                                                                     \
    }                                                                                       \
    ++cq;                                                                                   \
    NV_CH_ISSUE(B); /* the position kRing ahead, possibly in the next phase */              \
  } while (0)

  // The first phase's input (the attention output) is ready when the kernel starts: request it
  // before the weights, so that it returns first instead of queueing behind 16 KiB of them.
  const uint32_t x0_pieces = p.attn_dim / (4 * kStreamThreads);
  uint64_t x0[6];
#pragma unroll
  for (int j = 0; j < 6; ++j)
    if (static_cast<uint32_t>(j) < x0_pieces)
      x0[j] = ld_coherent(reinterpret_cast<const uint64_t *>(p.attn16) + threadIdx.x + j * kStreamThreads);
  if (tracer) p.trace[17] = wall_clock64();
  NV_CH_ISSUE(a);
  NV_CH_ISSUE(b);
  NV_CH_ISSUE(c);
  NV_CH_ISSUE(d);
  if (tracer) p.trace[18] = wall_clock64();

#pragma unroll 1
  for (int ph = 0; ph < nph; ++ph) {
    const Phase f = phase_of(p, ph);
    const uint32_t nb = wave_nrows(f, gw) * f.bpr;
    const uint32_t nbp = (nb + kRing - 1) / kRing * kRing;
    __syncthreads();  // B1: every workgroup has published the previous phase
    if (lds_abort != 0u) return;
    if (tracer && ph == 0) p.trace[19] = wall_clock64();
    if (ph == kPhO) {
#pragma unroll
      for (int j = 0; j < 6; ++j)
        if (static_cast<uint32_t>(j) < x0_pieces)
          reinterpret_cast<uint64_t *>(xs)[threadIdx.x + j * kStreamThreads] = x0[j];
    } else if (ph == kPhGateUp) {
      stage_rmsnorm<DT>(p.r, p.rms_mlp, p.hidden, p.eps, xs, red, lane, wave);
    } else if (ph == kPhDown) {
      stage_x16(p.ff16, p.inter, xs);
    } else {
      stage_rmsnorm<DT>(p.x, p.rms_next, p.hidden, p.eps, xs, red, lane, wave);
    }
    if (tracer && ph == 0) p.trace[20] = wall_clock64();
    __syncthreads();  // B2: the input vector of this phase is in LDS
    if (tracer && ph == 0) p.trace[21] = wall_clock64();
    uint32_t cq = 0, ci = 0, cb = 0;
    float acc0 = 0.0f, acc1 = 0.0f;
    for (uint32_t g = 0; g < nbp; g += kRing) {
      NV_CH_STEP(a);
      NV_CH_STEP(b);
      NV_CH_STEP(c);
      NV_CH_STEP(d);
    }
    __syncthreads();  // A: this workgroup's rows of the phase are in res[]
  }
#undef NV_CH_ISSUE
#undef NV_CH_STEP
#undef NV_CH_LOAD4
#undef NV_CH_AWAIT
#undef NV_CH_U4
}

bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

namespace {
bool chain_shapes_ok(uint32_t hidden, uint32_t attn_dim, uint32_t inter, uint32_t qkv_rows) {
  const uint32_t max_units = kChainWaveCount * (kMaxRowsPerCu / kChainWaves);  // rows per phase
  if (hidden == 0 || hidden % 2048u != 0 || hidden > 4096u) return false;     // RMSNorm held in 64 lanes
  if (attn_dim == 0 || attn_dim % 2048u != 0 || attn_dim > 12288u) return false;
  if (inter == 0 || inter % 2048u != 0 || inter > 12288u) return false;
  return qkv_rows != 0 && qkv_rows <= max_units && inter <= max_units;
}
}  // namespace

bool chain_supported(uint32_t hidden, uint32_t attn_dim, uint32_t inter, uint32_t qkv_rows) {
  if (!chain_shapes_ok(hidden, attn_dim, inter, qkv_rows)) return false;
  int device = 0, cus = 0;
  if (hipGetDevice(&device) != hipSuccess) return false;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return false;
  return cus >= static_cast<int>(kChainGrid);  // every workgroup must be resident at once
}

hipError_t launch_decode_chain(uint32_t dtype, const ChainParams &p, hipStream_t stream) {
  if (!chain_shapes_ok(p.hidden, p.attn_dim, p.inter, p.qkv_rows == 0 ? 1u : p.qkv_rows)) return hipErrorInvalidValue;
  if (p.wo == nullptr || p.rms_mlp == nullptr || p.wgu == nullptr || p.wdown == nullptr || p.attn16 == nullptr ||
      p.x == nullptr || p.r == nullptr || p.ff16 == nullptr || p.flags == nullptr || p.abort_flag == nullptr ||
      p.cursor == nullptr)
    return hipErrorInvalidValue;
  if (p.wqkv_next != nullptr && (p.rms_next == nullptr || p.qkv == nullptr || p.qkv_rows == 0)) return hipErrorInvalidValue;
  if (!aligned16(p.wo) || !aligned16(p.wgu) || !aligned16(p.wdown) || !aligned16(p.wqkv_next) || !aligned16(p.attn16) ||
      !aligned16(p.x) || !aligned16(p.r) || !aligned16(p.ff16) || !aligned16(p.rms_mlp) || !aligned16(p.rms_next))
    return hipErrorInvalidValue;
  if (p.barriers_per_step == 0 || p.barrier_base + kChainMaxBarriers > p.barriers_per_step) return hipErrorInvalidValue;
  if (dtype == kBF16)
    hipLaunchKernelGGL((decode_chain_kernel<kBF16>), dim3(kChainGrid), dim3(kChainThreads), kChainLdsBytes, stream, p);
  else if (dtype == kF16)
    hipLaunchKernelGGL((decode_chain_kernel<kF16>), dim3(kChainGrid), dim3(kChainThreads), kChainLdsBytes, stream, p);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t chain_prepare(uint32_t dtype) {
  if (dtype == kBF16)
    return hipFuncSetAttribute(reinterpret_cast<const void *>(&decode_chain_kernel<kBF16>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, kChainLdsBytes);
  if (dtype == kF16)
    return hipFuncSetAttribute(reinterpret_cast<const void *>(&decode_chain_kernel<kF16>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, kChainLdsBytes);
  return hipErrorInvalidValue;
}

}  // namespace nv
