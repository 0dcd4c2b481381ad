// Fused layer front (see layer_front.cuh): qkv rows -> attention splits -> o rows in one launch.
//
// Workgroup roles, by index:
//   [0, q_wgs)            qkv role: 32 rows of the fused q|k|v matrix, four per wave (two in
//                         flight, refilled once). The rows of one workgroup belong to one kv head
//                         (its G query heads, its key row block or its value row block), so an
//                         attention workgroup waits for the (G + 2) * 4 row flags of its own kv
//                         head only.
//   [q_wgs, q_wgs+a_wgs)  attention role: (kv head, split), the matrix-core kernel body of
//                         attn_tile.cuh. Its first KV tiles are requested before it waits.
//   the rest              o role: 16 rows of the o projection, two per wave, the whole rows held
//                         in registers before the wait; after the kv-head flags are up it turns
//                         the f32 attention output into the 16-bit GEMV input in LDS.
// A GEMV wave requests two complete rows (at most 2 x 8 KiB) at once: with every workgroup of
// the o role resident, that role's entire weight matrix is in flight or in registers before
// the attention output exists.
#include "layer_front.cuh"

#include "attn_tile.cuh"
#include "gemv_stream.cuh"

namespace nv {

namespace {

using namespace attn;

constexpr int kFW = kFrontThreads / kWave;   // 8 waves
constexpr int kMaxChunks = 8;                // 16-byte chunks per lane per row: cols <= 4096
constexpr uint32_t kChunkCols = kWave * 8;   // columns one wave covers with one load instruction
constexpr int kQRowsPerWave = 4;             // qkv role: two rows in flight, then two more
constexpr uint32_t kFrontQRowsPerWg = kFW * kQRowsPerWave;

struct GemvShared {
  alignas(16) uint16_t xs[kMaxChunks * kChunkCols];  // 16-bit input vector
  float red[kFW];
};

// Requests row `row` of W[.][cols] (cols = nchunk * 512) into registers: 16 bytes per lane and chunk.
__device__ __forceinline__ void request_row(const uint16_t *w, uint32_t row, uint32_t cols, uint32_t nchunk, int lane,
                                            uint4 (&buf)[kMaxChunks]) {
  const uint16_t *wp = w + static_cast<uint64_t>(row) * cols + lane * 8;
#pragma unroll
  for (int u = 0; u < kMaxChunks; ++u) {
    buf[u] = make_uint4(0u, 0u, 0u, 0u);
    if (static_cast<uint32_t>(u) < nchunk) buf[u] = load_stream(wp + u * kChunkCols);
  }
}

// The row against the 16-bit vector in LDS; every lane returns the full sum.
template <uint32_t DT>
__device__ __forceinline__ float dot_row(const uint4 (&buf)[kMaxChunks], const uint16_t *xs, uint32_t nchunk, int lane) {
  float a = 0.0f;
#pragma unroll
  for (int u = 0; u < kMaxChunks; ++u) {
    if (static_cast<uint32_t>(u) < nchunk) {
      const uint4 xv = *reinterpret_cast<const uint4 *>(xs + u * kChunkCols + lane * 8);
      a = dot8<DT, false>(buf[u], xv, a);
    }
  }
  return wave_sum(a);
}

// qkv role of workgroup `wg`.
template <uint32_t DT, int G>
__device__ __forceinline__ void front_q_role(const FrontParams &p, uint32_t wg, uint32_t epoch, GemvShared &sh) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint32_t cols = p.hidden, nchunk = cols / kChunkCols;
  const uint32_t A = p.attn.heads * kHD, KV = p.attn.kv_heads * kHD;
  constexpr uint32_t kBlocksPerHead = kHD / kFrontQRowsPerWg;         // 4 workgroups per 128 rows
  constexpr uint32_t kWgsPerKvHead = (G + 2) * kBlocksPerHead;
  const uint32_t h = wg / kWgsPerKvHead, j = wg % kWgsPerKvHead;
  uint32_t base;
  if (j < G * kBlocksPerHead) base = h * G * kHD + j * kFrontQRowsPerWg;
  else if (j < (G + 1) * kBlocksPerHead) base = A + h * kHD + (j - G * kBlocksPerHead) * kFrontQRowsPerWg;
  else base = A + KV + h * kHD + (j - (G + 1) * kBlocksPerHead) * kFrontQRowsPerWg;
  const uint32_t row0 = base + wave * kQRowsPerWave;
  uint64_t *tr = wg == 0 ? p.trace : nullptr;
  link_mark(tr, 0);

  // the layer input first (cache hits), then the two rows
  const uint32_t c = threadIdx.x * 8;
  float4 xa = make_float4(0.f, 0.f, 0.f, 0.f), xb = xa;
  uint4 gw = make_uint4(0u, 0u, 0u, 0u);
  if (c < cols) {
    xa = *reinterpret_cast<const float4 *>(p.x + c);
    xb = *reinterpret_cast<const float4 *>(p.x + c + 4);
    gw = *reinterpret_cast<const uint4 *>(p.rms_attn + c);
  }
  uint4 w0[kMaxChunks], w1[kMaxChunks];  // two rows in flight, refilled as they are consumed
  request_row(p.wqkv, row0, cols, nchunk, lane, w0);
  request_row(p.wqkv, row0 + 1, cols, nchunk, lane, w1);

  // RMSNorm -> 16 bit -> LDS (hidden under the first HBM round trip)
  float ss = xa.x * xa.x + xa.y * xa.y + xa.z * xa.z + xa.w * xa.w + xb.x * xb.x + xb.y * xb.y + xb.z * xb.z +
             xb.w * xb.w;
  ss = wave_sum(ss);
  if (lane == 0) sh.red[wave] = ss;
  __syncthreads();
  float total = 0.0f;
#pragma unroll
  for (int w = 0; w < kFW; ++w) total += sh.red[w];
  const float scale = 1.0f / sqrtf(total / static_cast<float>(cols) + p.rms_eps);
  if (c < cols) {
    float g0, g1, g2, g3, g4, g5, g6, g7;
    unpack2<DT>(gw.x, g0, g1);
    unpack2<DT>(gw.y, g2, g3);
    unpack2<DT>(gw.z, g4, g5);
    unpack2<DT>(gw.w, g6, g7);
    uint4 o;
    o.x = enc16<DT>(xa.x * scale * g0) | (static_cast<uint32_t>(enc16<DT>(xa.y * scale * g1)) << 16);
    o.y = enc16<DT>(xa.z * scale * g2) | (static_cast<uint32_t>(enc16<DT>(xa.w * scale * g3)) << 16);
    o.z = enc16<DT>(xb.x * scale * g4) | (static_cast<uint32_t>(enc16<DT>(xb.y * scale * g5)) << 16);
    o.w = enc16<DT>(xb.z * scale * g6) | (static_cast<uint32_t>(enc16<DT>(xb.w * scale * g7)) << 16);
    *reinterpret_cast<uint4 *>(sh.xs + c) = o;
  }
  __syncthreads();
  link_mark(tr, 1);

#pragma unroll
  for (int r = 0; r < kQRowsPerWave; r += 2) {
    const float y0 = dot_row<DT>(w0, sh.xs, nchunk, lane);
    if (r + 2 < kQRowsPerWave) request_row(p.wqkv, row0 + r + 2, cols, nchunk, lane, w0);
    const float y1 = dot_row<DT>(w1, sh.xs, nchunk, lane);
    if (r + 3 < kQRowsPerWave) request_row(p.wqkv, row0 + r + 3, cols, nchunk, lane, w1);
    if (lane == 0) {
      store_tagged(p.qkv_tagged + row0 + r, y0, epoch);
      store_tagged(p.qkv_tagged + row0 + r + 1, y1, epoch);
    }
    if (r == 0) link_mark(tr, 2);
  }
  link_mark(tr, 3);
  if (p.trace != nullptr && wg + 1 == gridDim.x - p.attn.kv_heads * p.attn.splits - p.hidden / kFrontRowsPerWg)
    link_mark(p.trace, 4);
}

// o role of its `wg`-th workgroup.
template <uint32_t DT>
__device__ __forceinline__ void front_o_role(const FrontParams &p, uint32_t wg, uint32_t epoch, GemvShared &sh) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint32_t cols = p.attn.heads * kHD, nchunk = cols / kChunkCols;
  const uint32_t row0 = wg * kFrontRowsPerWg + wave * 2;
  const bool last_wg = wg + 1 == p.hidden / kFrontRowsPerWg;
  uint64_t *tr = p.trace == nullptr ? nullptr : (wg == 0 ? p.trace + 20 : (last_wg ? p.trace + 24 : nullptr));
  link_mark(tr, 0);

  uint4 w0[kMaxChunks], w1[kMaxChunks];
  request_row(p.wo, row0, cols, nchunk, lane, w0);
  request_row(p.wo, row0 + 1, cols, nchunk, lane, w1);
  float res0 = 0.0f, res1 = 0.0f, bias0 = 0.0f, bias1 = 0.0f;  // residual and bias of the two rows
  if (lane == 0) {
    res0 = p.x[row0];
    res1 = p.x[row0 + 1];
    if (p.o_bias != nullptr) {
      bias0 = dec16<DT>(p.o_bias[row0]);
      bias1 = dec16<DT>(p.o_bias[row0 + 1]);
    }
  }

  // ---- a light wait first: one wave polls this workgroup's own hint words, one per kv head (the
  // output itself is 16 KiB, too much for 256 workgroups to poll all along)
  if (wave == 0) {
    uint32_t spins = 0;
    for (;;) {
      const bool mine = static_cast<uint32_t>(lane) >= p.attn.kv_heads ||
                        load_coherent(p.head_hints + wg * kFrontFlagStride + lane) == epoch;
      if (__all(mine)) break;
      if (link_give_up(p.abort_flag, spins)) break;
    }
  }
  __syncthreads();
  link_mark(tr, 1);

  // ---- attention output: (two 16-bit values, epoch) words -> LDS; polled until every word is current
  const uint32_t c = threadIdx.x * 8;
  if (c < cols) {
    uint64_t v[4];
    uint32_t spins = 0;
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[i] = load_tagged(p.out_tagged + c / 2 + i);
        ok = ok && tag_is(v[i], epoch);
      }
      if (__all(ok)) break;
      if (link_give_up(p.abort_flag, spins)) break;
      __builtin_amdgcn_s_sleep(8);
    }
    *reinterpret_cast<uint4 *>(sh.xs + c) = make_uint4(static_cast<uint32_t>(v[0]), static_cast<uint32_t>(v[1]),
                                                       static_cast<uint32_t>(v[2]), static_cast<uint32_t>(v[3]));
  }
  __syncthreads();
  link_mark(tr, 2);

  const float y0 = dot_row<DT>(w0, sh.xs, nchunk, lane), y1 = dot_row<DT>(w1, sh.xs, nchunk, lane);
  if (lane == 0) {
    p.r[row0] = (y0 + bias0) + res0;   // same order as the stand-alone GEMV epilogue
    p.r[row0 + 1] = (y1 + bias1) + res1;
  }
  link_mark(tr, 3);
}

template <uint32_t DT, int G>
__global__ __launch_bounds__(kFrontThreads, 4) void layer_front_kernel(FrontParams p, uint32_t q_wgs, uint32_t a_wgs) {
  __shared__ union {
    AttnShared<G, kFW> attn;
    GemvShared gemv;
  } sh;
  const uint32_t pos = p.attn.cursor != nullptr ? *p.attn.cursor : p.attn.position;
  if (p.attn.cursor != nullptr && pos >= p.attn.max_steps) return;  // same decision in every workgroup
  const uint32_t epoch = *p.step_counter * p.layers + p.layer + 1u;
  const uint32_t b = blockIdx.x;
  if (b < q_wgs) {
    front_q_role<DT, G>(p, b, epoch, sh.gemv);
  } else if (b < q_wgs + a_wgs) {
    const uint32_t a = b - q_wgs;
    const uint32_t kvh = a % p.attn.kv_heads, split = a / p.attn.kv_heads;
    AttnLink link;
    link.qkv_tagged = q_wgs != 0 ? p.qkv_tagged : nullptr;
    link.part_tagged = p.part_tagged;
    link.out_tagged = p.out_tagged;
    link.hints = p.head_hints;
    link.hint_count = p.hidden / kFrontRowsPerWg;
    link.hint_stride = kFrontFlagStride;
    link.split_hints = p.split_hints;
    link.abort_flag = p.abort_flag;
    link.epoch = epoch;
    link.trace = p.trace != nullptr && kvh == 0 && split == 0 ? p.trace : nullptr;
    link.trace_merge = p.trace != nullptr && kvh == 0 ? p.trace : nullptr;
    attn_fast_body<DT, G, kFW, true>(p.attn, pos, kvh, split, p.attn.splits, sh.attn, link, RawHeads<G, kFW>{});
  } else {
    front_o_role<DT>(p, b - q_wgs - a_wgs, epoch, sh.gemv);
  }
}

bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

bool front_supported(uint32_t hidden, uint32_t heads, uint32_t kv_heads, uint32_t head_dim) {
  if (head_dim != static_cast<uint32_t>(kHD) || kv_heads == 0 || heads != 4 * kv_heads) return false;
  if (kv_heads > kFrontFlagStride) return false;                             // one hint word per kv head in a 64-byte line
  if (hidden % kChunkCols != 0 || hidden > kMaxChunks * kChunkCols) return false;  // rows live in registers
  const uint32_t attn_dim = heads * head_dim;
  if (attn_dim > kMaxChunks * kChunkCols) return false;
  return hidden % kFrontRowsPerWg == 0;
}

void front_grid(const FrontParams &p, uint32_t *q_wgs, uint32_t *a_wgs, uint32_t *o_wgs) {
  const uint32_t rows = (p.attn.heads + 2 * p.attn.kv_heads) * p.attn.head_dim;
  *q_wgs = p.wqkv != nullptr ? rows / kFrontQRowsPerWg : 0u;
  *a_wgs = p.attn.kv_heads * p.attn.splits;
  *o_wgs = p.hidden / kFrontRowsPerWg;
}

namespace {
uint64_t round256(uint64_t v) { return (v + 255u) & ~static_cast<uint64_t>(255u); }
}  // namespace

uint64_t front_workspace_bytes(uint32_t heads, uint32_t kv_heads) {
  const uint64_t qkv = round256(static_cast<uint64_t>(heads + 2 * kv_heads) * kHD * 8);
  const uint64_t part = round256(static_cast<uint64_t>(heads) * kAttnMaxSplits * kPartRecord * 8);
  const uint64_t out = round256(static_cast<uint64_t>(heads) * kHD * 8);
  const uint64_t hints = round256(static_cast<uint64_t>(kFrontMaxOWgs) * kFrontFlagStride * 4);
  const uint64_t split_hints = round256(static_cast<uint64_t>(kv_heads) * kAttnMaxSplits * 4);
  return qkv + part + out + hints + split_hints;
}

void front_bind_workspace(FrontParams &p, void *workspace) {
  char *base = static_cast<char *>(workspace);
  const uint32_t heads = p.attn.heads, kv_heads = p.attn.kv_heads;
  p.qkv_tagged = reinterpret_cast<uint64_t *>(base);
  base += round256(static_cast<uint64_t>(heads + 2 * kv_heads) * kHD * 8);
  p.part_tagged = reinterpret_cast<uint64_t *>(base);
  base += round256(static_cast<uint64_t>(heads) * kAttnMaxSplits * kPartRecord * 8);
  p.out_tagged = reinterpret_cast<uint64_t *>(base);
  base += round256(static_cast<uint64_t>(heads) * kHD * 8);
  p.head_hints = reinterpret_cast<uint32_t *>(base);
  base += round256(static_cast<uint64_t>(kFrontMaxOWgs) * kFrontFlagStride * 4);
  p.split_hints = reinterpret_cast<uint32_t *>(base);
}

hipError_t launch_layer_front(uint32_t dtype, const FrontParams &p, hipStream_t stream) {
  const AttnParams &a = p.attn;
  if (a.qkv == nullptr || a.k_cache == nullptr || a.v_cache == nullptr || a.table == nullptr || a.out16 == nullptr)
    return hipErrorInvalidValue;
  if (p.x == nullptr || p.wo == nullptr || p.r == nullptr || p.qkv_tagged == nullptr || p.part_tagged == nullptr ||
      p.out_tagged == nullptr || p.head_hints == nullptr || p.abort_flag == nullptr || p.step_counter == nullptr)
    return hipErrorInvalidValue;
  if (p.wqkv != nullptr && p.rms_attn == nullptr) return hipErrorInvalidValue;
  if (!front_supported(p.hidden, a.heads, a.kv_heads, a.head_dim)) return hipErrorInvalidValue;
  if (a.block_count == 0 || a.splits == 0 || a.splits > kAttnMaxSplits || p.layers == 0 || p.layer >= p.layers)
    return hipErrorInvalidValue;
  if (a.rope_freq != nullptr && a.head_dim % 2 != 0) return hipErrorInvalidValue;
  if (a.cursor == nullptr &&
      static_cast<uint64_t>(a.position) >= static_cast<uint64_t>(a.block_count) * kKvBlockTokens)
    return hipErrorInvalidValue;
  if (!aligned16(p.x) || !aligned16(p.wo) || !aligned16(p.out_tagged) || !aligned16(p.qkv_tagged) ||
      (p.wqkv != nullptr && (!aligned16(p.wqkv) || !aligned16(p.rms_attn))))
    return hipErrorInvalidValue;
  uint32_t q_wgs, a_wgs, o_wgs;
  front_grid(p, &q_wgs, &a_wgs, &o_wgs);
  const dim3 grid(q_wgs + a_wgs + o_wgs);
  if (dtype == kBF16)
    hipLaunchKernelGGL((layer_front_kernel<kBF16, 4>), grid, dim3(kFrontThreads), 0, stream, p, q_wgs, a_wgs);
  else if (dtype == kF16)
    hipLaunchKernelGGL((layer_front_kernel<kF16, 4>), grid, dim3(kFrontThreads), 0, stream, p, q_wgs, a_wgs);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace nv
