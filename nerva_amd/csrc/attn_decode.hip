// Fused decode attention for one new token:
//   bias -> per-head RMSNorm (q_norm/k_norm) -> half-split RoPE -> K/V rounded to
//   16 bits and appended to the paged cache -> split-KV online-softmax attention
//   over keys 0..pos -> merge of the splits -> 16-bit attention output.
// Reference: hf_layer_qkv_prepare_kernel / chunk kernels / reduce kernel
// (kernels.cu:287-555, attention_kernels.cu:263-760), per_head_rms_norm
// (precision/block/ops.rs:52-73), apply_rotary_to_heads (common/rope.rs:54-79),
// exact_blockwise_attention_into (attention/exact/run.rs:13-127).
//
// gfx950 mapping of the fast path (head_dim 128, G = heads/kv_heads in {1,2,4,8}):
//   grid (kv_heads, splits), 8 waves per workgroup; a wave owns whole 16-token KV
//   tiles of its workgroup's token range and runs q.K^T and P.V on the matrix cores
//   (details at attn_fast_kernel). The cache keeps each tile in matrix-operand order,
//   so a tile is eight coalesced 1 KiB loads straight into operand registers; two tiles
//   are in flight per wave. LDS only carries q, the new K/V row and the cross-wave
//   merge. The last workgroup to finish a kv head merges its split partials (arrival
//   counter; nobody waits), so a layer needs no separate reduce launch.
#include "attn_decode.cuh"
#include "attn_tile.cuh"

namespace nv {

namespace {

using namespace attn;

// Parameters of token z of a block launch.
__device__ __forceinline__ void token_view(AttnParams &p, uint32_t z) {
  if (p.seqs != nullptr) {
    const AttnSeq seq = p.seqs[z];
    p.k_cache = seq.k_cache;
    p.v_cache = seq.v_cache;
    p.table = seq.table;
    p.block_count = seq.block_count;
    p.position = seq.position;
  } else {
    p.position += z;
  }
  p.qkv += static_cast<uint64_t>(z) * p.qkv_token_stride;
  p.out16 += attn_out_token(p, z);
  if (p.out_f32 != nullptr) p.out_f32 += static_cast<uint64_t>(z) * p.out_token_stride;
  if (p.rope_cs != nullptr) p.rope_cs += static_cast<uint64_t>(z) * p.rope_token_stride;
  const uint64_t ws = z * p.ws_token_stride;
  p.part_acc = reinterpret_cast<float *>(reinterpret_cast<char *>(p.part_acc) + ws);
  p.part_m = reinterpret_cast<float *>(reinterpret_cast<char *>(p.part_m) + ws);
  p.part_l = reinterpret_cast<float *>(reinterpret_cast<char *>(p.part_l) + ws);
  p.counters = reinterpret_cast<uint32_t *>(reinterpret_cast<char *>(p.counters) + ws);
}

// K and V rows of a prompt block into the cache: grid (kv head, token), two waves (key, value).
template <uint32_t DT>
__global__ __launch_bounds__(2 * kWave) void kv_publish_rows_kernel(AttnParams p) {
  __shared__ __align__(16) uint16_t row16[2][kHD];
  const uint32_t kvh = blockIdx.x, z = blockIdx.y;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  uint32_t pos = p.position + z;
  if (p.seqs != nullptr) {
    const AttnSeq seq = p.seqs[z];
    p.k_cache = seq.k_cache;
    p.v_cache = seq.v_cache;
    p.table = seq.table;
    p.block_count = seq.block_count;
    pos = seq.position;
  }
  const uint32_t A = p.heads * kHD, KV = p.kv_heads * kHD;
  const float *qkv = p.qkv + static_cast<uint64_t>(z) * p.qkv_token_stride;
  const float *rope_cs = p.rope_cs != nullptr ? p.rope_cs + static_cast<uint64_t>(z) * p.rope_token_stride : nullptr;
  const uint32_t off = (wave == 0 ? A : A + KV) + kvh * kHD;
  const uint16_t *bias = wave == 0 ? p.k_bias : p.v_bias;
  prep_head128<DT>(qkv[off + lane], qkv[off + lane + 64], bias ? bias + kvh * kHD : nullptr, wave == 0 ? p.k_norm : nullptr,
                   wave == 0 ? p.rope_freq : nullptr, rope_cs, pos, p.eps, lane, nullptr, row16[wave]);
  __syncthreads();
  const uint64_t tile = kv_tile_offset(p.block_count, p.kv_heads, kHD, p.layer, p.table[pos / kKvBlockTokens], kvh);
  const uint32_t row = pos % kKvBlockTokens;
  if (wave == 0) {
    if (lane < 16)  // K: 16 pieces of 8 consecutive dims
      *reinterpret_cast<uint4 *>(p.k_cache + tile + kv_k_elem(kHD, row, lane * 8)) =
          *reinterpret_cast<const uint4 *>(row16[0] + lane * 8);
  } else {
#pragma unroll
    for (int i = 0; i < 2; ++i) {  // V: one 16-bit element per dim
      const uint32_t d = lane + i * kWave;
      p.v_cache[tile + kv_v_elem(kHD, row, d)] = row16[1][d];
    }
  }
}

// Stand-alone launch of the matrix-core attention (attn_fast_body): grid (kv_heads, splits[, tokens]).
template <uint32_t DT, int G, int W>
__global__ __launch_bounds__(W *kWave) void attn_fast_kernel(AttnParams p) {
  __shared__ AttnShared<G, W> sh;
  if (blockIdx.z != 0) token_view(p, blockIdx.z);
  const RawHeads<G, W> raw = attn_request_raw<G, W>(p, blockIdx.x);  // before anything they could queue behind
  const uint32_t pos = p.cursor != nullptr ? *p.cursor : p.position;
  if (p.cursor != nullptr && pos >= p.max_steps) return;
  attn_fast_body<DT, G, W, false>(p, pos, blockIdx.x, blockIdx.y, gridDim.y, sh, AttnLink{}, raw);
}

// Prompt-block launch of the same body (grid z = tokens): the lean variant, two workgroups per CU.
template <uint32_t DT, int G, int W>
__global__ __launch_bounds__(W *kWave, W / 2) void attn_block_kernel(AttnParams p) {
  __shared__ AttnShared<G, W> sh;
  if (blockIdx.z != 0 || p.seqs != nullptr) token_view(p, blockIdx.z);
  const RawHeads<G, W> raw = attn_request_raw<G, W>(p, blockIdx.x);
  attn_fast_body<DT, G, W, false, 1>(p, p.position, blockIdx.x, blockIdx.y, gridDim.y, sh, AttnLink{}, raw);
}

// Any head_dim (even when RoPE is on) / any group size: one workgroup per query
// head, waves stride over tokens, lanes over dims. Used for shapes the fast path
// does not cover (the tiny known-answer models).
template <uint32_t DT>
__global__ __launch_bounds__(kBlock) void attn_generic_kernel(AttnParams p) {
  extern __shared__ __align__(16) float sm[];
  __shared__ float red[kWavesPerBlock];
  __shared__ float wm[kWavesPerBlock], wl[kWavesPerBlock];
  const uint32_t hd = p.head_dim, half = hd / 2;
  float *q = sm;                 // [hd]
  float *kn = sm + hd;           // [hd] rounded new key
  float *vn = sm + 2 * hd;       // [hd] rounded new value
  float *wacc = sm + 3 * hd;     // [waves][hd]

  const uint32_t pos = p.cursor != nullptr ? *p.cursor : p.position;
  if (p.cursor != nullptr && pos >= p.max_steps) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint32_t h = blockIdx.x, group = p.heads / p.kv_heads, kvh = h / group;
  const uint32_t A = p.heads * hd, KV = p.kv_heads * hd;
  const uint32_t n_keys = pos + 1;

  // q: bias -> per-head norm -> RoPE
  float ss = 0.0f;
  for (uint32_t d = threadIdx.x; d < hd; d += kBlock) {
    float v = p.qkv[h * hd + d];
    if (p.q_bias) v += dec16<DT>(p.q_bias[h * hd + d]);
    q[d] = v;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  if (p.q_norm) {
    const float sc = 1.0f / sqrtf(ss / static_cast<float>(hd) + p.eps);
    for (uint32_t d = threadIdx.x; d < hd; d += kBlock) q[d] *= sc * dec16<DT>(p.q_norm[d]);
  }
  __syncthreads();
  if (p.rope_freq) {
    for (uint32_t i = threadIdx.x; i < half; i += kBlock) {
      const float angle = static_cast<float>(pos) / p.rope_freq[i];
      float s, c;
      sincosf(angle, &s, &c);
      const float a = q[i], b = q[i + half];
      q[i] = a * c - b * s;
      q[i + half] = b * c + a * s;
    }
  }
  if (p.append) {
    float ks = 0.0f;
    for (uint32_t d = threadIdx.x; d < hd; d += kBlock) {
      float kv = p.qkv[A + kvh * hd + d];
      if (p.k_bias) kv += dec16<DT>(p.k_bias[kvh * hd + d]);
      kn[d] = kv;
      ks += kv * kv;
      float vv = p.qkv[A + KV + kvh * hd + d];
      if (p.v_bias) vv += dec16<DT>(p.v_bias[kvh * hd + d]);
      vn[d] = vv;
    }
    ks = block_sum(ks, red);
    if (p.k_norm) {
      const float sc = 1.0f / sqrtf(ks / static_cast<float>(hd) + p.eps);
      for (uint32_t d = threadIdx.x; d < hd; d += kBlock) kn[d] *= sc * dec16<DT>(p.k_norm[d]);
    }
    __syncthreads();
    if (p.rope_freq) {
      for (uint32_t i = threadIdx.x; i < half; i += kBlock) {
        const float angle = static_cast<float>(pos) / p.rope_freq[i];
        float s, c;
        sincosf(angle, &s, &c);
        const float a = kn[i], b = kn[i + half];
        kn[i] = a * c - b * s;
        kn[i + half] = b * c + a * s;
      }
    }
    __syncthreads();
    const uint64_t tile = kv_tile_offset(p.block_count, p.kv_heads, hd, p.layer,
                                         p.table[pos / kKvBlockTokens], kvh);
    const uint32_t prow = pos % kKvBlockTokens;
    for (uint32_t d = threadIdx.x; d < hd; d += kBlock) {
      const uint16_t k16 = enc16<DT>(kn[d]), v16 = enc16<DT>(vn[d]);
      if (h % group == 0) {
        p.k_cache[tile + kv_k_elem(hd, prow, d)] = k16;
        p.v_cache[tile + kv_v_elem(hd, prow, d)] = v16;
      }
      kn[d] = dec16<DT>(k16);
      vn[d] = dec16<DT>(v16);
    }
  }
  __syncthreads();

  constexpr int kMaxPerLane = 8;  // head_dim <= 512
  float acc[kMaxPerLane];
#pragma unroll
  for (int j = 0; j < kMaxPerLane; ++j) acc[j] = 0.0f;
  float m = -INFINITY, l = 0.0f;
  const float scale = 1.0f / sqrtf(static_cast<float>(hd));
  for (uint32_t t = wave; t < n_keys; t += kWavesPerBlock) {
    const bool fresh = p.append && t == pos;
    const uint64_t tile = kv_tile_offset(p.block_count, p.kv_heads, hd, p.layer,
                                         p.table[t / kKvBlockTokens], kvh);
    const uint32_t trow = t % kKvBlockTokens;
    float partial = 0.0f;
    for (uint32_t d = lane; d < hd; d += kWave)
      partial = fmaf(q[d], fresh ? kn[d] : dec16<DT>(p.k_cache[tile + kv_k_elem(hd, trow, d)]), partial);
    const float score = wave_sum(partial) * scale;
    const float m_new = fmaxf(m, score);
    const float alpha = l == 0.0f ? 0.0f : expf(m - m_new);
    const float pnew = expf(score - m_new);
#pragma unroll
    for (int j = 0; j < kMaxPerLane; ++j) {
      const uint32_t d = lane + j * kWave;
      if (d < hd) acc[j] = acc[j] * alpha + (fresh ? vn[d] : dec16<DT>(p.v_cache[tile + kv_v_elem(hd, trow, d)])) * pnew;
    }
    l = l * alpha + pnew;
    m = m_new;
  }
#pragma unroll
  for (int j = 0; j < kMaxPerLane; ++j) {
    const uint32_t d = lane + j * kWave;
    if (d < hd) wacc[wave * hd + d] = acc[j];
  }
  if (lane == 0) {
    wm[wave] = m;
    wl[wave] = l;
  }
  __syncthreads();
  float M = -INFINITY;
  for (int w = 0; w < kWavesPerBlock; ++w) M = fmaxf(M, wm[w]);
  for (uint32_t d = threadIdx.x; d < hd; d += kBlock) {
    float L = 0.0f, o = 0.0f;
    for (int w = 0; w < kWavesPerBlock; ++w) {
      if (wm[w] > -INFINITY) {
        const float f = expf(wm[w] - M);
        L += wl[w] * f;
        o += wacc[w * hd + d] * f;
      }
    }
    if (L > 0.0f && isfinite(L)) o /= L;
    if (p.out_f32) p.out_f32[h * hd + d] = o;
    p.out16[h * hd + d] = enc16<DT>(o);
  }
}

template <uint32_t DT>
hipError_t launch_dt(const AttnParams &p, hipStream_t stream) {
  const uint32_t group = p.heads / p.kv_heads;
  const bool fast = p.head_dim == kHD && (group == 1 || group == 2 || group == 4 || group == 8) &&
                    p.part_acc != nullptr && p.splits >= 1;
  if (fast) {
    const dim3 grid(p.kv_heads, p.splits, p.tokens > 1 ? p.tokens : 1);
    if (p.tokens > 1 || p.seqs != nullptr) {
      switch (group) {
        case 1: hipLaunchKernelGGL((attn_block_kernel<DT, 1, kAttnWaves>), grid, dim3(kAttnWaves * kWave), 0, stream, p); break;
        case 2: hipLaunchKernelGGL((attn_block_kernel<DT, 2, kAttnWaves>), grid, dim3(kAttnWaves * kWave), 0, stream, p); break;
        case 4: hipLaunchKernelGGL((attn_block_kernel<DT, 4, kAttnWaves>), grid, dim3(kAttnWaves * kWave), 0, stream, p); break;
        default: hipLaunchKernelGGL((attn_block_kernel<DT, 8, kAttnWaves / 2>), grid, dim3(kAttnWaves / 2 * kWave), 0, stream, p); break;
      }
      return hipGetLastError();
    }
    switch (group) {
      case 1: hipLaunchKernelGGL((attn_fast_kernel<DT, 1, kAttnWaves>), grid, dim3(kAttnWaves * kWave), 0, stream, p); break;
      case 2: hipLaunchKernelGGL((attn_fast_kernel<DT, 2, kAttnWaves>), grid, dim3(kAttnWaves * kWave), 0, stream, p); break;
      case 4: hipLaunchKernelGGL((attn_fast_kernel<DT, 4, kAttnWaves>), grid, dim3(kAttnWaves * kWave), 0, stream, p); break;
      default: hipLaunchKernelGGL((attn_fast_kernel<DT, 8, kAttnWaves / 2>), grid, dim3(kAttnWaves / 2 * kWave), 0, stream, p); break;
    }
  } else {
    if (p.head_dim > 512) return hipErrorInvalidValue;
    const size_t lds = static_cast<size_t>(3 + kWavesPerBlock) * p.head_dim * sizeof(float);
    hipLaunchKernelGGL((attn_generic_kernel<DT>), dim3(p.heads), dim3(kBlock), lds, stream, p);
  }
  return hipGetLastError();
}

}  // namespace

uint64_t attn_workspace_bytes(uint32_t heads, uint32_t head_dim) {
  const uint64_t acc = static_cast<uint64_t>(heads) * kAttnMaxSplits * head_dim * sizeof(float);
  const uint64_t ml = static_cast<uint64_t>(heads) * kAttnMaxSplits * sizeof(float) * 2;
  return acc + ml + 1024 * sizeof(uint32_t);
}

void attn_bind_workspace(AttnParams &p, void *workspace) {
  char *base = static_cast<char *>(workspace);
  const uint64_t acc = static_cast<uint64_t>(p.heads) * kAttnMaxSplits * p.head_dim * sizeof(float);
  const uint64_t ml = static_cast<uint64_t>(p.heads) * kAttnMaxSplits * sizeof(float);
  p.part_acc = reinterpret_cast<float *>(base);
  p.part_m = reinterpret_cast<float *>(base + acc);
  p.part_l = reinterpret_cast<float *>(base + acc + ml);
  p.counters = reinterpret_cast<uint32_t *>(base + acc + 2 * ml);
}

hipError_t launch_kv_publish_rows(uint32_t dtype, const AttnParams &p, hipStream_t stream) {
  const bool caches = p.seqs != nullptr || (p.k_cache != nullptr && p.v_cache != nullptr && p.table != nullptr);
  if (p.qkv == nullptr || !caches || p.tokens == 0 || p.head_dim != static_cast<uint32_t>(kHD) || p.kv_heads == 0)
    return hipErrorInvalidValue;
  if (p.seqs == nullptr &&
      static_cast<uint64_t>(p.position) + p.tokens > static_cast<uint64_t>(p.block_count) * kKvBlockTokens)
    return hipErrorInvalidValue;
  const dim3 grid(p.kv_heads, p.tokens);
  if (dtype == kBF16) hipLaunchKernelGGL(kv_publish_rows_kernel<kBF16>, grid, dim3(2 * kWave), 0, stream, p);
  else if (dtype == kF16) hipLaunchKernelGGL(kv_publish_rows_kernel<kF16>, grid, dim3(2 * kWave), 0, stream, p);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launch_attn_decode(uint32_t dtype, const AttnParams &p, hipStream_t stream) {
  const bool caches = p.seqs != nullptr || (p.k_cache != nullptr && p.v_cache != nullptr && p.table != nullptr);
  if (p.qkv == nullptr || !caches || p.out16 == nullptr) return hipErrorInvalidValue;
  if (p.heads == 0 || p.kv_heads == 0 || p.head_dim == 0 || p.heads % p.kv_heads != 0 ||
      (p.seqs == nullptr && p.block_count == 0) || p.kv_heads > 1024)
    return hipErrorInvalidValue;
  if (p.rope_freq != nullptr && p.head_dim % 2 != 0) return hipErrorInvalidValue;
  if (p.splits > kAttnMaxSplits) return hipErrorInvalidValue;
  if (p.cursor == nullptr && p.seqs == nullptr &&
      static_cast<uint64_t>(p.position) >= static_cast<uint64_t>(p.block_count) * kKvBlockTokens)
    return hipErrorInvalidValue;
  if (p.out_packed_tiles != 0 && (!(p.tokens > 1 || p.seqs != nullptr) || p.out_packed_tiles * 16u < p.tokens || p.out_f32 != nullptr))
    return hipErrorInvalidValue;
  if (p.tokens > 1 || p.seqs != nullptr) {
    // a block of positions or of sequences: host-given positions, matrix-core kernel only
    const uint32_t group = p.heads / p.kv_heads;
    const bool fast = p.head_dim == 128 && (group == 1 || group == 2 || group == 4 || group == 8) && p.part_acc != nullptr;
    // (rows of consecutive positions have to be in the cache before the launch; rows of different
    // sequences can be appended by the launch itself, as the single-token kernel does)
    if (p.cursor != nullptr || (p.append != 0 && p.seqs == nullptr) || !fast || p.tokens == 0 || p.tokens > 65535 ||
        (p.seqs == nullptr &&
         static_cast<uint64_t>(p.position) + p.tokens > static_cast<uint64_t>(p.block_count) * kKvBlockTokens))
      return hipErrorInvalidValue;
  }
  if (dtype == kBF16) return launch_dt<kBF16>(p, stream);
  if (dtype == kF16) return launch_dt<kF16>(p, stream);
  return hipErrorInvalidValue;
}

}  // namespace nv
