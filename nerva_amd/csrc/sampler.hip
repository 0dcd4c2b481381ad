// Device sampler beyond greedy (see sampler.cuh).
#include "sampler.cuh"

#include <math.h>

namespace nv {

namespace {

constexpr int kChunkThreads = 256;
constexpr int kSelectThreads = 1024;
constexpr uint32_t kDigitBits = 11;            // radix selection: five 11-bit digits and one of 9 bits
constexpr uint32_t kBins = 1u << kDigitBits;
constexpr int kLevels = 6;

// sampler.cu:18-23
__device__ __forceinline__ uint64_t mix64(uint64_t value) {
  value += 0x9e3779b97f4a7c15ull;
  value = (value ^ (value >> 30)) * 0xbf58476d1ce4e5b9ull;
  value = (value ^ (value >> 27)) * 0x94d049bb133111ebull;
  return value ^ (value >> 31);
}
// sampler.cu:25-33: 24 hashed bits -> (0, 1]
__device__ __forceinline__ float uniform_open(uint64_t seed, uint32_t position, uint32_t token, uint32_t salt) {
  uint64_t value = seed ^ (static_cast<uint64_t>(position) << 32) ^ static_cast<uint64_t>(token) ^
                   (static_cast<uint64_t>(salt) << 48);
  value = mix64(value);
  const uint32_t mantissa = static_cast<uint32_t>((value >> 40) & 0x00ffffffu);
  return (static_cast<float>(mantissa) + 1.0f) / 16777217.0f;
}
// sampler.cu:42-66: larger floats get larger unsigned codes; with the inverted index below them
// an integer comparison of two keys is (value desc, index asc). No finite value encodes as 0 in
// the upper word, so key 0 marks "no candidate".
__device__ __forceinline__ uint64_t make_key(float value, uint32_t index) {
  const uint32_t bits = __float_as_uint(value);
  const uint32_t ordered = (bits & 0x80000000u) != 0u ? ~bits : (bits | 0x80000000u);
  return (static_cast<uint64_t>(ordered) << 32) | static_cast<uint64_t>(~index);
}
__device__ __forceinline__ float key_value(uint64_t key) {
  const uint32_t ordered = static_cast<uint32_t>(key >> 32);
  return __uint_as_float((ordered & 0x80000000u) != 0u ? (ordered & 0x7fffffffu) : ~ordered);
}
__device__ __forceinline__ uint32_t key_index(uint64_t key) { return ~static_cast<uint32_t>(key); }

__device__ __forceinline__ uint32_t wanted_candidates(uint32_t top_k, uint32_t vocab) {
  const uint32_t requested = top_k == 0 ? kSamplerTopKMax : (top_k < kSamplerTopKMax ? top_k : kSamplerTopKMax);
  return requested < vocab ? requested : vocab;  // sampler.cu:169-174
}

// `batch` (device memory) replaces `p` by its entry blockIdx.y: one launch for several sequences.
__global__ __launch_bounds__(kChunkThreads) void sample_chunk_kernel(SamplerParams p, const SamplerParams *batch) {
  if (batch != nullptr) p = batch[blockIdx.y];
  __shared__ uint64_t keys[kChunkThreads / kWave];
  __shared__ float red_v[kChunkThreads / kWave];
  __shared__ uint32_t red_i[kChunkThreads / kWave];
  __shared__ uint32_t red_h[kChunkThreads / kWave];
  const uint32_t pos = p.cursor != nullptr ? *p.cursor : p.position;
  if (p.cursor != nullptr && pos >= p.max_steps) return;
  const SamplerDev cfg = *p.config;
  const uint32_t base = blockIdx.x * kSamplerChunk;

  if (cfg.mode != kSamplerTopK) {
    // best (score, index) of the chunk: the raw logit, or logit / T plus Gumbel noise
    const bool noisy = cfg.mode == kSamplerGumbel;
    const float inv_temperature = noisy ? 1.0f / cfg.temperature : 1.0f;
    Best b{0.0f, 0u, 0u};
    for (uint32_t j = 0; j < kSamplerChunk / kChunkThreads; ++j) {
      const uint32_t i = base + j * kChunkThreads + threadIdx.x;
      if (i >= p.vocab) continue;
      const float v = p.logits[i];
      if (!isfinite(v)) continue;
      float score = v;
      if (noisy) {
        const float u = uniform_open(cfg.seed, pos, i, 0);
        score = v * inv_temperature + (-logf(-logf(u)));
      }
      const Best cand{score, i, 1u};
      if (better(cand, b)) b = cand;
    }
    b = wave_best(b);
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) {
      red_v[wave] = b.value;
      red_i[wave] = b.index;
      red_h[wave] = b.has;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      Best t{red_v[0], red_i[0], red_h[0]};
      for (int w = 1; w < kChunkThreads / kWave; ++w) {
        const Best o{red_v[w], red_i[w], red_h[w]};
        if (better(o, t)) t = o;
      }
      p.out.part_value[blockIdx.x] = t.value;
      p.out.part_index[blockIdx.x] = t.index;
      p.out.part_has[blockIdx.x] = t.has;
    }
    return;
  }

  // top-k: the chunk's best key and the number of its finite logits (words 0 and 1 of the chunk's workspace row)
  uint64_t best = 0;
  uint32_t finite = 0;
  for (uint32_t e = threadIdx.x; e < kSamplerChunk; e += kChunkThreads) {
    const uint32_t i = base + e;
    if (i < p.vocab) {
      const float v = p.logits[i];
      if (isfinite(v)) {
        const uint64_t key = make_key(v, i);
        best = key > best ? key : best;
        ++finite;
      }
    }
  }
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const uint64_t other = (static_cast<uint64_t>(__shfl_xor(static_cast<uint32_t>(best >> 32), o, kWave)) << 32) |
                           __shfl_xor(static_cast<uint32_t>(best), o, kWave);
    best = other > best ? other : best;
    finite += __shfl_xor(finite, o, kWave);
  }
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) {
    keys[wave] = best;
    red_i[wave] = finite;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kChunkThreads / kWave; ++w) {
      best = keys[w] > best ? keys[w] : best;
      finite += red_i[w];
    }
    p.keys[static_cast<uint64_t>(blockIdx.x) * kSamplerTopKMax] = best;
    p.keys[static_cast<uint64_t>(blockIdx.x) * kSamplerTopKMax + 1] = finite;
  }
}

__global__ __launch_bounds__(kSelectThreads) void sample_select_kernel(SamplerParams p, uint32_t chunks,
                                                                      const SamplerParams *batch) {
  if (batch != nullptr) p = batch[blockIdx.y];
  __shared__ uint32_t hist[kBins];
  __shared__ uint32_t scan[kSelectThreads];
  __shared__ uint64_t top[kSamplerTopKMax];
  __shared__ uint64_t cand[kSelectThreads];
  __shared__ float ex[kSamplerTopKMax];
  __shared__ float red_v[kSelectThreads / kWave];
  __shared__ uint32_t red_i[kSelectThreads / kWave];
  __shared__ uint32_t red_h[kSelectThreads / kWave];
  __shared__ uint64_t prefix_s;
  __shared__ uint32_t need_s, count_s;
  const uint32_t pos = p.cursor != nullptr ? *p.cursor : p.position;
  if (p.cursor != nullptr && pos >= p.max_steps) return;
  const SamplerDev cfg = *p.config;
  const uint32_t tid = threadIdx.x;

  if (cfg.mode != kSamplerTopK) {
    Best b{0.0f, 0u, 0u};
    for (uint32_t i = tid; i < chunks; i += kSelectThreads) {
      const Best o{p.out.part_value[i], p.out.part_index[i], p.out.part_has[i]};
      if (better(o, b)) b = o;
    }
    b = wave_best(b);
    const int wave = tid / kWave;
    if ((tid & (kWave - 1)) == 0) {
      red_v[wave] = b.value;
      red_i[wave] = b.index;
      red_h[wave] = b.has;
    }
    __syncthreads();
    if (tid == 0) {
      Best t{red_v[0], red_i[0], red_h[0]};
      for (int w = 1; w < kSelectThreads / kWave; ++w) {
        const Best o{red_v[w], red_i[w], red_h[w]};
        if (better(o, t)) t = o;
      }
      publish_token(p.out, t.has ? t.index : 0u);
    }
    return;
  }

  // ---- top-k: how many finite logits are there at all
  // (a workgroup barrier of sixteen waves costs a third of a microsecond: sums and orders below are arranged to
  // need few of them - wave sums first, ranks by counting instead of sorting networks)
  uint32_t mine = 0;
  for (uint32_t c = tid; c < chunks; c += kSelectThreads)
    mine += static_cast<uint32_t>(p.keys[static_cast<uint64_t>(c) * kSamplerTopKMax + 1]);
  for (int o = kWave / 2; o > 0; o >>= 1) mine += __shfl_xor(mine, o, kWave);
  if ((tid & (kWave - 1)) == 0) red_i[tid / kWave] = mine;
  __syncthreads();
  uint32_t finite_candidates = 0;
  for (int w = 0; w < kSelectThreads / kWave; ++w) finite_candidates += red_i[w];
  __syncthreads();
  uint32_t selected = wanted_candidates(cfg.top_k, p.vocab);
  if (selected > finite_candidates) selected = finite_candidates;  // fewer finite logits than requested
  if (selected == 0) {
    if (tid == 0) publish_token(p.out, 0u);  // sampler.cu:345-346
    return;
  }

  // ---- fast path: a bound from the chunk maxima. The selected-th largest of the chunks' best keys is no
  // larger than the selected-th largest key overall, so only keys at or above it matter: with logits spread
  // over the chunks that leaves a few hundred of the whole vocabulary, which one pass over the logits collects
  // and a sort in LDS orders. (Keys are distinct, so the order they are collected in does not show.)
  bool fast = chunks <= static_cast<uint32_t>(kSelectThreads);
  if (fast) {
    cand[tid] = tid < chunks ? p.keys[static_cast<uint64_t>(tid) * kSamplerTopKMax] : 0ull;
    if (tid == 0) {
      prefix_s = 0;   // the bound: 0 (everything) when fewer chunks than `selected` hold a finite logit
      count_s = 0;
    }
    __syncthreads();
    const uint64_t mine_max = cand[tid];
    if (mine_max != 0ull) {
      uint32_t above = 0;
      for (uint32_t c = 0; c < chunks; ++c) above += cand[c] > mine_max ? 1u : 0u;
      if (above == selected - 1) prefix_s = mine_max;   // distinct keys: exactly one chunk has this rank
    }
    __syncthreads();
    const uint64_t bound = prefix_s;
    __syncthreads();
    // One workgroup looks at every logit, so the look is two comparisons (a float at or above the bound's value,
    // and finite); the key is formed and compared exactly only for the few that pass (forming every key was 15
    // instructions a logit: 17 of the kernel's 36 us). Eight logits are requested before the first is looked at.
    const float bound_value = bound != 0ull ? key_value(bound) : -INFINITY;
    constexpr uint32_t kScan = 8;
    for (uint32_t i0 = tid; i0 < p.vocab; i0 += kScan * kSelectThreads) {
      float v[kScan];
#pragma unroll
      for (uint32_t u = 0; u < kScan; ++u) v[u] = p.logits[min(i0 + u * kSelectThreads, p.vocab - 1)];
#pragma unroll
      for (uint32_t u = 0; u < kScan; ++u) {
        const uint32_t i = i0 + u * kSelectThreads;
        if (v[u] >= bound_value && fabsf(v[u]) <= 3.402823466e+38f && i < p.vocab) {   // (finite: a NaN passes neither)
          const uint64_t key = make_key(v[u], i);
          if (key >= bound) {
            const uint32_t slot = atomicAdd(&count_s, 1u);
            if (slot < static_cast<uint32_t>(kSelectThreads)) cand[slot] = key;
          }
        }
      }
    }
    __syncthreads();
    const uint32_t total = count_s;
    fast = total <= static_cast<uint32_t>(kSelectThreads);   // same value in every thread
    if (fast) {
      // order by counting: a key's place is the number of keys above it (distinct keys: no two share a place)
      if (tid < kSamplerTopKMax) top[tid] = 0ull;
      __syncthreads();
      if (tid < total) {
        const uint64_t key = cand[tid];
        uint32_t above = 0;
        for (uint32_t c = 0; c < total; ++c) above += cand[c] > key ? 1u : 0u;
        if (above < kSamplerTopKMax) top[above] = key;
      }
      __syncthreads();
    }
  }
  if (!fast) {
    // ---- the selected-th largest key of the whole vocabulary, digit by digit from the top
    uint64_t prefix = 0, mask = 0;
    uint32_t need = selected;
    for (int level = 0; level < kLevels; ++level) {
      const uint32_t width = level + 1 < kLevels ? kDigitBits : 64u - kDigitBits * (kLevels - 1);
      const uint32_t shift = level + 1 < kLevels ? 64u - kDigitBits * (level + 1) : 0u;
      const uint32_t bins = 1u << width;
      for (uint32_t b = tid; b < kBins; b += kSelectThreads) hist[b] = 0;
      __syncthreads();
      for (uint32_t i = tid; i < p.vocab; i += kSelectThreads) {
        const float v = p.logits[i];
        const uint64_t key = isfinite(v) ? make_key(v, i) : 0ull;
        if (key != 0ull && (key & mask) == prefix) atomicAdd(&hist[static_cast<uint32_t>(key >> shift) & (bins - 1u)], 1u);
      }
      __syncthreads();
      // suffix sums over the bins: thread t owns bins 2t and 2t + 1
      const uint32_t h0 = hist[2 * tid], h1 = hist[2 * tid + 1];
      scan[tid] = h0 + h1;
      __syncthreads();
      for (uint32_t d = 1; d < kSelectThreads; d <<= 1) {
        const uint32_t v = scan[tid] + (tid + d < kSelectThreads ? scan[tid + d] : 0u);
        __syncthreads();
        scan[tid] = v;
        __syncthreads();
      }
      const uint32_t above_pair = tid + 1 < kSelectThreads ? scan[tid + 1] : 0u;  // keys in bins > 2t + 1
      const uint32_t from_hi = above_pair + h1;                                   // keys in bins >= 2t + 1
      const uint32_t from_lo = from_hi + h0;                                      // keys in bins >= 2t
      // the digit's bin is the one whose suffix sum reaches `need` while the next one's does not
      if (from_hi >= need && above_pair < need) {
        prefix_s = prefix | (static_cast<uint64_t>(2 * tid + 1) << shift);
        need_s = need - above_pair;
      } else if (from_lo >= need && from_hi < need) {
        prefix_s = prefix | (static_cast<uint64_t>(2 * tid) << shift);
        need_s = need - from_hi;
      }
      __syncthreads();
      prefix = prefix_s;
      need = need_s;
      mask |= static_cast<uint64_t>(bins - 1u) << shift;
      __syncthreads();
    }

    // ---- keys are distinct, so `prefix` is that key itself: gather everything at or above it
    if (tid == 0) count_s = 0;
    for (uint32_t e = tid; e < kSamplerTopKMax; e += kSelectThreads) top[e] = 0ull;
    __syncthreads();
    for (uint32_t i = tid; i < p.vocab; i += kSelectThreads) {
      const float v = p.logits[i];
      const uint64_t key = isfinite(v) ? make_key(v, i) : 0ull;
      if (key != 0ull && key >= prefix) {
        const uint32_t slot = atomicAdd(&count_s, 1u);
        if (slot < kSamplerTopKMax) top[slot] = key;
      }
    }
    __syncthreads();
    uint64_t key = 0;
    uint32_t above = 0;
    if (tid < kSamplerTopKMax) {
      key = top[tid];
      for (uint32_t c = 0; c < kSamplerTopKMax; ++c) above += top[c] > key ? 1u : 0u;
    }
    __syncthreads();
    if (tid < kSamplerTopKMax) top[tid] = 0ull;
    __syncthreads();
    if (tid < kSamplerTopKMax && key != 0ull) top[above] = key;
    __syncthreads();
  }

  // ---- softmax with temperature over the sorted candidates, nucleus, draw (sampler.cu:343-388)
  const float inv_temperature = 1.0f / cfg.temperature;
  const float max_value = key_value(top[0]);
  if (tid < selected) ex[tid] = expf((key_value(top[tid]) - max_value) * inv_temperature);
  __syncthreads();
  // The rule's three sums (total, nucleus, draw) are one running sum over the candidates in order, read at
  // three places: lane 0 forms it once - sequential float additions, the rule's order, eight LDS values
  // requested per turn - and the two searches ("first candidate whose running share reaches top_p", "first whose
  // running sum reaches the draw") test every candidate at once.
  if (tid == 0) {
    float run = 0.0f;
    for (uint32_t i0 = 0; i0 < selected; i0 += 8) {
      float e[8];
#pragma unroll
      for (uint32_t u = 0; u < 8; ++u) e[u] = ex[min(i0 + u, selected - 1)];
#pragma unroll
      for (uint32_t u = 0; u < 8; ++u) {
        if (i0 + u < selected) {
          run += e[u];
          ex[i0 + u] = run;
        }
      }
    }
    need_s = selected;   // kept: candidates inside the nucleus
    count_s = selected;  // first candidate at or above the draw
  }
  __syncthreads();
  const float total = ex[selected - 1];
  if (cfg.top_p < 0.999999f && tid < selected && total > 0.0f && ex[tid] / total >= cfg.top_p) atomicMin(&need_s, tid + 1);
  __syncthreads();
  const uint32_t kept = need_s;
  const float kept_total = ex[kept - 1];
  const float draw = uniform_open(cfg.seed, pos, 0, 1) * kept_total;
  if (tid < kept && draw <= ex[tid]) atomicMin(&count_s, tid);
  __syncthreads();
  if (tid == 0) {
    uint32_t token = key_index(top[0]);
    if (kept_total > 0.0f) token = key_index(top[count_s < kept ? count_s : kept - 1]);
    publish_token(p.out, token);
  }
}

uint64_t round256(uint64_t v) { return (v + 255u) & ~static_cast<uint64_t>(255u); }

}  // namespace

SamplerDev sampler_device_config(const NervaHipHfDecodeSamplerConfig &config) {
  SamplerDev d{};
  d.temperature = (isfinite(config.temperature) && config.temperature >= 0.0f) ? config.temperature : 0.0f;
  d.top_p = (isfinite(config.top_p) && config.top_p > 0.0f && config.top_p <= 1.0f) ? config.top_p : 1.0f;
  d.top_k = config.top_k;
  d.seed = config.seed;
  if (!(d.temperature > 0.0f) || d.top_k == 1) d.mode = kSamplerGreedy;           // sampler.cu:89
  else if (d.top_k == 0 && d.top_p >= 0.999999f) d.mode = kSamplerGumbel;         // sampler.cu:121
  else d.mode = kSamplerTopK;
  return d;
}

uint64_t sampler_workspace_bytes(uint32_t vocab) {
  return round256(static_cast<uint64_t>(sampler_chunks(vocab)) * kSamplerTopKMax * sizeof(uint64_t));
}

hipError_t launch_sampler(const SamplerParams &p, hipStream_t stream) {
  if (p.logits == nullptr || p.config == nullptr || p.keys == nullptr || p.vocab == 0 ||
      p.out.part_value == nullptr || p.out.part_index == nullptr || p.out.part_has == nullptr)
    return hipErrorInvalidValue;
  const uint32_t chunks = sampler_chunks(p.vocab);
  if (chunks > kSampleMaxBlocks) return hipErrorInvalidValue;
  hipLaunchKernelGGL(sample_chunk_kernel, dim3(chunks), dim3(kChunkThreads), 0, stream, p, nullptr);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(sample_select_kernel, dim3(1), dim3(kSelectThreads), 0, stream, p, chunks, nullptr);
  return hipGetLastError();
}

hipError_t launch_sampler_batch(const SamplerParams *batch, uint32_t count, uint32_t vocab, hipStream_t stream) {
  if (batch == nullptr || count == 0 || count > 65535 || vocab == 0) return hipErrorInvalidValue;
  const uint32_t chunks = sampler_chunks(vocab);
  if (chunks > kSampleMaxBlocks) return hipErrorInvalidValue;
  hipLaunchKernelGGL(sample_chunk_kernel, dim3(chunks, count), dim3(kChunkThreads), 0, stream, SamplerParams{}, batch);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(sample_select_kernel, dim3(1, count), dim3(kSelectThreads), 0, stream, SamplerParams{}, chunks, batch);
  return hipGetLastError();
}

}  // namespace nv
