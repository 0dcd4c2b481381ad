// Token sampling beyond greedy for the decode step: temperature with the whole vocabulary
// (Gumbel-max) or with top-k / top-p, on the device, from the logits the LM-head GEMV left in
// memory. Same decision rule and the same counter-based random numbers as the reference's
// sampler (native/cuda/hf_decode_sequence/sampler.cu:18-33 hash and uniform, :89-156 greedy and
// Gumbel-max, :157-392 exact top-k by (value desc, index asc), softmax in that order, nucleus,
// one draw), so that a given (seed, position) picks the same token.
//
// gfx950 mapping: the reference runs one 1024-thread block over the whole vocabulary; here the
// vocabulary is cut into 1024-logit chunks, one workgroup each, and a second one-workgroup
// kernel finishes:
//   chunk kernel   greedy / Gumbel: best (score, index) of the chunk.
//                  top-k: the chunk's best logit as a 64-bit key (order-preserving value bits above the
//                  inverted index, so a plain integer order is (value desc, index asc)) and the number
//                  of its finite logits.
//   select kernel  greedy / Gumbel: best of the chunk candidates.
//                  top-k: the k-th largest of the chunks' best keys bounds the k-th largest key of the
//                  vocabulary from below, so one pass over the logits collects the keys at or above
//                  that bound - a few hundred when the logits are spread over the chunks - and each
//                  survivor finds its place by counting the survivors with a larger key. If more than 1024
//                  survive (logits piled into few chunks), the exact k-th largest key comes from a radix
//                  selection over the whole vocabulary (six digits, histogram in LDS, parallel suffix scan)
//                  instead. Then exponentials in parallel, one running sum in the rule's order by one
//                  lane, and the nucleus and the draw read from it by parallel searches.
//                  (The chunks used to sort their 1024 keys and hand out their best 128: 38 + 30-43 us for
//                  the two launches at 151936 logits, barrier-bound.)
//   then the token slot is written and the device cursor advanced, as the greedy finish does.
#pragma once

#include "gemv_stream.cuh"
#include "nerva_hip_api.h"

namespace nv {

enum : uint32_t { kSamplerGreedy = 0, kSamplerGumbel = 1, kSamplerTopK = 2 };
constexpr uint32_t kSamplerChunk = 1024;    // logits per chunk workgroup
constexpr uint32_t kSamplerTopKMax = 128;   // sampler.cu:12

// Sampler parameters as the kernels read them from device memory (one captured graph serves
// every non-greedy configuration).
struct SamplerDev {
  float temperature, top_p;
  uint32_t top_k, mode;
  uint64_t seed;
};

// sampler.cu:422-433 normalisation (a non-finite or negative temperature becomes 0, a top_p
// outside (0, 1] becomes 1) followed by the branch the kernel would take.
SamplerDev sampler_device_config(const NervaHipHfDecodeSamplerConfig &config);

inline uint32_t sampler_chunks(uint32_t vocab) { return (vocab + kSamplerChunk - 1) / kSamplerChunk; }
// Bytes of the chunk-candidate key buffer for a vocabulary.
uint64_t sampler_workspace_bytes(uint32_t vocab);

struct SamplerParams {
  const float *logits;
  uint32_t vocab;
  const SamplerDev *config;   // device memory
  uint64_t *keys;             // [chunks][kSamplerTopKMax] workspace (top-k: word 0 of a row the chunk's best key, word 1 its finite count)
  SampleParams out;           // chunk candidates (greedy / Gumbel), slot / cursor / plain token output
  const uint32_t *cursor;     // device position (slot index and random-number counter), or null -> position
  uint32_t position, max_steps;
};
// Both kernels on `stream`. vocab <= kSampleMaxBlocks * kSamplerChunk.
hipError_t launch_sampler(const SamplerParams &p, hipStream_t stream);
// The same two kernels for `count` sequences in one launch each: batch[i] (device memory) holds what
// launch_sampler takes for sequence i - its own logits, configuration, workspaces, slots and cursor.
// All of them over the same vocabulary size.
hipError_t launch_sampler_batch(const SamplerParams *batch, uint32_t count, uint32_t vocab, hipStream_t stream);

}  // namespace nv
