// Host-side token selection from a row of fp16 logits: greedy argmax and the
// seeded top-k / min-p / top-p sampler.  Same contract as caml_llmopt_f16_argmax
// and caml_llmopt_sample_f16_native (native/ocaml_metal_stubs.m:2565-2765), which
// lib/sampling.ml:193-207 calls on the last logits row after suppression:
//
//  * greedy when temperature <= 1e-4 or top_k == 1: the first maximum of the row
//    in fp16 comparison order (a NaN never wins);
//  * otherwise the k = 64 (top_k == 0), top_k (1..256) or 256 (larger) best
//    tokens are kept by a bounded min-heap over one pass, listed best first,
//    weighted with exp((logit - best) / temperature) in float32, cut by min-p
//    (probability >= min_p * best probability, a prefix of the list) and top-p
//    (shortest prefix whose probability reaches top_p), and one token is drawn
//    with a xoroshiro128+ generator seeded from `seed` (0 = from the clock).
//
// Every float32 operation happens in the order the reference performs it and
// the heap breaks ties the same way, so a seed gives the same token.
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstring>

#include "../runtime.h"

namespace {

float half_to_float(uint16_t bits) {
  const uint32_t sign = (uint32_t)(bits & 0x8000u) << 16;
  const uint32_t exponent = (bits >> 10) & 0x1fu;
  uint32_t fraction = bits & 0x3ffu;
  uint32_t word;
  if (exponent == 0) {
    if (fraction == 0) {
      word = sign;
    } else {  // subnormal: renormalise
      int shift = 0;
      while ((fraction & 0x400u) == 0) {
        fraction <<= 1;
        ++shift;
      }
      word = sign | ((uint32_t)(113 - shift) << 23) | ((fraction & 0x3ffu) << 13);
    }
  } else if (exponent == 31) {
    word = sign | 0x7f800000u | (fraction << 13);
  } else {
    word = sign | ((exponent + 112) << 23) | (fraction << 13);
  }
  float value;
  std::memcpy(&value, &word, sizeof(value));
  return value;
}

// a > b in IEEE comparison order (false when either is NaN); fp16 -> fp32 is exact and monotonic
bool half_greater(uint16_t a, uint16_t b) { return half_to_float(a) > half_to_float(b); }

int64_t first_maximum(const uint16_t *logits, int64_t count) {
  int64_t best = 0;
  for (int64_t i = 1; i < count; ++i)
    if (half_greater(logits[i], logits[best])) best = i;
  return best;
}

struct Candidate {
  uint32_t token;
  float logit;
};

// Min-heap on the logit, at most 256 entries, the smallest kept candidate at the root.
class BoundedHeap {
 public:
  int size() const { return size_; }
  const Candidate &root() const { return items_[0]; }

  void push(Candidate item) {
    int at = size_++;
    items_[at] = item;
    while (at > 0) {  // a child strictly smaller than its parent moves up
      const int parent = (at - 1) / 2;
      if (!(items_[at].logit < items_[parent].logit)) break;
      swap(at, parent);
      at = parent;
    }
  }

  void replace_root(Candidate item) {
    items_[0] = item;
    settle(0);
  }

  Candidate pop() {
    const Candidate top = items_[0];
    items_[0] = items_[size_ - 1];
    --size_;
    settle(0);
    return top;
  }

 private:
  void swap(int a, int b) {
    const Candidate held = items_[a];
    items_[a] = items_[b];
    items_[b] = held;
  }
  // the entry sinks towards its smaller child; of two equal children the left one, and it
  // stays above a child it merely equals
  void settle(int at) {
    for (;;) {
      int least = at;
      const int left = 2 * at + 1, right = 2 * at + 2;
      if (left < size_ && items_[left].logit < items_[least].logit) least = left;
      if (right < size_ && items_[right].logit < items_[least].logit) least = right;
      if (least == at) return;
      swap(at, least);
      at = least;
    }
  }

  Candidate items_[256];
  int size_ = 0;
};

uint64_t rotate_left(uint64_t value, int bits) { return (value << bits) | (value >> (64 - bits)); }

// xoroshiro128+ with the 24 / 16 / 37 constants; the draw uses the top 53 bits
struct Generator {
  uint64_t s0, s1;
  uint64_t next() {
    const uint64_t result = s0 + s1;
    const uint64_t mixed = s1 ^ s0;
    s0 = rotate_left(s0, 24) ^ mixed ^ (mixed << 16);
    s1 = rotate_left(mixed, 37);
    return result;
  }
  float uniform() { return (float)(next() >> 11) * (1.0f / 9007199254740992.0f); }
};

}  // namespace

extern "C" int llmopt_hip_f16_argmax(const uint16_t *logits, int64_t count, int64_t *out_index) {
  if (out_index == nullptr) return llmopt::fail(LLMOPT_ERR_INVALID, "f16 argmax needs an output");
  if (count < 0 || (count > 0 && logits == nullptr))
    return llmopt::fail(LLMOPT_ERR_INVALID, "f16 argmax needs %lld logits", (long long)count);
  *out_index = count == 0 ? 0 : first_maximum(logits, count);
  return LLMOPT_OK;
}

extern "C" int llmopt_hip_sample_f16(const uint16_t *logits, int64_t count, double temperature, int64_t top_k,
                                     double top_p, double min_p, int64_t seed, int64_t *out_token) {
  if (out_token == nullptr) return llmopt::fail(LLMOPT_ERR_INVALID, "f16 sampling needs an output");
  if (count < 0 || (count > 0 && logits == nullptr))
    return llmopt::fail(LLMOPT_ERR_INVALID, "f16 sampling needs %lld logits", (long long)count);
  if (count == 0) {
    *out_token = 0;
    return LLMOPT_OK;
  }
  const float temp = (float)temperature;
  const float nucleus = (float)top_p;
  const float floor_ratio = (float)min_p;
  const int requested = (int)top_k;
  if (temp <= 0.0001f || requested == 1) {
    *out_token = first_maximum(logits, count);
    return LLMOPT_OK;
  }

  const int keep = requested <= 0 ? 64 : requested <= 256 ? requested : 256;
  BoundedHeap heap;
  for (int64_t i = 0; i < count; ++i) {
    const float value = half_to_float(logits[i]);
    if (heap.size() < keep)
      heap.push({(uint32_t)i, value});
    else if (value > heap.root().logit)
      heap.replace_root({(uint32_t)i, value});
  }

  // best first: the heap gives its candidates up smallest first
  Candidate ranked[256];
  const int candidates = heap.size();
  for (int i = candidates - 1; i >= 0; --i) ranked[i] = heap.pop();

  const float best = ranked[0].logit;
  const float inverse_temperature = 1.0f / temp;
  float weight[256];
  float total = 0.0f;
  for (int i = 0; i < candidates; ++i) {
    weight[i] = expf((ranked[i].logit - best) * inverse_temperature);
    total += weight[i];
  }

  int live = candidates;
  if (floor_ratio > 0.0f && total > 0.0f) {  // min-p: a prefix, since the list is sorted
    const float threshold = weight[0] / total * floor_ratio;
    float kept_total = 0.0f;
    int kept = 0;
    for (int i = 0; i < candidates; ++i) {
      if (!(weight[i] / total >= threshold)) break;
      kept_total += weight[i];
      ++kept;
    }
    if (kept > 0) {
      live = kept;
      total = kept_total;
    }
  }
  if (nucleus > 0.0f && nucleus < 1.0f && total > 0.0f) {  // top-p
    float cumulative = 0.0f, kept_total = 0.0f;
    int cut = live;
    for (int i = 0; i < live; ++i) {
      cumulative += weight[i] / total;
      kept_total += weight[i];
      if (cumulative >= nucleus) {
        cut = i + 1;
        break;
      }
    }
    live = cut;
    total = kept_total;
  }

  uint64_t state = (uint64_t)seed;
  if (state == 0)
    state = (uint64_t)std::chrono::steady_clock::now().time_since_epoch().count();
  Generator generator{state ^ 0x9E3779B97F4A7C15ull, (state << 31) | (state >> 33)};
  if (generator.s0 == 0 && generator.s1 == 0) generator = Generator{1, 2};

  const float target = generator.uniform() * total;
  float reached = 0.0f;
  uint32_t chosen = ranked[0].token;
  for (int i = 0; i < live; ++i) {
    reached += weight[i];
    if (reached >= target) {
      chosen = ranked[i].token;
      break;
    }
  }
  *out_token = (int64_t)chosen;
  return LLMOPT_OK;
}
