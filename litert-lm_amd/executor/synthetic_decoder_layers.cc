#include <cmath>

#include "decoder_layers.h"

namespace litert::lm {

std::vector<LayerTransform> SyntheticDecoderLayers::Transforms(const AttentionShape& shape) {
  std::vector<LayerTransform> out(shape.num_layers);
  const int d = shape.head_dim;
  for (int layer = 0; layer < shape.num_layers; ++layer) {
    LayerTransform& t = out[layer];
    t.norm_q = t.norm_k = true;
    t.eps = 1e-6f;
    t.weight_offset = 1.f;
    t.q_weight.resize(d);
    t.k_weight.resize(d);
    for (int c = 0; c < d; ++c) {
      t.q_weight[c] = 0.25f * Unit((uint32_t)layer * 0x9E3779B1U + (uint32_t)c * 0x85EBCA77U + 9U);
      t.k_weight[c] = 0.25f * Unit((uint32_t)layer * 0x9E3779B1U + (uint32_t)c * 0x85EBCA77U + 10U);
    }
    const bool local = !shape.layer_window.empty() && shape.layer_window[layer] > 0;
    const double theta = local ? 10000.0 : 1000000.0;
    t.rope_inv_freq.resize(d / 2);
    for (int i = 0; i < d / 2; ++i)
      t.rope_inv_freq[i] = static_cast<float>(1.0 / std::pow(theta, static_cast<double>(2 * i) / d));
  }
  return out;
}

Status SyntheticDecoderLayers::Begin(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions) {
  RET_CHECK_EQ(tokens.size(), positions.size());
  n_ = static_cast<int>(tokens.size());
  const int hidden = Hidden();
  state_.assign(static_cast<size_t>(n_) * hidden, 0.f);
  for (int t = 0; t < n_; ++t) {
    const uint32_t tok = static_cast<uint32_t>(tokens[t]), pos = static_cast<uint32_t>(positions[t]);
    for (int i = 0; i < hidden; ++i) {
      const uint32_t ui = static_cast<uint32_t>(i);
      state_[(size_t)t * hidden + i] =
          Unit(tok * 0x9E3779B1U + ui * 0x85EBCA77U + 1U) + 0.5f * Unit(pos * 0xC2B2AE3DU + ui * 0x27D4EB2FU + 2U);
    }
  }
  return OkStatus();
}

Status SyntheticDecoderLayers::ProjectQkv(int layer, float* q, float* k, float* v) {
  const int hidden = Hidden(), d = shape_.head_dim, hkv = shape_.num_kv_heads;
  const int group = shape_.num_q_heads / hkv;
  const uint32_t ul = static_cast<uint32_t>(layer);
  const float inv_group = 1.0f / static_cast<float>(group);
  for (int t = 0; t < n_; ++t) {
    const float* s = &state_[(size_t)t * hidden];
    for (int i = 0; i < hidden; ++i)
      q[(size_t)t * hidden + i] = s[i] * (1.0f + 0.5f * Unit(ul * 0x165667B1U + (uint32_t)i * 0x9E3779B1U + 3U));
    for (int kh = 0; kh < hkv; ++kh) {
      for (int c = 0; c < d; ++c) {
        float sum = 0.f;
        for (int j = 0; j < group; ++j) sum += s[(kh * group + j) * d + c];
        const float mean = sum * inv_group;
        const uint32_t idx = static_cast<uint32_t>(kh * d + c);
        k[((size_t)t * hkv + kh) * d + c] = mean * (1.0f + 0.5f * Unit(ul * 0x27D4EB2FU + idx * 0x165667B1U + 5U));
        v[((size_t)t * hkv + kh) * d + c] = mean * Unit(ul * 0x85EBCA77U + idx * 0xC2B2AE3DU + 6U) +
                                            0.25f * Unit(idx * 0x9E3779B1U + ul + 7U);
      }
    }
  }
  return OkStatus();
}

Status SyntheticDecoderLayers::ConsumeAttention(int layer, const float* attn) {
  const int hidden = Hidden();
  const uint32_t ul = static_cast<uint32_t>(layer);
  for (int t = 0; t < n_; ++t) {
    float* s = &state_[(size_t)t * hidden];
    double sq = 0.0;
    for (int i = 0; i < hidden; ++i) {
      s[i] = s[i] + attn[(size_t)t * hidden + i] * Unit(ul * 0xC2B2AE3DU + (uint32_t)i * 0x27D4EB2FU + 8U);
      sq += static_cast<double>(s[i]) * static_cast<double>(s[i]);
    }
    const float inv_rms = static_cast<float>(1.0 / std::sqrt(sq / hidden + 1e-6));
    for (int i = 0; i < hidden; ++i) s[i] = s[i] * inv_rms;
  }
  return OkStatus();
}

Status SyntheticDecoderLayers::Logits(float* logits) {
  RET_CHECK_GT(n_, 0);
  const int hidden = Hidden();
  const float* s = &state_[(size_t)(n_ - 1) * hidden];
  const double norm = 1.0 / std::sqrt(static_cast<double>(hidden));
  for (int vtok = 0; vtok < vocab_; ++vtok) {
    double acc = 0.0;
    for (int i = 0; i < hidden; ++i)
      acc += static_cast<double>(s[i]) *
             static_cast<double>(Unit((uint32_t)vtok * 0x2545F491U + (uint32_t)i * 0x61C88647U + 4U));
    logits[vtok] = static_cast<float>(acc * norm);
  }
  return OkStatus();
}

}  // namespace litert::lm
