// Where a LLaMA checkpoint keeps each weight, and the row order the attention kernels expect:
// the host-side mirror of adrastea_models/src/llama.rs:30-243.
//
//  * tensor addresses (llama.rs:30-58) and the two name tables: Meta's consolidated.*.pth
//    (llama.rs:121-169) and Hugging Face's pytorch_model-*.bin (llama.rs:70-119);
//  * MetaLlamaModelLoader / HuggingFaceLlamaModelLoader (llama.rs:171-243).  The Hugging Face
//    conversion stores the query and key projections with the two rotary halves of every head
//    de-interleaved; the loader puts the rows back in Meta's order, which is the order the
//    rotary embedding and QK^T of this code path assume.  The reference does that with an
//    elementwise copy on the device (llama.rs:216-236); here the rows are gathered while the
//    file's bytes are copied into the upload buffer, so the device sees one contiguous copy.
//
// A loaded tensor is host memory ready for the caller's hipMemcpy: either a view of the mapped
// file (no copy) or, for the re-ordered projections, an owned buffer.
#pragma once

#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "pickle.hpp"

namespace adrastea {

// llama.rs:30-58
enum class LlamaAttentionAddress { Query, Key, Value, Out };
enum class LlamaMLPAddress { Expand, Contract, Gate };

struct LlamaTransformerBlockAddress {
  enum Kind { AttentionNorm, Attention, MLPNorm, MLP } kind;
  LlamaAttentionAddress attention = LlamaAttentionAddress::Query;  // kind == Attention
  LlamaMLPAddress mlp = LlamaMLPAddress::Expand;                   // kind == MLP

  static LlamaTransformerBlockAddress attention_norm() { return {AttentionNorm}; }
  static LlamaTransformerBlockAddress mlp_norm() { return {MLPNorm}; }
  static LlamaTransformerBlockAddress of(LlamaAttentionAddress a) { return {Attention, a}; }
  static LlamaTransformerBlockAddress of(LlamaMLPAddress m) {
    return {MLP, LlamaAttentionAddress::Query, m};
  }
};

struct LlamaModelAddress {
  enum Kind { TokenEmbedding, OutputNorm, TokenProjection, Layer } kind;
  size_t layer = 0;                                                // kind == Layer
  LlamaTransformerBlockAddress block = LlamaTransformerBlockAddress::attention_norm();

  static LlamaModelAddress token_embedding() { return {TokenEmbedding}; }
  static LlamaModelAddress output_norm() { return {OutputNorm}; }
  static LlamaModelAddress token_projection() { return {TokenProjection}; }
  static LlamaModelAddress in_layer(size_t n, LlamaTransformerBlockAddress b) { return {Layer, n, b}; }
};

// llama.rs:70-119
struct HuggingFaceTensorNames {
  static std::string resolve(LlamaAttentionAddress a) {
    switch (a) {
      case LlamaAttentionAddress::Query: return "q_proj.weight";
      case LlamaAttentionAddress::Key: return "k_proj.weight";
      case LlamaAttentionAddress::Value: return "v_proj.weight";
      default: return "o_proj.weight";
    }
  }
  static std::string resolve(LlamaMLPAddress a) {
    switch (a) {
      case LlamaMLPAddress::Expand: return "up_proj.weight";
      case LlamaMLPAddress::Contract: return "down_proj.weight";
      default: return "gate_proj.weight";
    }
  }
  static std::string resolve(const LlamaTransformerBlockAddress& a) {
    switch (a.kind) {
      case LlamaTransformerBlockAddress::Attention: return "self_attn." + resolve(a.attention);
      case LlamaTransformerBlockAddress::MLP: return "mlp." + resolve(a.mlp);
      case LlamaTransformerBlockAddress::AttentionNorm: return "input_layernorm.weight";
      default: return "post_attention_layernorm.weight";
    }
  }
  static std::string resolve(const LlamaModelAddress& a) {
    switch (a.kind) {
      case LlamaModelAddress::TokenEmbedding: return "model.embed_tokens.weight";
      case LlamaModelAddress::OutputNorm: return "model.norm.weight";
      case LlamaModelAddress::TokenProjection: return "lm_head.weight";
      default: return "model.layers." + std::to_string(a.layer) + "." + resolve(a.block);
    }
  }
};

// llama.rs:121-169
struct MetaTensorNames {
  static std::string resolve(LlamaAttentionAddress a) {
    switch (a) {
      case LlamaAttentionAddress::Query: return "wq.weight";
      case LlamaAttentionAddress::Key: return "wk.weight";
      case LlamaAttentionAddress::Value: return "wv.weight";
      default: return "wo.weight";
    }
  }
  static std::string resolve(LlamaMLPAddress a) {
    switch (a) {
      case LlamaMLPAddress::Expand: return "w3.weight";
      case LlamaMLPAddress::Contract: return "w2.weight";
      default: return "w1.weight";
    }
  }
  static std::string resolve(const LlamaTransformerBlockAddress& a) {
    switch (a.kind) {
      case LlamaTransformerBlockAddress::Attention: return "attention." + resolve(a.attention);
      case LlamaTransformerBlockAddress::MLP: return "feed_forward." + resolve(a.mlp);
      case LlamaTransformerBlockAddress::AttentionNorm: return "attention_norm.weight";
      default: return "ffn_norm.weight";
    }
  }
  static std::string resolve(const LlamaModelAddress& a) {
    switch (a.kind) {
      case LlamaModelAddress::TokenEmbedding: return "tok_embeddings.weight";
      case LlamaModelAddress::OutputNorm: return "norm.weight";
      case LlamaModelAddress::TokenProjection: return "output.weight";
      default: return "layers." + std::to_string(a.layer) + "." + resolve(a.block);
    }
  }
};

// Host bytes of one weight, in the element order of (shape, stride), ready to be copied to the
// device as they are (what load_tensor's copy_from_slice sends, pickle.rs:322-338).
struct LoadedTensor {
  LoadedTensor() = default;
  LoadedTensor(LoadedTensor&&) = default;              // (a moved vector keeps its buffer, so
  LoadedTensor& operator=(LoadedTensor&&) = default;   //  `data` stays valid; copies would not)
  LoadedTensor(const LoadedTensor&) = delete;
  LoadedTensor& operator=(const LoadedTensor&) = delete;

  TensorDataType dtype = TensorDataType::F16;
  std::vector<size_t> shape, stride;
  const uint8_t* data = nullptr;   // `bytes` bytes: into the mapped file, or into `owned`
  size_t bytes = 0;
  std::vector<uint8_t> owned;      // empty when data points into the mapping
};

inline LoadedTensor view_of(const PickledModel& m, const PickledTensor& t) {
  LoadedTensor r;
  r.dtype = t.dtype;
  r.shape = t.shape;
  r.stride = t.stride;
  r.data = m.bytes(t);
  r.bytes = t.end - t.begin;
  return r;
}

// llama.rs:171-188
class MetaLlamaModelLoader {
 public:
  explicit MetaLlamaModelLoader(const PickledModel& model) : model_(model) {}
  LoadedTensor load_tensor(const LlamaModelAddress& address) const {
    return view_of(model_, model_.tensor(MetaTensorNames::resolve(address)));
  }

 private:
  const PickledModel& model_;
};

// The subset of LlamaParams (llama.rs:245-262) the loader reads.
struct LlamaLoaderParams {
  size_t dim, n_heads;
};

// llama.rs:190-243
class HuggingFaceLlamaModelLoader {
 public:
  HuggingFaceLlamaModelLoader(const ShardedModel& model, LlamaLoaderParams params)
      : model_(model), params_(params) {
    if (params.n_heads == 0 || params.dim % params.n_heads != 0 || (params.dim / params.n_heads) % 2 != 0)
      throw std::runtime_error("dim must be a multiple of 2 * n_heads");
  }

  LoadedTensor load_tensor(const LlamaModelAddress& address) const {
    const auto found = model_.find(HuggingFaceTensorNames::resolve(address));
    const bool qk = address.kind == LlamaModelAddress::Layer &&
                    address.block.kind == LlamaTransformerBlockAddress::Attention &&
                    (address.block.attention == LlamaAttentionAddress::Query ||
                     address.block.attention == LlamaAttentionAddress::Key);
    if (!qk) return view_of(*found.first, *found.second);
    return unpermute(*found.first, *found.second);
  }

 private:
  // The file's [dim, dim] matrix read as [n_heads, 2, half, dim] holds, for head h, first the
  // rows Meta keeps at even positions of the head and then those at odd positions.  The result,
  // read as [n_heads, half, 2, dim], is out[h][j][t][:] = in[h][t][j][:]: a contiguous row-major
  // [dim, dim] matrix whatever strides the file had (llama.rs:216-236).
  LoadedTensor unpermute(const PickledModel& m, const PickledTensor& t) const {
    const size_t dim = params_.dim, heads = params_.n_heads, head = dim / heads, half = head / 2;
    if (t.shape.size() != 2 || t.shape[0] != dim || t.shape[1] != dim)
      throw std::runtime_error("query/key projection is not [dim, dim]");
    const size_t el = element_size(t.dtype);
    LoadedTensor r;
    r.dtype = t.dtype;
    r.shape = {dim, dim};
    r.stride = {dim, 1};
    r.owned.resize(dim * dim * el);
    const uint8_t* src = m.bytes(t);   // the span covers every (row, column) of the record
    for (size_t h = 0; h < heads; h++)
      for (size_t j = 0; j < half; j++)
        for (size_t s = 0; s < 2; s++) {
          const size_t from = h * head + s * half + j, to = h * head + j * 2 + s;
          uint8_t* dst = r.owned.data() + to * dim * el;
          const uint8_t* row = src + from * t.stride[0] * el;
          if (t.stride[1] == 1) {
            std::memcpy(dst, row, dim * el);
          } else {
            for (size_t c = 0; c < dim; c++) std::memcpy(dst + c * el, row + c * t.stride[1] * el, el);
          }
        }
    r.data = r.owned.data();
    r.bytes = r.owned.size();
    return r;
  }

  const ShardedModel& model_;
  LlamaLoaderParams params_;
};

}  // namespace adrastea
