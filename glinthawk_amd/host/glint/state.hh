// The reader side of the reference's BatchedInferenceState (models/common/state.hh:157-338,596-648):
// the batch metadata and per-prompt fields the model driver reads and writes, plus the three host
// buffers (activations, queries, kvs).  Splitting, merging and the wire format belong to the
// networking layer and are not part of this backend.
#pragma once

#include <cstdint>
#include <cstring>
#include <vector>

#include "glint/config.hh"
#include "glint/types.hh"

namespace glint {

struct PromptData
{
  bool active { false };
  ContextID context_id {};
  uint32_t token {};
  uint32_t token_pos {};
  uint8_t temperature {}; // compact: value / 255.0f
  uint32_t prompt_length {};
  uint32_t max_completion_length {};
  bool finished { false };
  int8_t kv_tier { -1 };
  uint8_t kv_rank { 0 };
};

// host buffer with the DataBuffer surface the driver uses (models/types.hh:78-125)
class DataBuffer
{
  std::vector<uint8_t> bytes_ {};

public:
  DataBuffer() = default;
  explicit DataBuffer( size_t n )
    : bytes_( n )
  {
  }
  uint64_t len() const { return bytes_.size(); }
  uint8_t* data() { return bytes_.data(); }
  const uint8_t* data() const { return bytes_.data(); }
};

template<typename Config>
requires ModelConfig<Config>
class BatchedInferenceState
{
  uint32_t batch_size_ {};
  DataType dtype_ { DataType::Float32 };
  uint32_t next_layer_ { 0 };
  InferenceStage next_stage_ { InferenceStage::PreAttention };
  bool has_activations_ { false }, has_queries_ { false }, has_kvs_ { false };
  std::vector<PromptData> prompts_ {};
  DataBuffer activations_ {}, queries_ {}, kvs_ {};

  size_t activation_len() const { return Config::dim * DataTypeSize( dtype_ ); }
  size_t q_len() const { return Config::dim * DataTypeSize( dtype_ ); }
  size_t kv_len() const { return 2 * Config::kv_dim * DataTypeSize( dtype_ ); }

public:
  using ConfigType = Config;

  BatchedInferenceState() = default;
  BatchedInferenceState( uint32_t batch_size, DataType dtype )
    : batch_size_( batch_size )
    , dtype_( dtype )
    , prompts_( batch_size )
  {
  }

  bool empty() const { return batch_size_ == 0; }
  uint32_t batch_size() const { return batch_size_; }
  DataType dtype() const { return dtype_; }
  uint32_t next_layer() const { return next_layer_; }
  InferenceStage next_stage() const { return next_stage_; }
  bool has_activations() const { return has_activations_; }
  bool has_queries() const { return has_queries_; }
  bool has_kvs() const { return has_kvs_; }
  void set_next_layer( uint32_t l ) { next_layer_ = l; }
  void set_next_stage( InferenceStage s ) { next_stage_ = s; }

  void set_prompt( size_t i, ContextID context_id, uint32_t token, uint32_t token_pos, float temperature, uint32_t prompt_length,
                   uint32_t max_completion_length, int8_t kv_tier = 0, uint8_t kv_rank = 0 )
  {
    auto& p = prompts_[i];
    p.context_id = context_id;
    p.token = token;
    p.token_pos = token_pos;
    p.temperature = static_cast<uint8_t>( temperature * 255.0f );
    p.prompt_length = prompt_length;
    p.max_completion_length = max_completion_length;
    p.finished = false;
    p.active = true;
    p.kv_tier = kv_tier;
    p.kv_rank = kv_rank;
  }

  ContextID context_id( size_t i ) const { return prompts_[i].context_id; }
  uint32_t token( size_t i ) const { return prompts_[i].token; }
  uint32_t token_pos( size_t i ) const { return prompts_[i].token_pos; }
  uint32_t prompt_length( size_t i ) const { return prompts_[i].prompt_length; }
  uint32_t max_completion_length( size_t i ) const { return prompts_[i].max_completion_length; }
  float temperature( size_t i ) const { return prompts_[i].temperature / 255.0f; }
  bool finished( size_t i ) const { return prompts_[i].finished; }
  bool active( size_t i ) const { return prompts_[i].active; }

  void set_token( size_t i, uint32_t token ) { prompts_[i].token = token; }
  void set_token_pos( size_t i, uint32_t pos ) { prompts_[i].token_pos = pos; }
  void set_finished( size_t i ) { prompts_[i].finished = true; }
  void set_context_id( size_t i, ContextID id ) { prompts_[i].context_id = id; }

  // keeps the slot's context id and placement so that a refill inherits the same context
  void discard( size_t i )
  {
    const auto context_id = prompts_[i].context_id;
    const auto kv_tier = prompts_[i].kv_tier;
    const auto kv_rank = prompts_[i].kv_rank;
    prompts_[i] = {};
    prompts_[i].context_id = context_id;
    prompts_[i].kv_tier = kv_tier;
    prompts_[i].kv_rank = kv_rank;
    prompts_[i].active = false;
  }

  bool check_finished( size_t i ) const
  {
    const auto& p = prompts_[i];
    const bool saw_end = p.max_completion_length == 0 && ( p.token == Config::token_eos || p.token == Config::token_eot );
    const bool out_of_seq = p.token_pos >= Config::seq_len;
    const bool end_of_gen = p.max_completion_length > 0 && p.token_pos >= p.max_completion_length + p.prompt_length;
    return saw_end || out_of_seq || end_of_gen;
  }

  DataBuffer& activations() { return activations_; }
  DataBuffer& queries() { return queries_; }
  DataBuffer& kvs() { return kvs_; }
  const DataBuffer& activations() const { return activations_; }
  const DataBuffer& queries() const { return queries_; }
  const DataBuffer& kvs() const { return kvs_; }
  uint8_t* kv( size_t i ) { return kvs_.data() + i * kv_len(); }
  const uint8_t* kv( size_t i ) const { return kvs_.data() + i * kv_len(); }

  void allocate_activations()
  {
    activations_ = DataBuffer( batch_size_ * activation_len() );
    has_activations_ = true;
  }
  void allocate_queries()
  {
    queries_ = DataBuffer( batch_size_ * q_len() );
    has_queries_ = true;
  }
  void allocate_kvs()
  {
    kvs_ = DataBuffer( batch_size_ * kv_len() );
    has_kvs_ = true;
  }
  void deallocate_activations()
  {
    activations_ = {};
    has_activations_ = false;
  }
  void deallocate_queries()
  {
    queries_ = {};
    has_queries_ = false;
  }
  void deallocate_kvs()
  {
    kvs_ = {};
    has_kvs_ = false;
  }
};

} // namespace glint
