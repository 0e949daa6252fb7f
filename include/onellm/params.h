// Parameter carriers of the decode path, as the oneLLM layers and examples construct them:
//   LLaMAAttentionStaticParams, LLaMAAttentionDynParams   <- src/models/llama/llama_params.h:2-15
//   IntDict, floatDict                                      <- src/utils/params.h:4-5
#pragma once
#include <string>
#include <unordered_map>

// Fixed for the lifetime of a model.  Aggregate-initialised in this order by the callers
// ({rotary_embedding_dim, rotary_embedding_base, max_position_embeddings, use_dynamic_ntk}).
struct LLaMAAttentionStaticParams {
    int   rotary_embedding_dim;     // pairs (2i, 2i+1) with 2i below this are rotated; may exceed the head size
    float rotary_embedding_base;    // 10000 for LLaMA-2
    int   max_position_embeddings;  // carried, not used by the decode path
    bool  use_dynamic_ntk;          // carried, not used by the decode path
};

// Per call.  Only the layers read it; the launchers take their sizes from tensor shapes.
struct LLaMAAttentionDynParams {
    int batch_size;
    int num_tokens;
    int max_q_len;
    int max_k_len;
    int num_layers;
};

// string-keyed scalars handed to launchSampling ("vocab_size", "step", "end_id")
using IntDict   = std::unordered_map<std::string, int>;
using floatDict = std::unordered_map<std::string, float>;
