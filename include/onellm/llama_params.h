// src/models/llama/llama_params.h:2-15 restated.
#pragma once
struct LLaMAAttentionStaticParams {
    int   rotary_embedding_dim;
    float rotary_embedding_base;
    int   max_position_embeddings;  // read and ignored by the decode path
    bool  use_dynamic_ntk;          // read and ignored by the decode path
};

struct LLaMAAttentionDynParams {
    int batch_size;
    int num_tokens;
    int max_q_len;
    int max_k_len;
    int num_layers;
};
