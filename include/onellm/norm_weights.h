// src/weights/llama/norm_weights.h:2-4 restated.
#pragma once
struct LayerNormWeight {
    float* gamma;
};
