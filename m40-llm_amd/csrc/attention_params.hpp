// Launch parameters shared by the dense attention kernels (attention.hip, attention_mfma.hip).
#pragma once

#include "common.hpp"

struct AttnParams {
    const uint16_t* K;
    const uint16_t* V;
    const float* Q;
    float* Out;
    float* ws;                    // partials: [batch][q_heads][nchunks][hd + 2]
    const uint32_t* seq_ids_dev;  // may be null
    const uint32_t* seq_lens_dev; // may be null
    uint32_t seq_id, seq_len;
    uint32_t max_seq_len, kv_heads, q_heads, window;
    uint32_t chunk, nchunks;
    uint32_t subgroups;           // q-head subgroups per kv head
    uint32_t len_bias;            // added to a device-side length (position -> length)
    uint32_t max_batch;           // device-side sequence ids at or above this are skipped (0 = not checked)
    uint32_t span_limit;          // tokens a row may attend (the length bound the grid and chunking were sized for): rows
                                  // whose device-side length asks for more are skipped
};

// attention_mfma.hip: chunks of `p.chunk` tokens (a multiple of 128), G <= 8 q heads per workgroup
void m40_launch_attn_mfma(hipStream_t stream, const AttnParams& p, uint32_t head_dim, uint32_t batch);
