// The attention variants behind hfa_paged_attention.
#pragma once
#include <hip/hip_runtime.h>

struct AttnArgs {
    const void* q; int ldq;
    const void* k_cache; const void* v_cache; int kv_width;
    const int* block_table; int max_blocks;
    const int* token_slot; const int* positions; const int* q_start;
    int n_seqs, max_q_len, max_seq_len;
    void* out; int ldo;
    int n_tokens, n_heads, n_kv_heads, head_dim, page_tokens, window;
    float scale;
    void* workspace; size_t workspace_bytes;
    hipStream_t stream;
    // decoded tokens whose queries, new key and new value still lie in 32-bit rows [q | k | v] (see attn_mfma_kernel,
    // FUSED): raw is null otherwise
    const float* raw; int ld_raw;
    const float* cos_sin;          // [token][head_dim / 2 cosines, head_dim / 2 sines], null: no rotation
    const int* slot_map;           // the cache row of each token's key and value
    int mask_chunk;                // > 0: a query sees only the keys of its own run of mask_chunk positions, counted from 0
    int sink;                      // 1: the softmax's denominator holds one more term of score 0 that has no value
    int v_rot;                     // the weights of a head of group c are applied to the values of group (c + v_rot) mod G (0: its own)
    float softcap;                 // > 0 (with weights 1 only): score <- softcap tanh(score / softcap)
    int weights;                   // 0: softmax; 1: sigmoid(score + head_bias[head]), not normalised over the keys
    const float* head_bias;        // one number a query head, or null
};

// The first key that the query at `pos` sees: a window of the last `window` positions (0: none) and/or the start
// of the query's own masking chunk (0: none). It never falls as pos grows.
__host__ __device__ __forceinline__ int first_visible(int pos, int window, int mask_chunk) {
    int lo = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
    if (mask_chunk > 0) {
        const int c = pos - pos % mask_chunk;
        lo = c > lo ? c : lo;
    }
    return lo;
}

int attn_generic_launch(const void* q, int dtype, int ldq, const void* k_cache, const void* v_cache, int kv_width,
                        int v_width, const int* block_table, int max_blocks, const int* token_slot, const int* positions,
                        void* out, int ldo, int n_tokens, int n_heads, int n_kv_heads, int head_dim, int v_head_dim,
                        int page_tokens, int window, int mask_chunk, float scale, const float* slopes, int sink, int cross, float softcap,
                        int weights, const float* head_bias, hipStream_t stream);

// Single tokens of a mixer that mixes its heads' weights after the softmax: every head's weights on the values of every
// group in one pass over the cache, written in rounds of groups (see attention_cross.hip). `supports` leaves the cut
// of the keys that `launch` takes.
bool attn_cross_supports(const AttnArgs& a, int* chunk_keys, int* n_chunks);
int attn_cross_launch(const AttnArgs& a, int chunk_keys, int n_chunks);

// Many query heads on one key/value head with wide key rows and value rows of another size (attention through latents), bf16 on
// the matrix cores; see attention_shared.hip for what it needs.
bool attn_shared_supports(const AttnArgs& a, int v_head_dim, int v_width);
int attn_shared_launch(const AttnArgs& a, int v_head_dim);

// bf16 on the matrix cores; see attention_mfma.hip for what it needs.
bool attn_mfma_supports(const AttnArgs& a);
int attn_mfma_launch(const AttnArgs& a);
