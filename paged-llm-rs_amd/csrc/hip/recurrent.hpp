// Shared by the kernels of the mixers that carry a matrix of state: what a launch is told, and the
// gates' functions, all 32-bit.
#pragma once

#include "common.hpp"

#define PL_SCAN_LIGHTNING 0
#define PL_SCAN_MLSTM 1
#define PL_SCAN_DELTA 2

struct ScanArgs {
    const float* qkv;         // rows holding q, k and v (for the delta rule: already convolved and activated)
    int qkv_stride, q_off, k_off, v_off;
    const float* gates;       // rows holding the two pre-activations of the gates (mlstm: i, f; delta: beta, a)
    int gates_stride, g1_off, g2_off;
    const float* p1;          // lightning: decay a head; mlstm: bias of i; delta: A_log
    const float* p2;          // mlstm: bias of f; delta: dt_bias
    float cap;                // mlstm: the cap of the gates' pre-activations
    float* state;             // [slots, state_stride]
    long state_stride;
    int s_off, n_off, m_off;  // where S [H, D, V], n [H, tiles, D] and m [H, tiles] start inside a slot (tiles of 64
                              // columns of V: every tile's wave keeps a copy of n and m of its own)
    float* out;               // [rows, H * V]
    const int* q_start;
    const int* q_len;
    const int* state_slots;
    int H, G, D, V;           // heads, heads of q and k (G divides H), size of q and k, size of v
    int below;                // the token-by-token kernel takes requests of fewer tokens than this (0: all);
                              // the chunked kernels take the others
};

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float logsigmoid_f(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }

