// Prompt portions through the mixers whose state decays by one number a token and head (linear
// attention with a fixed decay; the matrix memory with exponential gates), in chunks of tokens instead
// of token by token.  With a = log decay of a token, w = log weight of its write, b_t = a_1 + ... + a_t
// inside a chunk and S_0 the state before the chunk,
//     S_t = e^(b_t) S_0 + sum_{s<=t} e^(b_t - b_s + w_s) k_s v_s^T ,
// so a chunk's effect on the state is one weighted sum of outer products (`summary`, every chunk at
// once), the states before the chunks follow from those by a short walk over the chunks (`carry`), and
// a chunk's read-outs are (Q K^T, weighted and masked) V + (scaled Q) S_0 (`output`, every chunk at once).
// For the matrix memory the running maximum m_t = b_t + max(m_0, max_{s<=t}(w_s - b_s)) keeps every
// exponent at or below zero, and is the very sequence the token-by-token form walks through.
// All arithmetic is 32-bit on the vector units; the sums are taken in a fixed order.
#include "recurrent.hpp"

struct ChunkArgs {
    ScanArgs a;
    float* U;        // [chunks, H, D, V]  a chunk's weighted sum of k v^T
    float* Uk;       // [chunks, H, D]     ... of k (the matrix memory's normaliser)
    float* Sin;      // [chunks, H, D, V]  the state before a chunk
    float* nin;      // [chunks, H, D]
    float* scal;     // [chunks, H, 4]     b at the chunk's end; max of w_s - b_s; m before the chunk
};

// A request's chunks have numbers of their own among all chunks of the step: requests lie one behind the
// other in the step's rows, so q_start / C + (index of the request) + (chunk in the request) is unique.
template <int C>
__device__ __forceinline__ int chunk_number(const ScanArgs& a, int s, int c) { return a.q_start[s] / C + s + c; }

// The gates of the tokens of one chunk, a thread a token: a (log decay) into b, w (log weight of the write) into g.
// `sum_gates` then turns b into its running sum and g into w - b.
template <int KIND>
__device__ __forceinline__ void token_gates(const ScanArgs& a, int h, int row, float* b, float* g) {
    if (KIND == PL_SCAN_LIGHTNING) {
        *b = logf(a.p1[h]);
        *g = 0.f;
    } else {
        const float* gates = a.gates + static_cast<size_t>(row) * a.gates_stride;
        *g = a.cap * tanhf((gates[a.g1_off + h] + a.p1[h]) / a.cap);
        *b = logsigmoid_f(a.cap * tanhf((gates[a.g2_off + h] + a.p2[h]) / a.cap));
    }
}

// One thread, after a barrier behind token_gates.
__device__ __forceinline__ void sum_gates(int L, float* b, float* g) {
    float sum = 0.f;
    for (int t = 0; t < L; ++t) {
        sum += b[t];
        b[t] = sum;
        g[t] -= sum;
    }
}

template <int KIND>
__device__ __forceinline__ void load_qk(const ScanArgs& a, const float* row, int h, int i, float scale, float& q, float& k) {
    q = row[a.q_off + h * a.D + i];
    k = row[a.k_off + h * a.D + i];
    if (KIND == PL_SCAN_LIGHTNING) { q = silu_f(q); k = silu_f(k); }
    if (KIND == PL_SCAN_MLSTM) q *= scale;
}

// ---- summary: U = sum_s e^(b_L - b_s + w_s - M) k_s v_s^T for one chunk, head and tile of 64 columns ----
template <int KIND, int C, int DR>
__global__ __launch_bounds__(256) void chunk_summary_kernel(ChunkArgs ca) {
    const ScanArgs& a = ca.a;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int D = a.D, V = a.V, H = a.H;
    const int tiles = (V + 63) / 64;
    const int c = blockIdx.x, h = blockIdx.y / tiles, vt = blockIdx.y % tiles, s = blockIdx.z;
    const int slot = a.state_slots[s], n = a.q_len[s];
    if (slot < 0 || n < a.below || c * C >= n) return;
    const int L = min(C, n - c * C), row0 = a.q_start[s] + c * C;
    const int idx = chunk_number<C>(a, s, c) * H + h;
    float* ks = lds;                 // [C][D]
    float* vs = ks + C * D;          // [C][64]
    float* bs = vs + C * 64;         // [C]
    float* ws = bs + C;              // [C]
    const int tid = threadIdx.x;
    for (int e = tid; e < L * D; e += 256) {
        const int t = e / D, i = e - t * D;
        float q, k;
        load_qk<KIND>(a, a.qkv + static_cast<size_t>(row0 + t) * a.qkv_stride, h, i, 1.f, q, k);
        ks[e] = k;
    }
    for (int e = tid; e < L * 64; e += 256) {
        const int t = e / 64, j = vt * 64 + (e & 63);
        float v = j < V ? a.qkv[static_cast<size_t>(row0 + t) * a.qkv_stride + a.v_off + h * V + j] : 0.f;
        if (KIND == PL_SCAN_LIGHTNING) v = silu_f(v);
        vs[e] = v;
    }
    if (tid < L) token_gates<KIND>(a, h, row0 + tid, bs + tid, ws + tid);
    __syncthreads();
    if (tid == 0) {
        sum_gates(L, bs, ws);
        const float end = bs[L - 1];
        float most = ws[0];
        for (int t = 1; t < L; ++t) most = fmaxf(most, ws[t]);
        if (KIND == PL_SCAN_LIGHTNING) most = -end;          // (no stabiliser: the weights are e^(b_L - b_s) themselves)
        for (int t = 0; t < L; ++t) ws[t] = expf(ws[t] - most);
        if (vt == 0) {
            ca.scal[idx * 4 + 0] = end;
            ca.scal[idx * 4 + 1] = most;
            // the m that the request's first chunk starts from: the carry reads it here, not in the slot it writes
            if (KIND == PL_SCAN_MLSTM && c == 0)
                ca.scal[idx * 4 + 2] = a.state[static_cast<size_t>(slot) * a.state_stride + a.m_off + h * tiles];
        }
    }
    __syncthreads();
    const int ty = tid / 16, tx = tid % 16;
    float acc[DR][4];
#pragma unroll
    for (int i = 0; i < DR; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int t = 0; t < L; ++t) {
        float vv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) vv[j] = ws[t] * vs[t * 64 + tx + 16 * j];
#pragma unroll
        for (int i = 0; i < DR; ++i) {
            const int d = ty + 16 * i;
            const float kk = d < D ? ks[t * D + d] : 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] += kk * vv[j];
        }
    }
    float* U = ca.U + static_cast<size_t>(idx) * D * V;
#pragma unroll
    for (int i = 0; i < DR; ++i) {
        const int d = ty + 16 * i;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int v = vt * 64 + tx + 16 * j;
            if (d < D && v < V) U[static_cast<size_t>(d) * V + v] = acc[i][j];
        }
    }
    if (KIND == PL_SCAN_MLSTM && vt == 0) {
        for (int d = tid; d < D; d += 256) {
            float sum = 0.f;
            for (int t = 0; t < L; ++t) sum += ws[t] * ks[t * D + d];
            ca.Uk[static_cast<size_t>(idx) * D + d] = sum;
        }
    }
}

// ---- carry: the state before every chunk, and the request's state after its last ----
template <int KIND, int C>
__global__ __launch_bounds__(256) void chunk_carry_kernel(ChunkArgs ca) {
    const ScanArgs& a = ca.a;
    const int D = a.D, V = a.V, H = a.H;
    const int h = blockIdx.y, s = blockIdx.z;
    const int slot = a.state_slots[s], n = a.q_len[s];
    if (slot < 0 || n < a.below) return;
    const int chunks = (n + C - 1) / C;
    const int e = blockIdx.x * 256 + threadIdx.x;
    const size_t DV = static_cast<size_t>(D) * V;
    float* slot_state = a.state + static_cast<size_t>(slot) * a.state_stride;
    const bool element = e < D * V;
    // the normaliser's D values ride along in the first workgroup's first threads (after the matrix's)
    const bool of_n = KIND == PL_SCAN_MLSTM && blockIdx.x == 0 && e < D;
    const int tiles = (V + 63) / 64;       // (n and m have a copy a tile of columns in the slot; all are equal)
    const int first = chunk_number<C>(a, s, 0);
    float S = element ? slot_state[a.s_off + h * DV + e] : 0.f;
    float nv = of_n ? slot_state[a.n_off + static_cast<size_t>(h) * tiles * D + e] : 0.f;
    float m = KIND == PL_SCAN_MLSTM ? ca.scal[(static_cast<size_t>(first) * H + h) * 4 + 2] : 0.f;
    for (int c = 0; c < chunks; ++c) {
        const size_t idx = static_cast<size_t>(first + c) * H + h;
        const float u = element ? ca.U[idx * DV + e] : 0.f;
        const float uk = of_n ? ca.Uk[idx * D + e] : 0.f;
        const float end = ca.scal[idx * 4 + 0], most = ca.scal[idx * 4 + 1];
        if (element) ca.Sin[idx * DV + e] = S;
        if (of_n) ca.nin[idx * D + e] = nv;
        if (KIND == PL_SCAN_LIGHTNING) {
            S = expf(end) * S + u;
        } else {
            if (c > 0 && blockIdx.x == 0 && threadIdx.x == 0) ca.scal[idx * 4 + 2] = m;
            const float top = fmaxf(m, most);
            const float keep = expf(m - top), add = expf(most - top);
            S = keep * S + add * u;
            nv = keep * nv + add * uk;
            m = end + top;
        }
    }
    if (element) slot_state[a.s_off + h * DV + e] = S;
    if (of_n)
        for (int t = 0; t < tiles; ++t) slot_state[a.n_off + (static_cast<size_t>(h) * tiles + t) * D + e] = nv;
    if (KIND == PL_SCAN_MLSTM && blockIdx.x == 0 && threadIdx.x < tiles) slot_state[a.m_off + h * tiles + threadIdx.x] = m;
}

// ---- output: the read-outs of one chunk, head and tile of 64 columns ----
template <int KIND, int C>
__global__ __launch_bounds__(256) void chunk_output_kernel(ChunkArgs ca) {
    const ScanArgs& a = ca.a;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int TT = C / 16;
    const int D = a.D, V = a.V, H = a.H;
    const int tiles = (V + 63) / 64;
    const int c = blockIdx.x, h = blockIdx.y / tiles, vt = blockIdx.y % tiles, s = blockIdx.z;
    const int slot = a.state_slots[s], n = a.q_len[s];
    if (slot < 0 || n < a.below || c * C >= n) return;
    const int L = min(C, n - c * C), row0 = a.q_start[s] + c * C;
    const size_t idx = static_cast<size_t>(chunk_number<C>(a, s, c)) * H + h;
    const int Dq = ((D + 3) & ~3) + 4;       // a row of q or k in LDS: whole quads, and a quad of slack between rows
    float* qs = lds;                 // [C][Dq]
    float* ks = qs + C * Dq;         // [C][Dq]
    float* vs = ks + C * Dq;         // [C][64]
    float* A = vs + C * 64;          // [C][C + 1]
    float* bs = A + C * (C + 1);     // [C]  b_t
    float* gs = bs + C;              // [C]  w_s - b_s
    float* cm = gs + C;              // [C]  max(m_0, max_{s<=t} g_s)          (matrix memory)
    float* es = cm + C;              // [C]  what multiplies (S_0^T q_t)
    float* dn = es + C;              // [C]  1 / denominator                    (matrix memory)
    const int tid = threadIdx.x;
    const float q_scale = 1.f / sqrtf(static_cast<float>(D));
    for (int e = tid; e < C * Dq; e += 256) {
        const int t = e / Dq, i = e - t * Dq;
        float q = 0.f, k = 0.f;
        if (t < L && i < D) load_qk<KIND>(a, a.qkv + static_cast<size_t>(row0 + t) * a.qkv_stride, h, i, q_scale, q, k);
        qs[e] = q;
        ks[e] = k;
    }
    for (int e = tid; e < C * 64; e += 256) {
        const int t = e / 64, j = vt * 64 + (e & 63);
        float v = 0.f;
        if (t < L && j < V) {
            v = a.qkv[static_cast<size_t>(row0 + t) * a.qkv_stride + a.v_off + h * V + j];
            if (KIND == PL_SCAN_LIGHTNING) v = silu_f(v);
        }
        vs[e] = v;
    }
    if (tid < L) token_gates<KIND>(a, h, row0 + tid, bs + tid, gs + tid);
    __syncthreads();
    if (tid == 0) {
        sum_gates(L, bs, gs);
        if (KIND == PL_SCAN_MLSTM) {
            float top = ca.scal[idx * 4 + 2];
            for (int t = 0; t < L; ++t) {
                top = fmaxf(top, gs[t]);
                cm[t] = top;
            }
        }
    }
    __syncthreads();
    if (tid < L) es[tid] = KIND == PL_SCAN_LIGHTNING ? expf(bs[tid]) : expf(ca.scal[idx * 4 + 2] - cm[tid]);
    __syncthreads();
    const int ty = tid / 16, tx = tid % 16;
    {
        // A[t][s] = (q_t . k_s) times the weight of token s in token t's state, for s <= t
        float acc[TT][TT];
#pragma unroll
        for (int i = 0; i < TT; ++i)
#pragma unroll
            for (int j = 0; j < TT; ++j) acc[i][j] = 0.f;
        for (int d = 0; d < Dq - 4; d += 4) {
            float4 qv[TT], kv[TT];
#pragma unroll
            for (int i = 0; i < TT; ++i) qv[i] = *reinterpret_cast<const float4*>(qs + (ty + 16 * i) * Dq + d);
#pragma unroll
            for (int j = 0; j < TT; ++j) kv[j] = *reinterpret_cast<const float4*>(ks + (tx + 16 * j) * Dq + d);
#pragma unroll
            for (int i = 0; i < TT; ++i)
#pragma unroll
                for (int j = 0; j < TT; ++j)
                    acc[i][j] += qv[i].x * kv[j].x + qv[i].y * kv[j].y + qv[i].z * kv[j].z + qv[i].w * kv[j].w;
        }
#pragma unroll
        for (int i = 0; i < TT; ++i)
#pragma unroll
            for (int j = 0; j < TT; ++j) {
                const int t = ty + 16 * i, u = tx + 16 * j;
                float w = 0.f;
                if (u <= t && t < L)
                    w = KIND == PL_SCAN_LIGHTNING ? expf(bs[t] - bs[u]) : expf(gs[u] - cm[t]);
                A[t * (C + 1) + u] = acc[i][j] * w;
            }
    }
    __syncthreads();
    if (KIND == PL_SCAN_MLSTM && tid < L) {
        // n_t . q_t = (weights' row sum) + e_t (n_0 . q_t); the denominator max(|n . q|, e^(-m_t)) + 1e-6
        const int t = tid;
        float sum = 0.f;
        for (int u = 0; u <= t; ++u) sum += A[t * (C + 1) + u];
        float dot = 0.f;
        const float* n0 = ca.nin + idx * D;
        for (int d = 0; d < D; ++d) dot += n0[d] * qs[t * Dq + d];
        const float nq = sum + es[t] * dot;
        dn[t] = 1.f / (fmaxf(fabsf(nq), expf(-(bs[t] + cm[t]))) + 1e-6f);
    }
    float within[TT][4], before[TT][4];
#pragma unroll
    for (int i = 0; i < TT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) within[i][j] = before[i][j] = 0.f;
    for (int u = 0; u < L; ++u) {
        float vv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) vv[j] = vs[u * 64 + tx + 16 * j];
#pragma unroll
        for (int i = 0; i < TT; ++i) {
            const float w = A[(ty + 16 * i) * (C + 1) + u];
#pragma unroll
            for (int j = 0; j < 4; ++j) within[i][j] += w * vv[j];
        }
    }
    const float* S0 = ca.Sin + idx * D * V;
    if (C == 64) {
        // The tile of S_0 (D rows of 64 columns) goes through LDS, where k lay (nobody reads k behind the barrier
        // above, and C rows of Dq hold D rows of 64): all its loads are on their way at once.
        float* St = ks;
        for (int e = tid; e < D * 64; e += 256) {
            const int d = e / 64, v = vt * 64 + (e & 63);
            St[e] = v < V ? S0[static_cast<size_t>(d) * V + v] : 0.f;
        }
        __syncthreads();
#pragma unroll 4
        for (int d = 0; d < D; ++d) {
            float sv[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) sv[j] = St[d * 64 + tx + 16 * j];
#pragma unroll
            for (int i = 0; i < TT; ++i) {
                const float q = qs[(ty + 16 * i) * Dq + d];
#pragma unroll
                for (int j = 0; j < 4; ++j) before[i][j] += q * sv[j];
            }
        }
    } else {
        int col[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) col[j] = min(vt * 64 + tx + 16 * j, V - 1);
        for (int d = 0; d < D; ++d) {
            float sv[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) sv[j] = S0[static_cast<size_t>(d) * V + col[j]];
#pragma unroll
            for (int i = 0; i < TT; ++i) {
                const float q = qs[(ty + 16 * i) * Dq + d];
#pragma unroll
                for (int j = 0; j < 4; ++j) before[i][j] += q * sv[j];
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TT; ++i) {
        const int t = ty + 16 * i;
        if (t >= L) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int v = vt * 64 + tx + 16 * j;
            if (v >= V) continue;
            float o = within[i][j] + es[t] * before[i][j];
            if (KIND == PL_SCAN_MLSTM) o *= dn[t];
            a.out[static_cast<size_t>(row0 + t) * (H * V) + h * V + v] = o;
        }
    }
}

template <int KIND, int C>
static int launch_chunked(const ChunkArgs& ca, int seqs, int max_q_len, hipStream_t stream) {
    const ScanArgs& a = ca.a;
    const int chunks = pl_ceil_div(max_q_len, C), tiles = pl_ceil_div(a.V, 64);
    PL_REQUIRE(static_cast<long long>(a.H) * tiles <= 65535 && seqs <= 65535, "recurrent_chunked: %d heads of %d columns, %d requests", a.H, a.V, seqs);
    const dim3 grid(chunks, a.H * tiles, seqs);
    const size_t lds_a = (static_cast<size_t>(C) * a.D + C * 64 + 2 * C) * sizeof(float);
    const int Dq = ((a.D + 3) & ~3) + 4;
    const size_t lds_c = (2 * static_cast<size_t>(C) * Dq + C * 64 + C * (C + 1) + 5 * C) * sizeof(float);
#define PL_SUMMARY(DR)                                                                                                  \
    do {                                                                                                                \
        if (lds_a > 48 * 1024) {                                                                                        \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&chunk_summary_kernel<KIND, C, DR>),       \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_a));    \
            PL_REQUIRE(e == hipSuccess, "recurrent_chunked: %zu bytes of LDS refused: %s", lds_a, hipGetErrorString(e)); \
        }                                                                                                               \
        chunk_summary_kernel<KIND, C, DR><<<grid, 256, lds_a, stream>>>(ca);                                            \
    } while (0)
    if (a.D <= 32) PL_SUMMARY(2);
    else if (a.D <= 64) PL_SUMMARY(4);
    else if (a.D <= 128) PL_SUMMARY(8);
    else PL_SUMMARY(16);
#undef PL_SUMMARY
    PL_CHECK_LAUNCH("recurrent_chunked (summary)");
    chunk_carry_kernel<KIND, C><<<dim3(pl_ceil_div(a.D * a.V, 256), a.H, seqs), 256, 0, stream>>>(ca);
    PL_CHECK_LAUNCH("recurrent_chunked (carry)");
    if (lds_c > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&chunk_output_kernel<KIND, C>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_c));
        PL_REQUIRE(e == hipSuccess, "recurrent_chunked: %zu bytes of LDS refused: %s", lds_c, hipGetErrorString(e));
    }
    chunk_output_kernel<KIND, C><<<grid, 256, lds_c, stream>>>(ca);
    PL_CHECK_LAUNCH("recurrent_chunked (output)");
    return 0;
}

// How many tokens a chunk has for heads of q and k of size D (the longer rows of large heads leave LDS for fewer).
extern "C" int pl_recurrent_chunk_tokens(int D) { return D <= 128 ? 64 : 32; }

// The requests of the step that bring at least `from` tokens; the others are the token-by-token kernel's.
// U, Sin: room for (rows / chunk + requests) chunks of H * D * V floats; Uk, nin: of H * D; scal: of H * 4.
extern "C" int pl_recurrent_chunked(int kind, const float* qkv, int qkv_stride, int q_off, int k_off, int v_off,
                                    const float* gates, int gates_stride, int g1_off, int g2_off,
                                    const float* p1, const float* p2, float cap,
                                    float* state, long state_stride, int s_off, int n_off, int m_off,
                                    float* out, const int* q_start, const int* q_len, const int* state_slots,
                                    int seqs, int max_q_len, int H, int D, int V, int from,
                                    float* U, float* Uk, float* Sin, float* nin, float* scal, hipStream_t stream) {
    PL_REQUIRE(kind == PL_SCAN_LIGHTNING || kind == PL_SCAN_MLSTM, "recurrent_chunked: kind %d", kind);
    PL_REQUIRE(H > 0 && D > 0 && D <= 256 && V > 0 && from >= 1, "recurrent_chunked: %d heads of %d by %d, from %d tokens", H, D, V, from);
    PL_REQUIRE(p1 != nullptr && (kind == PL_SCAN_LIGHTNING || (gates != nullptr && p2 != nullptr && cap > 0.f)),
               "recurrent_chunked: the gates of kind %d are missing", kind);
    PL_REQUIRE(U != nullptr && Sin != nullptr && scal != nullptr && (kind == PL_SCAN_LIGHTNING || (Uk != nullptr && nin != nullptr)),
               "recurrent_chunked: no room for the chunks' sums");
    if (seqs == 0 || max_q_len < from) return 0;
    ChunkArgs ca{{qkv, qkv_stride, q_off, k_off, v_off, gates, gates_stride, g1_off, g2_off, p1, p2, cap, state, state_stride,
                  s_off, n_off, m_off, out, q_start, q_len, state_slots, H, H, D, V, from},
                 U, Uk, Sin, nin, scal};
    if (D <= 128) {
        return kind == PL_SCAN_LIGHTNING ? launch_chunked<PL_SCAN_LIGHTNING, 64>(ca, seqs, max_q_len, stream)
                                         : launch_chunked<PL_SCAN_MLSTM, 64>(ca, seqs, max_q_len, stream);
    }
    return kind == PL_SCAN_LIGHTNING ? launch_chunked<PL_SCAN_LIGHTNING, 32>(ca, seqs, max_q_len, stream)
                                     : launch_chunked<PL_SCAN_MLSTM, 32>(ca, seqs, max_q_len, stream);
}
