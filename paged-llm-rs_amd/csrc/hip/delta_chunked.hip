// Prompt portions through the gated delta rule in chunks of tokens.  For one head, with decays g_t,
// G_t = g_1 ... g_t inside a chunk, and S_0 the state before the chunk, the rule
//     S_t = g_t S_(t-1) + k_t u_t^T ,   u_t = beta_t (v_t - g_t S_(t-1)^T k_t)
// unrolls to  S_t = G_t S_0 + sum_{s<=t} (G_t / G_s) k_s u_s^T , and the u of a chunk solve
//     (I + M) U = R ,  M[t][s] = beta_t (G_t / G_s) (k_t . k_s) for s < t ,  R_t = beta_t (v_t - G_t S_0^T k_t) .
// `prepare` (every chunk and head at once) makes k and q unit vectors, and computes T = (I + M)^-1 by
// forward substitution and Aq[t][s] = (G_t / G_s) (q_t . k_s) for s <= t.  `walk` (one workgroup for a
// request, a head and 16 columns of the state) then goes through the chunks in order:
//     R = beta (V - G K S) ;  U = T R ;  O = G Q S + Aq U ;  S = G_L S + (K weighted by G_L / G_s)^T U .
// 32-bit throughout, on the vector units, sums in a fixed order.
#include "recurrent.hpp"

struct DeltaArgs {
    ScanArgs a;
    float* Kn;       // [chunks, H, C, Dr]  k as unit vectors, rows of Dr = D rounded up to 4
    float* Qn;       // [chunks, H, C, Dr]  q as unit vectors times D^-1/2
    float* Tm;       // [chunks, H, C, C]  (I + M)^-1
    float* Aq;       // [chunks, H, C, C]
    float* scal;     // [chunks, H, 3, C]  G_t; beta_t; G_L / G_t
};

// PER (4, 2 or 1) neighbouring values of a row of the column tile in LDS, in one read (the rows start on 32 bytes).
template <int PER>
__device__ __forceinline__ void read_run(const float* p, float* out) {
    if (PER == 4) {
        const float4 x = *reinterpret_cast<const float4*>(p);
        out[0] = x.x; out[1] = x.y; out[2] = x.z; out[3] = x.w;
    } else if (PER == 1) {
        out[0] = p[0];
    } else {
        const float2 x = *reinterpret_cast<const float2*>(p);
        out[0] = x.x; out[1] = x.y;
    }
}

template <int C>
__device__ __forceinline__ int delta_chunk_number(const ScanArgs& a, int s, int c) { return a.q_start[s] / C + s + c; }

template <int C>
__global__ __launch_bounds__(256) void delta_prepare_kernel(DeltaArgs da) {
    const ScanArgs& a = da.a;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int TT = C / 16;
    const int D = a.D, H = a.H;
    const int c = blockIdx.x, h = blockIdx.y, s = blockIdx.z;
    const int slot = a.state_slots[s], n = a.q_len[s];
    if (slot < 0 || n < a.below || c * C >= n) return;
    const int L = min(C, n - c * C), row0 = a.q_start[s] + c * C;
    const int g = h / (H / a.G);
    const size_t idx = static_cast<size_t>(delta_chunk_number<C>(a, s, c)) * H + h;
    const int Dq = ((D + 3) & ~3) + 4;
    float* qs = lds;                 // [C][Dq]
    float* ks = qs + C * Dq;         // [C][Dq]
    float* M = ks + C * Dq;          // [C][C + 1]
    float* bs = M + C * (C + 1);     // [C]
    float* be = bs + C;              // [C]
    float* nrm = be + C;             // [2 C]
    const int tid = threadIdx.x;
    for (int e = tid; e < C * Dq; e += 256) {
        const int t = e / Dq, i = e - t * Dq;
        float q = 0.f, k = 0.f;
        if (t < L && i < D) {
            const float* row = a.qkv + static_cast<size_t>(row0 + t) * a.qkv_stride;
            q = row[a.q_off + g * D + i];
            k = row[a.k_off + g * D + i];
        }
        qs[e] = q;
        ks[e] = k;
    }
    if (tid < C) {
        // a thread a token: beta, and the logarithm of the decay (summed up below)
        float beta = 0.f, log_decay = 0.f;
        if (tid < L) {
            const float* row = a.gates + static_cast<size_t>(row0 + tid) * a.gates_stride;
            beta = sigmoid_f(row[a.g1_off + h]);
            log_decay = -expf(a.p1[h]) * softplus_f(row[a.g2_off + h] + a.p2[h]);
        }
        bs[tid] = log_decay;
        be[tid] = beta;
    }
    __syncthreads();
    if (tid == 255) {
        float sum = 0.f;
        for (int t = 0; t < C; ++t) {
            sum += bs[t];
            bs[t] = sum;
        }
    }
    if (tid < 2 * C) {
        const float* x = (tid < C ? qs : ks) + (tid < C ? tid : tid - C) * Dq;
        float ss = 0.f;
        for (int i = 0; i < D; ++i) ss += x[i] * x[i];
        nrm[tid] = 1.f / sqrtf(ss + 1e-6f) * (tid < C ? 1.f / sqrtf(static_cast<float>(D)) : 1.f);
    }
    __syncthreads();
    for (int e = tid; e < C * Dq; e += 256) {
        const int t = e / Dq;
        qs[e] *= nrm[t];
        ks[e] *= nrm[C + t];
    }
    __syncthreads();
    // the unit vectors and the chunk's scalars go out for the walk
    const int Dr = Dq - 4;          // (rows of whole quads, zeros behind D: the walk fetches them in quads)
    float* Kn = da.Kn + idx * C * Dr;
    float* Qn = da.Qn + idx * C * Dr;
    for (int e = tid; e < C * Dr; e += 256) {
        const int t = e / Dr, i = e - t * Dr;
        Kn[e] = ks[t * Dq + i];
        Qn[e] = qs[t * Dq + i];
    }
    float* scal = da.scal + idx * 3 * C;
    if (tid < C) {
        scal[tid] = expf(bs[tid]);
        scal[C + tid] = be[tid];
        scal[2 * C + tid] = tid < L ? expf(bs[L - 1] - bs[tid]) : 0.f;
    }
    const int ty = tid / 16, tx = tid % 16;
    {
        float kk[TT][TT], qk[TT][TT];
#pragma unroll
        for (int i = 0; i < TT; ++i)
#pragma unroll
            for (int j = 0; j < TT; ++j) kk[i][j] = qk[i][j] = 0.f;
        for (int d = 0; d < Dq - 4; d += 4) {
            float4 qv[TT], kt[TT], kv[TT];
#pragma unroll
            for (int i = 0; i < TT; ++i) {
                qv[i] = *reinterpret_cast<const float4*>(qs + (ty + 16 * i) * Dq + d);
                kt[i] = *reinterpret_cast<const float4*>(ks + (ty + 16 * i) * Dq + d);
            }
#pragma unroll
            for (int j = 0; j < TT; ++j) kv[j] = *reinterpret_cast<const float4*>(ks + (tx + 16 * j) * Dq + d);
#pragma unroll
            for (int i = 0; i < TT; ++i)
#pragma unroll
                for (int j = 0; j < TT; ++j) {
                    kk[i][j] += kt[i].x * kv[j].x + kt[i].y * kv[j].y + kt[i].z * kv[j].z + kt[i].w * kv[j].w;
                    qk[i][j] += qv[i].x * kv[j].x + qv[i].y * kv[j].y + qv[i].z * kv[j].z + qv[i].w * kv[j].w;
                }
        }
        float* Aq = da.Aq + idx * C * C;
#pragma unroll
        for (int i = 0; i < TT; ++i)
#pragma unroll
            for (int j = 0; j < TT; ++j) {
                const int t = ty + 16 * i, u = tx + 16 * j;
                const float w = (u <= t && t < L) ? expf(bs[t] - bs[u]) : 0.f;
                M[t * (C + 1) + u] = u < t ? be[t] * w * kk[i][j] : 0.f;
                Aq[t * C + u] = w * qk[i][j];
            }
    }
    __syncthreads();
    // T = (I + M)^-1, a column a thread: T[t][j] = [t == j] - sum_{s < t} M[t][s] T[s][j]
    if (tid < C) {
        float col[C];
#pragma unroll
        for (int t = 0; t < C; ++t) {
            float val = t == tid ? 1.f : 0.f;
#pragma unroll
            for (int u = 0; u < t; ++u) val -= M[t * (C + 1) + u] * col[u];
            col[t] = val;
        }
        float* Tm = da.Tm + idx * C * C;
#pragma unroll
        for (int t = 0; t < C; ++t) Tm[t * C + tid] = col[t];
    }
}

// One workgroup: a request, a head, VT (16 or 8) columns of the state; the chunks in order.  What a chunk needs
// (its unit vectors, T, Aq, the columns of v, the scalars) is asked for while the chunk before is computed
// and waits in registers: with one workgroup a compute unit nothing else would hide the trip to memory.
template <int C, int VT>
__global__ __launch_bounds__(256) void delta_walk_kernel(DeltaArgs da) {
    const ScanArgs& a = da.a;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int D = a.D, V = a.V, H = a.H;
    const int v0 = blockIdx.x * VT, h = blockIdx.y, s = blockIdx.z;
    const int slot = a.state_slots[s], n = a.q_len[s];
    if (slot < 0 || n < a.below) return;
    const int chunks = (n + C - 1) / C;
    const int Dr = (D + 3) & ~3, Dq = Dr + 4;
    float* qs = lds;                 // [C][Dq]
    float* ks = qs + C * Dq;         // [C][Dq]
    float* Tm = ks + C * Dq;         // [C][C + 1]
    float* Aq = Tm + C * (C + 1);    // [C][C + 1]
    float* S = Aq + C * (C + 1);     // [Dr][VT]
    float* Vt = S + Dr * VT;         // [C][VT]
    float* R = Vt + C * VT;          // [C][VT]
    float* U = R + C * VT;           // [C][VT]
    float* sc = U + C * VT;          // [3][C]
    const int tid = threadIdx.x;
    float* Sg = a.state + static_cast<size_t>(slot) * a.state_stride + a.s_off + static_cast<size_t>(h) * D * V;
    for (int e = tid; e < Dr * VT; e += 256) {
        const int d = e / VT, v = v0 + e % VT;
        S[e] = (d < D && v < V) ? Sg[static_cast<size_t>(d) * V + v] : 0.f;
    }
    const int first = delta_chunk_number<C>(a, s, 0);
    // a thread's row and columns in the products with C rows: row t, columns vq .. vq + PER - 1
    constexpr int GROUPS = 256 / C, PER = VT / GROUPS;             // threads a row, columns a thread
    static_assert(PER == 4 || PER == 2 || PER == 1, "a thread takes 4, 2 or 1 columns");
    const int t_row = tid / GROUPS, vq = (tid % GROUPS) * PER;
    const int row_bound = (tid / 64 + 1) * (64 / GROUPS);          // one past the last row of this thread's wave

    // what a thread fetches of a chunk: up to KQ quads of k and of q, TA quads of T and of Aq, VS values of v
    constexpr int KQ = 8, TA = C * C / 4 / 256 > 0 ? C * C / 4 / 256 : 1, VS = C * VT / 256;
    const int quads_row = Dr / 4, kq_quads = C * quads_row;
    int kq_at[KQ];
#pragma unroll
    for (int r = 0; r < KQ; ++r) {
        const int f = tid + 256 * r;
        kq_at[r] = f < kq_quads ? (f / quads_row) * Dq + (f % quads_row) * 4 : -1;
    }
    float4 kreg[KQ], qreg[KQ], treg[TA], areg[TA];
    float vreg[VS], sreg = 0.f;
    auto fetch = [&](int c) {
        const size_t idx = static_cast<size_t>(first + c) * H + h;
        const float4* Kn = reinterpret_cast<const float4*>(da.Kn + idx * C * Dr);
        const float4* Qn = reinterpret_cast<const float4*>(da.Qn + idx * C * Dr);
#pragma unroll
        for (int r = 0; r < KQ; ++r)
            if (kq_at[r] >= 0) {
                kreg[r] = Kn[tid + 256 * r];
                qreg[r] = Qn[tid + 256 * r];
            }
        const float4* Tg = reinterpret_cast<const float4*>(da.Tm + idx * C * C);
        const float4* Ag = reinterpret_cast<const float4*>(da.Aq + idx * C * C);
#pragma unroll
        for (int r = 0; r < TA; ++r)
            if (tid + 256 * r < C * C / 4) {
                treg[r] = Tg[tid + 256 * r];
                areg[r] = Ag[tid + 256 * r];
            }
        const int L = min(C, n - c * C), row0 = a.q_start[s] + c * C;
#pragma unroll
        for (int r = 0; r < VS; ++r) {
            const int e = tid + 256 * r, t = e / VT, v = v0 + e % VT;
            vreg[r] = (t < L && v < V) ? a.qkv[static_cast<size_t>(row0 + t) * a.qkv_stride + a.v_off + h * V + v] : 0.f;
        }
        if (tid < 3 * C) sreg = da.scal[idx * 3 * C + tid];
    };
    auto stash = [&]() {
#pragma unroll
        for (int r = 0; r < KQ; ++r)
            if (kq_at[r] >= 0) {
                *reinterpret_cast<float4*>(ks + kq_at[r]) = kreg[r];
                *reinterpret_cast<float4*>(qs + kq_at[r]) = qreg[r];
            }
#pragma unroll
        for (int r = 0; r < TA; ++r) {
            const int f = tid + 256 * r;
            if (f < C * C / 4) {
                const int at = (f / (C / 4)) * (C + 1) + (f % (C / 4)) * 4;
                Tm[at] = treg[r].x; Tm[at + 1] = treg[r].y; Tm[at + 2] = treg[r].z; Tm[at + 3] = treg[r].w;
                Aq[at] = areg[r].x; Aq[at + 1] = areg[r].y; Aq[at + 2] = areg[r].z; Aq[at + 3] = areg[r].w;
            }
        }
#pragma unroll
        for (int r = 0; r < VS; ++r) Vt[tid + 256 * r] = vreg[r];
        if (tid < 3 * C) sc[tid] = sreg;
    };
    fetch(0);
    for (int c = 0; c < chunks; ++c) {
        const int L = min(C, n - c * C), row0 = a.q_start[s] + c * C;
        __syncthreads();
        stash();
        __syncthreads();
        if (c + 1 < chunks) fetch(c + 1);
        // K S and Q S for the thread's row
        float ksum[PER], qsum[PER];
#pragma unroll
        for (int j = 0; j < PER; ++j) ksum[j] = qsum[j] = 0.f;
#pragma unroll 4
        for (int d = 0; d < Dr; d += 4) {
            const float4 k4 = *reinterpret_cast<const float4*>(ks + t_row * Dq + d);
            const float4 q4 = *reinterpret_cast<const float4*>(qs + t_row * Dq + d);
            const float kd[4] = {k4.x, k4.y, k4.z, k4.w}, qd[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
            for (int dd = 0; dd < 4; ++dd) {
                float sv[PER];
                read_run<PER>(S + (d + dd) * VT + vq, sv);
#pragma unroll
                for (int j = 0; j < PER; ++j) {
                    ksum[j] += kd[dd] * sv[j];
                    qsum[j] += qd[dd] * sv[j];
                }
            }
        }
        const float gam = sc[t_row], beta = sc[C + t_row];
#pragma unroll
        for (int j = 0; j < PER; ++j) R[t_row * VT + vq + j] = beta * (Vt[t_row * VT + vq + j] - gam * ksum[j]);
        __syncthreads();
        float us[PER];
#pragma unroll
        for (int j = 0; j < PER; ++j) us[j] = 0.f;
        // (T and Aq are zero above the diagonal: a wave walks up to its last row's diagonal, the same for all its lanes)
#pragma unroll 8
        for (int u = 0; u < row_bound; ++u) {
            const float w = Tm[t_row * (C + 1) + u];
            float rv[PER];
            read_run<PER>(R + u * VT + vq, rv);
#pragma unroll
            for (int j = 0; j < PER; ++j) us[j] += w * rv[j];
        }
#pragma unroll
        for (int j = 0; j < PER; ++j) U[t_row * VT + vq + j] = us[j];
        __syncthreads();
        float os[PER];
#pragma unroll
        for (int j = 0; j < PER; ++j) os[j] = gam * qsum[j];
#pragma unroll 8
        for (int u = 0; u < row_bound; ++u) {
            const float w = Aq[t_row * (C + 1) + u];
            float uv[PER];
            read_run<PER>(U + u * VT + vq, uv);
#pragma unroll
            for (int j = 0; j < PER; ++j) os[j] += w * uv[j];
        }
        if (t_row < L) {
#pragma unroll
            for (int j = 0; j < PER; ++j)
                if (v0 + vq + j < V)
                    a.out[static_cast<size_t>(row0 + t_row) * (H * V) + h * V + v0 + vq + j] = os[j];
        }
        // S = G_L S + sum_s (G_L / G_s) k_s u_s^T : a thread owns a row d of S and half of its columns
        const float gl = sc[L - 1];
        constexpr int HALF = VT / 2;
        for (int d = tid / 2; d < Dr; d += 128) {
            const int half = (tid & 1) * HALF;
            float acc[HALF];
#pragma unroll
            for (int j = 0; j < HALF; ++j) acc[j] = gl * S[d * VT + half + j];
#pragma unroll 8
            for (int u = 0; u < C; ++u) {           // (rows behind L hold zeros in U)
                const float kw = ks[u * Dq + d] * sc[2 * C + u];
                float uv[HALF];
#pragma unroll
                for (int j = 0; j < HALF; j += 4) read_run<4>(U + u * VT + half + j, uv + j);
#pragma unroll
                for (int j = 0; j < HALF; ++j) acc[j] += kw * uv[j];
            }
#pragma unroll
            for (int j = 0; j < HALF; ++j) S[d * VT + half + j] = acc[j];
        }
    }
    __syncthreads();
    for (int e = tid; e < Dr * VT; e += 256) {
        const int d = e / VT, v = v0 + e % VT;
        if (d < D && v < V) Sg[static_cast<size_t>(d) * V + v] = S[e];
    }
}

template <int C, int VT>
static int launch_delta_walk(const DeltaArgs& da, int seqs, hipStream_t stream) {
    const ScanArgs& a = da.a;
    const int Dr = (a.D + 3) & ~3, Dq = Dr + 4;
    const size_t lds_w = (2 * static_cast<size_t>(C) * Dq + 2 * C * (C + 1) + Dr * VT + 3 * C * VT + 3 * C) * sizeof(float);
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&delta_walk_kernel<C, VT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_w));
    PL_REQUIRE(e == hipSuccess, "delta_chunked: %zu bytes of LDS refused: %s", lds_w, hipGetErrorString(e));
    delta_walk_kernel<C, VT><<<dim3(pl_ceil_div(a.V, VT), a.H, seqs), 256, lds_w, stream>>>(da);
    PL_CHECK_LAUNCH("delta_chunked (walk)");
    return 0;
}

template <int C>
static int launch_delta(const DeltaArgs& da, int seqs, int max_q_len, hipStream_t stream) {
    const ScanArgs& a = da.a;
    const int Dq = ((a.D + 3) & ~3) + 4;
    const size_t lds_p = (2 * static_cast<size_t>(C) * Dq + C * (C + 1) + 4 * C) * sizeof(float);
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&delta_prepare_kernel<C>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_p));
    PL_REQUIRE(e == hipSuccess, "delta_chunked: %zu bytes of LDS refused: %s", lds_p, hipGetErrorString(e));
    delta_prepare_kernel<C><<<dim3(pl_ceil_div(max_q_len, C), a.H, seqs), 256, lds_p, stream>>>(da);
    PL_CHECK_LAUNCH("delta_chunked (prepare)");
    // A request's chunks are a chain, so the walk has heads x tiles of columns workgroups a request and no more:
    // tiles of 8 columns where tiles of 16 would leave half of the chip's compute units without one.
    if (a.H * pl_ceil_div(a.V, 16) * 2 <= pl_compute_units()) return launch_delta_walk<C, 8>(da, seqs, stream);
    return launch_delta_walk<C, 16>(da, seqs, stream);
}

// The requests of the step that bring at least `from` tokens.  Kn, Qn: room for (rows / chunk + requests)
// chunks of H * chunk * (D rounded up to 4) floats; Tm, Aq: of H * chunk * chunk; scal: of H * 3 * chunk.
extern "C" int pl_delta_chunked(const float* qkv, int qkv_stride, int q_off, int k_off, int v_off,
                                const float* gates, int gates_stride, int g1_off, int g2_off,
                                const float* a_log, const float* dt_bias,
                                float* state, long state_stride, float* out,
                                const int* q_start, const int* q_len, const int* state_slots,
                                int seqs, int max_q_len, int H, int G, int D, int V, int from,
                                float* Kn, float* Qn, float* Tm, float* Aq, float* scal, hipStream_t stream) {
    PL_REQUIRE(H > 0 && G > 0 && H % G == 0 && D > 0 && D <= 256 && V > 0 && from >= 1,
               "delta_chunked: %d heads over %d of q and k, %d by %d, from %d tokens", H, G, D, V, from);
    PL_REQUIRE(gates != nullptr && a_log != nullptr && dt_bias != nullptr, "delta_chunked: the gates are missing");
    PL_REQUIRE(Kn != nullptr && Qn != nullptr && Tm != nullptr && Aq != nullptr && scal != nullptr, "delta_chunked: no room for the chunks");
    PL_REQUIRE(seqs >= 0 && seqs <= 65535 && H <= 65535, "delta_chunked: %d requests, %d heads", seqs, H);
    if (seqs == 0 || max_q_len < from) return 0;
    DeltaArgs da{{qkv, qkv_stride, q_off, k_off, v_off, gates, gates_stride, g1_off, g2_off, a_log, dt_bias, 0.f, state,
                  state_stride, 0, 0, 0, out, q_start, q_len, state_slots, H, G, D, V, from},
                 Kn, Qn, Tm, Aq, scal};
    return D <= 128 ? launch_delta<64>(da, seqs, max_q_len, stream) : launch_delta<32>(da, seqs, max_q_len, stream);
}
