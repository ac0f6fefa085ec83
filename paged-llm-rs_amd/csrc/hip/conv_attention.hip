// What an attention layer with short convolutions does between its projections and the attention
// kernels: for every token and head, the convolution over the projected rows (with the request's
// carried history), the norm over a head of q and k, the rotation of the first `rot` values of a head
// (value i with value i + rot/2, angle position * freq[i]), and then q into the query buffer and k
// and v into the request's pages.  Heads are stored in rows of Dp values, zeros behind a head's own
// size, so that queries, keys and values of different sizes share the attention kernels' one head size.
// Convolution, norm, angles and rotation are 32-bit; a value is rounded once, when it is stored.
#include "common.hpp"

struct ConvQkArgs {
    const float* rows;        // [n, stride]: the projections, q | k | v from column `off`
    int stride, off;
    const float* conv_w;      // [taps, H*D + G*D + G*V]: a tap's filter values of all channels side by side
    int taps;
    const float* state;       // [slots, state_stride], the history at hist_off: [taps - 1][channels]
    long state_stride;
    int hist_off;
    const float* q_gain;      // [D]
    const float* k_gain;      // [D]
    float eps;
    const float* freq;        // [rot / 2], or null
    int rot;
    const int* positions;
    const int* seq_of;
    const int* q_start;
    const int* state_slots;
    const int* block_table;
    int max_blocks, block_size;
    void* q_out;              // [n, H * Dp]
    void* k_pool;             // [pages * block_size, G * Dp]
    void* v_pool;
    int H, G, D, V, Dp;
};

// Few tokens (decode steps): a wave a token and head, all of them at once.
template <typename T>
__global__ __launch_bounds__(64) void conv_qk_prepare_heads_kernel(ConvQkArgs a) {
    __shared__ float head[256];
    const int t = blockIdx.x, which = blockIdx.y, lane = threadIdx.x;
    const int pos = a.positions[t];
    if (pos < 0) return;
    const int s = a.seq_of[t];
    const int slot = a.state_slots[s];
    if (slot < 0) return;
    const int H = a.H, G = a.G, D = a.D, V = a.V, Dp = a.Dp;
    const int channels = H * D + G * D + G * V;
    // which head this wave prepares: a query head, a key head or a value head
    const int kind = which < H ? 0 : (which < H + G ? 1 : 2);
    const int index = kind == 0 ? which : (kind == 1 ? which - H : which - H - G);
    const int width = kind == 2 ? V : D;
    const int c0 = kind == 0 ? index * D : (kind == 1 ? H * D + index * D : H * D + G * D + index * V);
    const float* hist = a.state + static_cast<size_t>(slot) * a.state_stride + a.hist_off;
    const int r = t - a.q_start[s];

    float ss = 0.f;
    for (int e = lane; e < width; e += 64) {
        const int c = c0 + e;
        float acc = 0.f;
        for (int jt = 0; jt < a.taps; ++jt) {
            const int back = a.taps - 1 - jt;
            const int src = r - back;
            const float u = src >= 0 ? a.rows[static_cast<size_t>(t - back) * a.stride + a.off + c]
                                     : hist[static_cast<size_t>(a.taps - 1 + src) * channels + c];
            acc += a.conv_w[jt * channels + c] * u;
        }
        head[e] = acc;
        ss += acc * acc;
    }
    if (kind != 2) {
        ss = wave_sum(ss);
        const float inv = 1.f / sqrtf(ss / static_cast<float>(D) + a.eps);
        const float* gain = kind == 0 ? a.q_gain : a.k_gain;
        for (int e = lane; e < width; e += 64) head[e] = head[e] * inv * gain[e];
    }
    __syncthreads();

    T* dst;
    if (kind == 0) {
        dst = static_cast<T*>(a.q_out) + (static_cast<size_t>(t) * H + index) * Dp;
    } else {
        const int page = a.block_table[static_cast<size_t>(s) * a.max_blocks + pos / a.block_size];
        if (page < 0) return;
        const size_t row = static_cast<size_t>(page) * a.block_size + pos % a.block_size;
        dst = static_cast<T*>(kind == 1 ? a.k_pool : a.v_pool) + (row * G + index) * Dp;
    }
    const int half = a.rot / 2;
    for (int e = lane; e < Dp; e += 64) {
        float x = 0.f;
        if (e < width) {
            x = head[e];
            if (kind != 2 && e < a.rot) {
                const int i = e < half ? e : e - half;
                float sn, cs;
                sincosf(static_cast<float>(pos) * a.freq[i], &sn, &cs);
                x = e < half ? head[e] * cs - head[e + half] * sn : head[e] * cs + head[e - half] * sn;
            }
        }
        dst[e] = from_float<T>(x);
    }
}

// Many tokens (prompt portions): one workgroup a token; its waves take the token's heads (query, key and value heads alike) in turn, and
// the angles' cosines and sines are worked out once for the token.
template <typename T>
__global__ __launch_bounds__(256) void conv_qk_prepare_kernel(ConvQkArgs a) {
    __shared__ float heads[4][256];
    __shared__ float cs[128], sn[128];
    const int t = blockIdx.x, wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int pos = a.positions[t];
    if (pos < 0) return;
    const int s = a.seq_of[t];
    const int slot = a.state_slots[s];
    if (slot < 0) return;
    const int H = a.H, G = a.G, D = a.D, V = a.V, Dp = a.Dp;
    const int channels = H * D + G * D + G * V;
    const float* hist = a.state + static_cast<size_t>(slot) * a.state_stride + a.hist_off;
    const int r = t - a.q_start[s];
    const int half = a.rot / 2;
    for (int i = threadIdx.x; i < half; i += 256) sincosf(static_cast<float>(pos) * a.freq[i], &sn[i], &cs[i]);
    __syncthreads();
    int page_row = -1;
    {
        const int page = a.block_table[static_cast<size_t>(s) * a.max_blocks + pos / a.block_size];
        if (page >= 0) page_row = page * a.block_size + pos % a.block_size;
    }
    float* head = heads[wave];
    for (int base = 0; base < H + 2 * G; base += 4) {
        // which head this wave prepares now: a query head, a key head or a value head (the last round may leave
        // waves without one; they still meet the others at the barriers)
        const int which = base + wave;
        const bool busy = which < H + 2 * G;
        const int kind = which < H ? 0 : (which < H + G ? 1 : 2);
        const int index = kind == 0 ? which : (kind == 1 ? which - H : which - H - G);
        const int width = kind == 2 ? V : D;
        const int c0 = kind == 0 ? index * D : (kind == 1 ? H * D + index * D : H * D + G * D + index * V);
        float ss = 0.f;
        for (int e = lane; busy && e < width; e += 64) {
            const int c = c0 + e;
            float acc = 0.f;
            for (int jt = 0; jt < a.taps; ++jt) {
                const int back = a.taps - 1 - jt;
                const int src = r - back;
                const float u = src >= 0 ? a.rows[static_cast<size_t>(t - back) * a.stride + a.off + c]
                                         : hist[static_cast<size_t>(a.taps - 1 + src) * channels + c];
                acc += a.conv_w[jt * channels + c] * u;
            }
            head[e] = acc;
            ss += acc * acc;
        }
        if (busy && kind != 2) {
            ss = wave_sum(ss);
            const float inv = 1.f / sqrtf(ss / static_cast<float>(D) + a.eps);
            const float* gain = kind == 0 ? a.q_gain : a.k_gain;
            for (int e = lane; e < width; e += 64) head[e] = head[e] * inv * gain[e];
        }
        __syncthreads();
        T* dst = nullptr;
        if (!busy)
            dst = nullptr;
        else if (kind == 0)
            dst = static_cast<T*>(a.q_out) + (static_cast<size_t>(t) * H + index) * Dp;
        else if (page_row >= 0)
            dst = static_cast<T*>(kind == 1 ? a.k_pool : a.v_pool) + (static_cast<size_t>(page_row) * G + index) * Dp;
        if (dst != nullptr) {
            for (int e = lane; e < Dp; e += 64) {
                float x = 0.f;
                if (e < width) {
                    x = head[e];
                    if (kind != 2 && e < a.rot) {
                        const int i = e < half ? e : e - half;
                        x = e < half ? head[e] * cs[i] - head[e + half] * sn[i] : head[e] * cs[i] + head[e - half] * sn[i];
                    }
                }
                dst[e] = from_float<T>(x);
            }
        }
        __syncthreads();
    }
}

extern "C" int pl_conv_qk_prepare(const float* rows, int stride, int off, const float* conv_w, int taps,
                                  const float* state, long state_stride, int hist_off,
                                  const float* q_gain, const float* k_gain, float eps, const float* freq, int rot,
                                  const int* positions, const int* seq_of, const int* q_start, const int* state_slots,
                                  const int* block_table, int max_blocks, int block_size,
                                  void* q_out, void* k_pool, void* v_pool, int dtype,
                                  int n, int H, int G, int D, int V, int Dp, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && H > 0 && G > 0 && H % G == 0, "conv_qk_prepare: rows %d, %d query heads over %d key heads", n, H, G);
    PL_REQUIRE(D > 0 && V > 0 && Dp >= D && Dp >= V && Dp <= 256, "conv_qk_prepare: heads of %d and %d in rows of %d (up to 256)", D, V, Dp);
    PL_REQUIRE(taps >= 1 && taps <= 16, "conv_qk_prepare: %d taps", taps);
    PL_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D && (rot == 0 || freq != nullptr), "conv_qk_prepare: a rotation over %d of %d values", rot, D);
    PL_REQUIRE(block_size > 0 && max_blocks > 0, "conv_qk_prepare: pages of %d, tables of %d", block_size, max_blocks);
    if (n == 0) return 0;
    ConvQkArgs a{rows, stride, off, conv_w, taps, state, state_stride, hist_off, q_gain, k_gain, eps, freq, rot,
                 positions, seq_of, q_start, state_slots, block_table, max_blocks, block_size, q_out, k_pool, v_pool,
                 H, G, D, V, Dp};
    // (steps of few tokens are bound by the chain of one token's work, which a wave a head keeps shortest;
    // large steps by what they compute and read, where the angles once a token and the heads in rounds pay)
    const bool few = n < 512 && H + 2 * G <= 65535;
    const dim3 grid(n, H + 2 * G);
    if (dtype == PL_DTYPE_F32) {
        if (few) conv_qk_prepare_heads_kernel<float><<<grid, 64, 0, stream>>>(a);
        else conv_qk_prepare_kernel<float><<<n, 256, 0, stream>>>(a);
    } else if (dtype == PL_DTYPE_BF16) {
        if (few) conv_qk_prepare_heads_kernel<bf16_t><<<grid, 64, 0, stream>>>(a);
        else conv_qk_prepare_kernel<bf16_t><<<n, 256, 0, stream>>>(a);
    }
    else
        PL_REQUIRE(false, "conv_qk_prepare: dtype code %d", dtype);
    PL_CHECK_LAUNCH("conv_qk_prepare");
    return 0;
}
