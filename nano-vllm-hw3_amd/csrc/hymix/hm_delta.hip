// Generalized delta rule: S <- diag(w) S - (a u)(u^T S) + k v^T per head, o = S^T r, with a float32 state S [D, D] per
// (state slot, head).  Three launches: the float32 inputs of the recurrence from the mixer's merged product (parallel
// over tokens), the recurrence (sequential over a portion's tokens, parallel over sequences, heads and value channels),
// and the per-head norm and output gate (parallel over tokens).
#include "hm_common.h"

namespace hm {

// One workgroup per (token, head), one thread per key channel.  prep[t, h] = decay | a*u | u | k | r, D floats each.
template <typename T>
__global__ void delta_prepare_kernel(const T* __restrict__ proj, int64_t row_stride, int r_off, int k_off, int a_off, int z_off,
                                     const T* __restrict__ w2, const T* __restrict__ w0, const T* __restrict__ a_bias, int rank,
                                     float decay_scale, float unit_eps, float* __restrict__ prep, int H, int D) {
    extern __shared__ float tz[];              // rank floats: tanh of the decay's inner projection
    __shared__ float red[16];
    const int64_t t = blockIdx.x;
    const int hd = blockIdx.y, i = threadIdx.x;
    const T* row = proj + (size_t)t * row_stride;
    for (int j = threadIdx.x; j < rank; j += blockDim.x) tz[j] = tanhf(to_f(row[z_off + j]));
    __syncthreads();
    const int c = hd * D + i;
    float k = 0.f, r = 0.f, a = 0.f, decay = 0.f;
    if (i < D) {
        k = to_f(row[k_off + c]);
        r = to_f(row[r_off + c]);
        a = sigmoid_f(to_f(row[a_off + c]) + to_f(a_bias[c]));
        float acc = 0.f;
        const T* wr = w2 + (size_t)c * rank;
        for (int j = 0; j < rank; ++j) acc += to_f(wr[j]) * tz[j];
        decay = expf(-decay_scale * sigmoid_f(acc + to_f(w0[c])));
    }
    const float ss = block_sum(k * k, red);
    if (i < D) {
        const float u = k / sqrtf(ss + unit_eps);
        float* out = prep + ((size_t)t * H + hd) * 5 * D + i;
        out[0] = decay;
        out[D] = a * u;
        out[2 * D] = u;
        out[3 * D] = k;
        out[4 * D] = r;
    }
}

// One wave per (sequence, head, 64 value channels); a thread owns one column of S (DK >= D key channels in registers).
// The five per-token vectors are staged in LDS (two buffers, one barrier per token) and read as broadcasts.
template <typename T, int DK>
__global__ __launch_bounds__(64) void delta_recurrence_kernel(const float* __restrict__ prep, const T* __restrict__ v,
                                                              int64_t v_stride, float* __restrict__ state,
                                                              const int32_t* __restrict__ qstart,
                                                              const int32_t* __restrict__ seq_pos0,
                                                              const int32_t* __restrict__ seq_slot, float* __restrict__ o,
                                                              int H, int D) {
    __shared__ float buf[2][5 * DK];
    const int b = blockIdx.x, hd = blockIdx.y;
    const int q0 = qstart[b], n = qstart[b + 1] - q0;
    if (n <= 0) return;
    const int lane = threadIdx.x;
    const int j = blockIdx.z * 64 + lane;
    const bool live = j < D;
    float* st = state + ((size_t)seq_slot[b] * H + hd) * (size_t)D * D;
    float s[DK];
    const bool fresh = seq_pos0[b] == 0;       // a sequence's first tokens: the state starts at zero, whatever the slot holds
#pragma unroll
    for (int i = 0; i < DK; ++i) s[i] = (!fresh && live && i < D) ? st[(size_t)i * D + j] : 0.f;

    auto stage = [&](int tok, int which) {     // rows beyond D are zero: they leave their registers at zero
        const float* src = prep + ((size_t)(q0 + tok) * H + hd) * 5 * D;
        for (int e = lane; e < 5 * DK; e += 64) {
            const int part = e / DK, i = e - part * DK;
            buf[which][e] = i < D ? src[part * D + i] : 0.f;
        }
    };
    stage(0, 0);
    __syncthreads();
    for (int tok = 0; tok < n; ++tok) {
        const int cur = tok & 1;
        if (tok + 1 < n) stage(tok + 1, cur ^ 1);
        const float* p = buf[cur];
        const float vj = live ? to_f(v[(size_t)(q0 + tok) * v_stride + hd * D + j]) : 0.f;
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < DK; ++i) dot += p[2 * DK + i] * s[i];
        float out = 0.f;
#pragma unroll
        for (int i = 0; i < DK; ++i) {
            s[i] = p[i] * s[i] - p[DK + i] * dot + p[3 * DK + i] * vj;
            out += s[i] * p[4 * DK + i];
        }
        if (live) o[((size_t)(q0 + tok) * H + hd) * D + j] = out;
        __syncthreads();
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < DK; ++i)
            if (i < D) st[(size_t)i * D + j] = s[i];
    }
}

template <typename T>
__global__ __launch_bounds__(64) void delta_gate_norm_kernel(const float* __restrict__ o, const T* __restrict__ g,
                                                             int64_t g_stride, const T* __restrict__ norm_w, float eps,
                                                             T* __restrict__ out, int H, int D) {
    const int64_t t = blockIdx.x;
    const int hd = blockIdx.y, lane = threadIdx.x;
    const float* orow = o + ((size_t)t * H + hd) * D;
    float ss = 0.f;
    for (int i = lane; i < D; i += 64) ss += orow[i] * orow[i];
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss / (float)D + eps);
    for (int i = lane; i < D; i += 64) {
        const int c = hd * D + i;
        out[(size_t)t * H * D + c] = from_f<T>(orow[i] * r * to_f(norm_w[c]) * sigmoid_f(to_f(g[(size_t)t * g_stride + c])));
    }
}

}  // namespace hm

using namespace hm;

extern "C" int hm_delta_prepare(int dtype, const void* proj, int64_t row_stride, int r_off, int k_off, int a_off, int z_off,
                                const void* w2, const void* w0, const void* a_bias, int rank, float decay_scale, float unit_eps,
                                float* prep, int64_t T, int H, int D, void* stream) {
    if (T < 0 || H < 1 || D < 1 || rank < 1 || r_off < 0 || k_off < 0 || a_off < 0 || z_off < 0 ||
        (T > 0 && (!proj || !w2 || !w0 || !a_bias || !prep))) {
        set_error("hm_delta_prepare: bad argument");
        return HM_EINVAL;
    }
    if (D > 256 || rank > 8192 || H > 65535) { set_error("hm_delta_prepare: dim <= 256, rank <= 8192, heads <= 65535"); return HM_ESHAPE; }
    if (T == 0) return HM_OK;
    dim3 grid((unsigned)T, (unsigned)H);
    const int threads = (D + 63) / 64 * 64;
    HM_DISPATCH(dtype, "hm_delta_prepare",
                hipLaunchKernelGGL(delta_prepare_kernel<DT>, grid, dim3(threads), (size_t)rank * 4, as_stream(stream),
                                   (const DT*)proj, row_stride, r_off, k_off, a_off, z_off, (const DT*)w2, (const DT*)w0,
                                   (const DT*)a_bias, rank, decay_scale, unit_eps, prep, H, D));
    HM_CHECK_LAUNCH("hm_delta_prepare");
    return HM_OK;
}

template <typename DT>
static int launch_recurrence(const float* prep, const void* v, int64_t v_stride, float* state, const int32_t* qstart,
                             const int32_t* seq_pos0, const int32_t* seq_slot, float* o, int B, int H, int D, hipStream_t s) {
    dim3 grid((unsigned)B, (unsigned)H, (unsigned)((D + 63) / 64));
#define HM_RECUR(DK)                                                                                                       \
    hipLaunchKernelGGL((delta_recurrence_kernel<DT, DK>), grid, dim3(64), 0, s, prep, (const DT*)v, v_stride, state, qstart, \
                       seq_pos0, seq_slot, o, H, D)
    if (D <= 32) HM_RECUR(32);
    else if (D <= 64) HM_RECUR(64);
    else if (D <= 128) HM_RECUR(128);
    else HM_RECUR(256);
#undef HM_RECUR
    return 0;
}

extern "C" int hm_delta_recurrence(int dtype, const float* prep, const void* v, int64_t v_stride, float* state,
                                   const int32_t* qstart, const int32_t* seq_pos0, const int32_t* seq_slot, float* o, int B,
                                   int H, int D, void* stream) {
    if (B < 0 || H < 1 || D < 1 || v_stride < (int64_t)H * D || (B > 0 && (!prep || !v || !state || !qstart || !seq_pos0 || !seq_slot || !o))) {
        set_error("hm_delta_recurrence: bad argument");
        return HM_EINVAL;
    }
    if (D > 256 || H > 65535) { set_error("hm_delta_recurrence: dim <= 256 and heads <= 65535"); return HM_ESHAPE; }
    if (B == 0) return HM_OK;
    HM_DISPATCH(dtype, "hm_delta_recurrence",
                launch_recurrence<DT>(prep, v, v_stride, state, qstart, seq_pos0, seq_slot, o, B, H, D, as_stream(stream)));
    HM_CHECK_LAUNCH("hm_delta_recurrence");
    return HM_OK;
}

extern "C" int hm_delta_gate_norm(int dtype, const float* o, const void* g, int64_t g_stride, const void* norm_w, float eps,
                                  void* out, int64_t T, int H, int D, void* stream) {
    if (T < 0 || H < 1 || D < 1 || g_stride < (int64_t)H * D || (T > 0 && (!o || !g || !norm_w || !out))) {
        set_error("hm_delta_gate_norm: bad argument");
        return HM_EINVAL;
    }
    if (H > 65535) { set_error("hm_delta_gate_norm: heads <= 65535"); return HM_ESHAPE; }
    if (T == 0) return HM_OK;
    dim3 grid((unsigned)T, (unsigned)H);
    HM_DISPATCH(dtype, "hm_delta_gate_norm",
                hipLaunchKernelGGL(delta_gate_norm_kernel<DT>, grid, dim3(64), 0, as_stream(stream), o, (const DT*)g, g_stride,
                                   (const DT*)norm_w, eps, (DT*)out, H, D));
    HM_CHECK_LAUNCH("hm_delta_gate_norm");
    return HM_OK;
}
