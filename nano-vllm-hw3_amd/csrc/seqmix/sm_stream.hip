// Token embedding into S residual streams, and the per-sublayer step of a multi-stream residual
// (hyper-connections): mix the streams and add the sublayer's output, then read the next sublayer's input
// as a weighted sum of the streams and RMS-normalise it.  One workgroup per token; the streams are f32.
#include "sm_common.h"

namespace sm {

static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

template <typename T>
__global__ void embed_streams_kernel(const int64_t* __restrict__ ids, const int32_t* __restrict__ positions,
                                     const T* __restrict__ embed, const T* __restrict__ pos_table, float* __restrict__ X,
                                     int S, int W) {
    const int64_t t = blockIdx.x;
    const T* e = embed + (size_t)ids[t] * W;
    const T* p = pos_table ? pos_table + (size_t)positions[t] * W : nullptr;
    float* x = X + (size_t)t * S * W;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float v = to_f(e[c]) + (p ? to_f(p[c]) : 0.f);
        for (int s = 0; s < S; ++s) x[(size_t)s * W + c] = v;
    }
}

constexpr int kMaxStreams = 8;

template <typename T, int VEC>
__global__ __launch_bounds__(256) void stream_step_kernel(float* __restrict__ X, const T* __restrict__ y,
                                                          const float* __restrict__ mix, const float* __restrict__ out,
                                                          const float* __restrict__ w_in, const T* __restrict__ norm_w,
                                                          float eps, T* __restrict__ h_out, int S, int W) {
    extern __shared__ float u_lds[];           // W floats: the sublayer input before the norm
    __shared__ float red[16];
    __shared__ float p_mix[kMaxStreams * kMaxStreams], p_out[kMaxStreams], p_in[kMaxStreams];
    const int64_t t = blockIdx.x;
    const bool wr = y != nullptr, rd = h_out != nullptr;
    if (threadIdx.x < S * S && wr) p_mix[threadIdx.x] = mix[threadIdx.x];
    if (threadIdx.x < S) {
        if (wr) p_out[threadIdx.x] = out[threadIdx.x];
        if (rd) p_in[threadIdx.x] = w_in[threadIdx.x];
    }
    __syncthreads();
    float* x = X + (size_t)t * S * W;
    float ss = 0.f;
    // VEC channels per thread (VEC = 4: 16-byte accesses to the f32 streams)
    for (int c = threadIdx.x * VEC; c < W; c += blockDim.x * VEC) {
        float old[kMaxStreams][VEC];
        for (int s = 0; s < S; ++s) {
            if (VEC == 4) {
                const float4 v = *(const float4*)(x + (size_t)s * W + c);
                old[s][0] = v.x; old[s][1] = v.y; old[s][2] = v.z; old[s][VEC - 1] = v.w;
            } else {
                old[s][0] = x[(size_t)s * W + c];
            }
        }
        float u[VEC];
        for (int e = 0; e < VEC; ++e) u[e] = 0.f;
        if (wr) {
            float yv[VEC];
            for (int e = 0; e < VEC; ++e) yv[e] = to_f(y[(size_t)t * W + c + e]);
            for (int r = 0; r < S; ++r) {
                float acc[VEC];
                for (int e = 0; e < VEC; ++e) {
                    float a = 0.f;
                    for (int s = 0; s < S; ++s) a += p_mix[s * S + r] * old[s][e];
                    a += p_out[r] * yv[e];
                    acc[e] = a;
                    if (rd) u[e] += p_in[r] * a;
                }
                if (VEC == 4) *(float4*)(x + (size_t)r * W + c) = make_float4(acc[0], acc[1], acc[2], acc[VEC - 1]);
                else x[(size_t)r * W + c] = acc[0];
            }
        } else if (rd) {
            for (int s = 0; s < S; ++s)
                for (int e = 0; e < VEC; ++e) u[e] += p_in[s] * old[s][e];
        }
        if (rd) {
            for (int e = 0; e < VEC; ++e) {
                u_lds[c + e] = u[e];
                ss += u[e] * u[e];
            }
        }
    }
    if (!rd) return;
    const float tot = block_sum(ss, red);
    const float r = 1.f / sqrtf(tot / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x)
        h_out[(size_t)t * W + c] = from_f<T>(u_lds[c] * r * to_f(norm_w[c]));
}

}  // namespace sm

using namespace sm;

extern "C" int sm_version(void) { return 1; }
extern "C" const char* sm_last_error(void) { return g_err; }

extern "C" int sm_embed_streams(int dtype, const int64_t* ids, const int32_t* positions, const void* embed,
                                const void* pos_table, float* X, int64_t T, int S, int W, void* stream) {
    if (T < 0 || S < 1 || W < 1 || (T > 0 && (!ids || !embed || !X || (pos_table && !positions)))) {
        set_error("sm_embed_streams: bad argument");
        return SM_EINVAL;
    }
    if (T == 0) return SM_OK;
    SM_DISPATCH(dtype, "sm_embed_streams",
                hipLaunchKernelGGL(embed_streams_kernel<DT>, dim3((unsigned)T), dim3(256), 0, as_stream(stream), ids, positions,
                                   (const DT*)embed, (const DT*)pos_table, X, S, W));
    SM_CHECK_LAUNCH("sm_embed_streams");
    return SM_OK;
}

extern "C" int sm_stream_step(int dtype, float* X, const void* y, const float* mix, const float* out, const float* w_in,
                              const void* norm_w, float eps, void* h_out, int64_t T, int S, int W, void* stream) {
    if (T < 0 || S < 1 || W < 1 || (T > 0 && !X) || (y && (!mix || !out)) || (h_out && (!w_in || !norm_w))) {
        set_error("sm_stream_step: bad argument");
        return SM_EINVAL;
    }
    if (S > kMaxStreams) { set_error("sm_stream_step: at most %d streams", kMaxStreams); return SM_ESHAPE; }
    if ((size_t)W * 4 > 60000) { set_error("sm_stream_step: width %d too large", W); return SM_ESHAPE; }
    if (T == 0 || (!y && !h_out)) return SM_OK;
    SM_DISPATCH(dtype, "sm_stream_step",
                if (W % 4 == 0)
                    hipLaunchKernelGGL((stream_step_kernel<DT, 4>), dim3((unsigned)T), dim3(256), (size_t)W * 4, as_stream(stream), X,
                                       (const DT*)y, mix, out, w_in, (const DT*)norm_w, eps, (DT*)h_out, S, W);
                else
                    hipLaunchKernelGGL((stream_step_kernel<DT, 1>), dim3((unsigned)T), dim3(256), (size_t)W * 4, as_stream(stream), X,
                                       (const DT*)y, mix, out, w_in, (const DT*)norm_w, eps, (DT*)h_out, S, W));
    SM_CHECK_LAUNCH("sm_stream_step");
    return SM_OK;
}
