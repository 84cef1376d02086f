// The float32 residual of a decoder whose sublayers are normalised on both sides and gated: scaled embedding, the
// boundary between two sublayers (gate, norm of the result, residual add, norm in front of the next sublayer, and the
// row a token shift carries to the next step) in one launch per token, the token shift itself, and squared ReLU.
#include <algorithm>

#include "hm_common.h"

namespace hm {

static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

template <typename T>
__global__ void embed_scaled_kernel(const int64_t* __restrict__ ids, const T* __restrict__ embed, float scale,
                                    float* __restrict__ x, int W) {
    const int64_t t = blockIdx.x;
    const T* e = embed + (size_t)ids[t] * W;
    for (int c = threadIdx.x; c < W; c += blockDim.x) x[(size_t)t * W + c] = to_f(e[c]) * scale;
}

template <typename T>
__global__ __launch_bounds__(256) void sublayer_close_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                             const T* __restrict__ gate, int64_t gate_stride,
                                                             const T* __restrict__ gate_bias, const T* __restrict__ post_w,
                                                             float mult, const T* __restrict__ next_w, float eps,
                                                             T* __restrict__ h_out, const T* __restrict__ carry_src,
                                                             T* __restrict__ carry_state, int64_t slot_stride,
                                                             const int32_t* __restrict__ tok_seq,
                                                             const int32_t* __restrict__ qstart,
                                                             const int32_t* __restrict__ seq_slot, int W) {
    extern __shared__ float row[];             // W floats: the gated result, then the new residual
    __shared__ float red[16];
    const int64_t t = blockIdx.x;
    float* xr = x + (size_t)t * W;
    float ss = 0.f;
    if (y != nullptr) {
        const T* yr = y + (size_t)t * W;
        const T* gr = gate + (size_t)t * gate_stride;
        float zz = 0.f;
        for (int c = threadIdx.x; c < W; c += 256) {
            const float z = to_f(yr[c]) * sigmoid_f(to_f(gr[c]) + to_f(gate_bias[c]));
            row[c] = z;
            zz += z * z;
        }
        zz = block_sum(zz, red);
        const float r = 1.f / sqrtf(zz / (float)W + eps);
        for (int c = threadIdx.x; c < W; c += 256) {
            const float v = xr[c] + mult * (row[c] * r * to_f(post_w[c]));
            xr[c] = v;
            row[c] = v;
            ss += v * v;
        }
    } else if (next_w != nullptr) {
        for (int c = threadIdx.x; c < W; c += 256) {
            const float v = xr[c];
            row[c] = v;
            ss += v * v;
        }
    }
    if (next_w != nullptr) {
        ss = block_sum(ss, red);
        const float r = 1.f / sqrtf(ss / (float)W + eps);
        T* hr = h_out + (size_t)t * W;
        for (int c = threadIdx.x; c < W; c += 256) hr[c] = from_f<T>(row[c] * r * to_f(next_w[c]));
    }
    if (carry_src != nullptr) {
        const int b = tok_seq[t];
        if (t == (int64_t)qstart[b + 1] - 1) {
            T* st = carry_state + (size_t)seq_slot[b] * slot_stride;
            const T* src = carry_src + (size_t)t * W;
            for (int c = threadIdx.x; c < W; c += 256) st[c] = src[c];
        }
    }
}

// VEC consecutive channels per thread (VEC = 8 when W % 8 == 0: 16-byte accesses for bf16)
template <typename T, int VEC>
__global__ void token_shift_kernel(const T* __restrict__ h, const T* __restrict__ mu, const T* __restrict__ state,
                                   int64_t slot_stride, const int32_t* __restrict__ tok_seq,
                                   const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ qstart,
                                   const int32_t* __restrict__ seq_slot, T* __restrict__ out, int W) {
    struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
    const int64_t t = blockIdx.x;
    const int b = tok_seq[t];
    const T* prev = nullptr;                   // position 0: nothing before it, whatever the slot holds
    if (tok_pos[t] > 0) prev = t > (int64_t)qstart[b] ? h + (size_t)(t - 1) * W : state + (size_t)seq_slot[b] * slot_stride;
    const T* hr = h + (size_t)t * W;
    for (int c = threadIdx.x * VEC; c < W; c += blockDim.x * VEC) {
        const Pack x = *(const Pack*)(hr + c), m = *(const Pack*)(mu + c);
        Pack p, r;
        if (prev) p = *(const Pack*)(prev + c);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float v = to_f(x.v[e]);
            const float pv = prev ? to_f(p.v[e]) : 0.f;
            r.v[e] = from_f<T>(v + (pv - v) * to_f(m.v[e]));
        }
        *(Pack*)(out + (size_t)t * W + c) = r;
    }
}

template <typename T>
__global__ void relu_squared_kernel(const T* __restrict__ z, int64_t z_stride, T* __restrict__ out, int F) {
    const int64_t t = blockIdx.x;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < F; c += gridDim.y * blockDim.x) {
        const float v = fmaxf(to_f(z[(size_t)t * z_stride + c]), 0.f);
        out[(size_t)t * F + c] = from_f<T>(v * v);
    }
}

}  // namespace hm

using namespace hm;

extern "C" int hm_version(void) { return 1; }
extern "C" const char* hm_last_error(void) { return g_err; }

extern "C" int hm_embed_scaled(int dtype, const int64_t* ids, const void* embed, float scale, float* x, int64_t T, int W,
                               void* stream) {
    if (T < 0 || W < 1 || (T > 0 && (!ids || !embed || !x))) { set_error("hm_embed_scaled: bad argument"); return HM_EINVAL; }
    if (T == 0) return HM_OK;
    HM_DISPATCH(dtype, "hm_embed_scaled",
                hipLaunchKernelGGL(embed_scaled_kernel<DT>, dim3((unsigned)T), dim3(256), 0, as_stream(stream), ids,
                                   (const DT*)embed, scale, x, W));
    HM_CHECK_LAUNCH("hm_embed_scaled");
    return HM_OK;
}

extern "C" int hm_sublayer_close(int dtype, float* x, const void* y, const void* gate, int64_t gate_stride, const void* gate_bias,
                                 const void* post_w, float mult, const void* next_w, float eps, void* h_out,
                                 const void* carry_src, void* carry_state, int64_t slot_stride, const int32_t* tok_seq,
                                 const int32_t* qstart, const int32_t* seq_slot, int64_t T, int W, void* stream) {
    if (T < 0 || W < 1 || (T > 0 && !x) || (y && (!gate || !gate_bias || !post_w || gate_stride < W)) || (next_w && !h_out) ||
        (carry_src && (!carry_state || !tok_seq || !qstart || !seq_slot || slot_stride < W))) {
        set_error("hm_sublayer_close: bad argument");
        return HM_EINVAL;
    }
    if ((size_t)W * 4 > 60 * 1024) { set_error("hm_sublayer_close: width %d does not fit the row buffer", W); return HM_ESHAPE; }
    if (T == 0) return HM_OK;
    HM_DISPATCH(dtype, "hm_sublayer_close",
                hipLaunchKernelGGL(sublayer_close_kernel<DT>, dim3((unsigned)T), dim3(256), (size_t)W * 4, as_stream(stream), x,
                                   (const DT*)y, (const DT*)gate, gate_stride, (const DT*)gate_bias, (const DT*)post_w, mult,
                                   (const DT*)next_w, eps, (DT*)h_out, (const DT*)carry_src, (DT*)carry_state, slot_stride,
                                   tok_seq, qstart, seq_slot, W));
    HM_CHECK_LAUNCH("hm_sublayer_close");
    return HM_OK;
}

extern "C" int hm_token_shift(int dtype, const void* h, const void* mu, const void* state, int64_t slot_stride,
                              const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* qstart, const int32_t* seq_slot,
                              void* out, int64_t T, int W, void* stream) {
    if (T < 0 || W < 1 || slot_stride < W || (T > 0 && (!h || !mu || !state || !tok_seq || !tok_pos || !qstart || !seq_slot || !out))) {
        set_error("hm_token_shift: bad argument");
        return HM_EINVAL;
    }
    if (T == 0) return HM_OK;
    // packs need aligned rows: the width and the slots' distance in whole packs
    const bool wide = W % 8 == 0 && slot_stride % 8 == 0;
    HM_DISPATCH(dtype, "hm_token_shift",
                if (wide)
                    hipLaunchKernelGGL((token_shift_kernel<DT, 8>), dim3((unsigned)T), dim3(std::min(256, (W / 8 + 63) / 64 * 64)), 0,
                                       as_stream(stream), (const DT*)h, (const DT*)mu, (const DT*)state, slot_stride, tok_seq,
                                       tok_pos, qstart, seq_slot, (DT*)out, W);
                else
                    hipLaunchKernelGGL((token_shift_kernel<DT, 1>), dim3((unsigned)T), dim3(256), 0, as_stream(stream), (const DT*)h,
                                       (const DT*)mu, (const DT*)state, slot_stride, tok_seq, tok_pos, qstart, seq_slot, (DT*)out, W));
    HM_CHECK_LAUNCH("hm_token_shift");
    return HM_OK;
}

extern "C" int hm_relu_squared(int dtype, const void* z, int64_t z_stride, void* out, int64_t T, int F, void* stream) {
    if (T < 0 || F < 1 || z_stride < F || (T > 0 && (!z || !out))) { set_error("hm_relu_squared: bad argument"); return HM_EINVAL; }
    if (T == 0) return HM_OK;
    dim3 grid((unsigned)T, (unsigned)((F + 1023) / 1024));
    HM_DISPATCH(dtype, "hm_relu_squared",
                hipLaunchKernelGGL(relu_squared_kernel<DT>, grid, dim3(256), 0, as_stream(stream), (const DT*)z, z_stride,
                                   (DT*)out, F));
    HM_CHECK_LAUNCH("hm_relu_squared");
    return HM_OK;
}
