// Short causal convolution over time on every channel, added to its input, with the last taps-1 inputs of every
// sequence carried as state between steps.
#include "sm_common.h"

namespace sm {

constexpr int kMaxTaps = 16;

// VEC consecutive channels per thread (VEC = 8 when W % 8 == 0: 16-byte accesses for bf16)
template <typename T, int VEC>
__global__ void canon_conv_kernel(const T* __restrict__ h, const T* __restrict__ w, const T* __restrict__ state, int run,
                                  int runs, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                  const int32_t* __restrict__ qstart, const int32_t* __restrict__ seq_slot,
                                  T* __restrict__ out, int W, int taps) {
    struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
    const int64_t t = blockIdx.x;
    const int b = tok_seq[t], pos = tok_pos[t];
    const int i = (int)t - qstart[b];                       // index of the token inside its sequence's portion
    const T* st = state + ((size_t)seq_slot[b] * runs + run) * (size_t)(taps - 1) * W;
    for (int c = (blockIdx.y * blockDim.x + threadIdx.x) * VEC; c < W; c += gridDim.y * blockDim.x * VEC) {
        const Pack x = *(const Pack*)(h + (size_t)t * W + c);
        float acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = to_f(w[(size_t)(c + e) * taps + taps - 1]) * to_f(x.v[e]);
        for (int j = 0; j < taps - 1; ++j) {
            const int back = taps - 1 - j;                  // the input `back` positions ago
            if (pos - back < 0) continue;
            const Pack v = (i - back >= 0) ? *(const Pack*)(h + (size_t)(t - back) * W + c) : *(const Pack*)(st + (size_t)(i + j) * W + c);
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += to_f(w[(size_t)(c + e) * taps + j]) * to_f(v.v[e]);
        }
        Pack o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o.v[e] = from_f<T>(to_f(x.v[e]) + acc[e]);
        *(Pack*)(out + (size_t)t * W + c) = o;
    }
}

template <typename T>
__global__ void canon_update_kernel(const T* __restrict__ h, T* __restrict__ state, int run, int runs,
                                    const int32_t* __restrict__ qstart, const int32_t* __restrict__ seq_slot, int W, int taps) {
    const int b = blockIdx.x;
    const int q0 = qstart[b], n = qstart[b + 1] - q0;
    if (n <= 0) return;
    T* st = state + ((size_t)seq_slot[b] * runs + run) * (size_t)(taps - 1) * W;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < W; c += gridDim.y * blockDim.x) {
        T nv[kMaxTaps];
        for (int k = 0; k < taps - 1; ++k) {
            const int src = n - (taps - 1) + k;             // index inside the portion of the input that lands at k
            nv[k] = src >= 0 ? h[(size_t)(q0 + src) * W + c] : st[(size_t)(k + n) * W + c];
        }
        for (int k = 0; k < taps - 1; ++k) st[(size_t)k * W + c] = nv[k];
    }
}

}  // namespace sm

using namespace sm;

extern "C" int sm_canon_conv(int dtype, const void* h, const void* w, const void* state, int run, int runs,
                             const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* qstart, const int32_t* seq_slot,
                             void* out, int64_t T, int W, int taps, void* stream) {
    if (T < 0 || W < 1 || taps < 1 || run < 0 || run >= runs ||
        (T > 0 && (!h || !w || !out || !tok_seq || !tok_pos || !qstart || !seq_slot || (taps > 1 && !state)))) {
        set_error("sm_canon_conv: bad argument");
        return SM_EINVAL;
    }
    if (taps > kMaxTaps) { set_error("sm_canon_conv: at most %d taps", kMaxTaps); return SM_ESHAPE; }
    if (T == 0) return SM_OK;
    const int vec = W % 8 == 0 ? 8 : 1;
    dim3 grid((unsigned)T, (unsigned)((W / vec + 255) / 256));
    SM_DISPATCH(dtype, "sm_canon_conv",
                if (vec == 8)
                    hipLaunchKernelGGL((canon_conv_kernel<DT, 8>), grid, dim3(256), 0, as_stream(stream), (const DT*)h, (const DT*)w,
                                       (const DT*)state, run, runs, tok_seq, tok_pos, qstart, seq_slot, (DT*)out, W, taps);
                else
                    hipLaunchKernelGGL((canon_conv_kernel<DT, 1>), grid, dim3(256), 0, as_stream(stream), (const DT*)h, (const DT*)w,
                                       (const DT*)state, run, runs, tok_seq, tok_pos, qstart, seq_slot, (DT*)out, W, taps));
    SM_CHECK_LAUNCH("sm_canon_conv");
    return SM_OK;
}

extern "C" int sm_canon_update(int dtype, const void* h, void* state, int run, int runs, const int32_t* qstart,
                               const int32_t* seq_slot, int B, int W, int taps, void* stream) {
    if (B < 0 || W < 1 || taps < 1 || run < 0 || run >= runs || (B > 0 && taps > 1 && (!h || !state || !qstart || !seq_slot))) {
        set_error("sm_canon_update: bad argument");
        return SM_EINVAL;
    }
    if (taps > kMaxTaps) { set_error("sm_canon_update: at most %d taps", kMaxTaps); return SM_ESHAPE; }
    if (B == 0 || taps == 1) return SM_OK;
    dim3 grid((unsigned)B, (unsigned)((W + 255) / 256));
    SM_DISPATCH(dtype, "sm_canon_update",
                hipLaunchKernelGGL(canon_update_kernel<DT>, grid, dim3(256), 0, as_stream(stream), (const DT*)h, (DT*)state, run,
                                   runs, qstart, seq_slot, W, taps));
    SM_CHECK_LAUNCH("sm_canon_update");
    return SM_OK;
}
