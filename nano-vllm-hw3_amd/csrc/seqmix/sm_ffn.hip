// Activations of the feed-forward layers: PolyNorm (a normalised cubic polynomial of a row) and the clamped GLU.
#include "sm_common.h"

namespace sm {

template <typename T, int VEC>
__global__ __launch_bounds__(256) void poly_norm_kernel(const T* __restrict__ z, const float* __restrict__ coef, float eps,
                                                        T* __restrict__ out, int F) {
    __shared__ float red[16];
    const int64_t t = blockIdx.x;
    const T* zr = z + (size_t)t * F;
    struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int c = threadIdx.x * VEC; c < F; c += 256 * VEC) {
        const Pack pk = *(const Pack*)(zr + c);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float v = to_f(pk.v[e]), v2 = v * v, v3 = v2 * v;
            s1 += v2;
            s2 += v2 * v2;
            s3 += v3 * v3;
        }
    }
    s1 = block_sum(s1, red);
    s2 = block_sum(s2, red);
    s3 = block_sum(s3, red);
    const float invF = 1.f / (float)F;
    const float r1 = coef[0] / sqrtf(s1 * invF + eps), r2 = coef[1] / sqrtf(s2 * invF + eps),
                r3 = coef[2] / sqrtf(s3 * invF + eps), e = coef[3];
    for (int c = threadIdx.x * VEC; c < F; c += 256 * VEC) {
        const Pack pk = *(const Pack*)(zr + c);
        Pack o;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            const float v = to_f(pk.v[k]), v2 = v * v;
            o.v[k] = from_f<T>(r1 * v + r2 * v2 + r3 * (v2 * v) + e);
        }
        *(Pack*)(out + (size_t)t * F + c) = o;
    }
}

__device__ __forceinline__ float clamped_glu(float g, float u, float limit, float alpha) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.f + __expf(-alpha * g)) * (u + 1.f);
}

// VEC consecutive columns per thread (VEC = 8 when F % 8 == 0: whole 16-byte accesses for bf16)
template <typename T, int VEC>
__global__ void clamped_glu_kernel(const T* __restrict__ gu, float limit, float alpha, T* __restrict__ out, int64_t n, int F) {
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if (i >= n) return;
    const int64_t t = i / F;
    const int c = (int)(i - t * F);
    const T* row = gu + (size_t)t * 2 * F;
    struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
    const Pack g = *(const Pack*)(row + c), u = *(const Pack*)(row + F + c);
    Pack o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) o.v[e] = from_f<T>(clamped_glu(to_f(g.v[e]), to_f(u.v[e]), limit, alpha));
    *(Pack*)(out + i) = o;
}

}  // namespace sm

using namespace sm;

extern "C" int sm_poly_norm(int dtype, const void* z, const float* coef, float eps, void* out, int64_t T, int F, void* stream) {
    if (T < 0 || F < 1 || (T > 0 && (!z || !coef || !out))) { set_error("sm_poly_norm: bad argument"); return SM_EINVAL; }
    if (T == 0) return SM_OK;
    SM_DISPATCH(dtype, "sm_poly_norm",
                if (F % 8 == 0)
                    hipLaunchKernelGGL((poly_norm_kernel<DT, 8>), dim3((unsigned)T), dim3(256), 0, as_stream(stream), (const DT*)z,
                                       coef, eps, (DT*)out, F);
                else
                    hipLaunchKernelGGL((poly_norm_kernel<DT, 1>), dim3((unsigned)T), dim3(256), 0, as_stream(stream), (const DT*)z,
                                       coef, eps, (DT*)out, F));
    SM_CHECK_LAUNCH("sm_poly_norm");
    return SM_OK;
}

extern "C" int sm_clamped_glu(int dtype, const void* gu, float limit, float alpha, void* out, int64_t T, int F, void* stream) {
    if (T < 0 || F < 1 || (T > 0 && (!gu || !out))) { set_error("sm_clamped_glu: bad argument"); return SM_EINVAL; }
    if (T == 0) return SM_OK;
    const int64_t n = T * F;
    SM_DISPATCH(dtype, "sm_clamped_glu",
                if (F % 8 == 0)
                    hipLaunchKernelGGL((clamped_glu_kernel<DT, 8>), dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0,
                                       as_stream(stream), (const DT*)gu, limit, alpha, (DT*)out, n, F);
                else
                    hipLaunchKernelGGL((clamped_glu_kernel<DT, 1>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                                       as_stream(stream), (const DT*)gu, limit, alpha, (DT*)out, n, F));
    SM_CHECK_LAUNCH("sm_clamped_glu");
    return SM_OK;
}
