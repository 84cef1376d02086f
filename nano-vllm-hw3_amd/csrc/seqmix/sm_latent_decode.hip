// Latent attention for single-token queries (decode) on the matrix cores.  The H heads of a sequence's one token are
// the query rows (they all see the same keys); the keys are split over workgroups in whole tiles, every
// (sequence, split) leaves an unnormalised partial state {m * c, l, O} in the workspace, and a second launch merges
// the splits in order.  The split count is the caller's and does not depend on the sequences' lengths.
#include "sm_latent_tile.h"

namespace sm {

// floats per (sequence, split, head) in the workspace: scaled maximum, sum, RP outputs
__host__ __device__ constexpr int part_stride(int nb) { return 32 * nb + 2; }

template <int NB, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void latent_attn_decode_kernel(const unsigned short* __restrict__ q,
                                                                        const unsigned short* __restrict__ cache,
                                                                        const int32_t* __restrict__ block_tables,
                                                                        const int32_t* __restrict__ ctx, float* __restrict__ ws,
                                                                        float c_log2, int H, int R, int block_size,
                                                                        int max_blocks, int splits) {
    typedef TileGeom<NB> G;
    __shared__ __attribute__((aligned(16))) unsigned char lds[G::LDS_BYTES];
    const int sp = blockIdx.x, b = blockIdx.y;
    const int n = ctx[b];
    const int per = ((n + kTileKeys - 1) / kTileKeys + splits - 1) / splits * kTileKeys;      // keys per split, whole tiles
    const int k_lo = sp * per, k_hi = min(n, k_lo + per);
    const int lane = threadIdx.x & 63, l31 = lane & 31, hi = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = 32 * wave + l31;
    float* part = ws + (((size_t)b * splits + sp) * H + min(r, H - 1)) * part_stride(NB);
    if (k_lo >= k_hi) {                                      // an empty split: the merge skips l == 0
        if (r < H && hi == 0) { part[0] = -INFINITY; part[1] = 0.f; }
        return;
    }
    const int rc = min(r, H - 1);
    f32x16 oacc[NB];
    float m_run, l_tot;
    latent_tile_loop<NB, WAVES>(q + ((size_t)b * H + rc) * R, cache, block_tables + (size_t)b * max_blocks, R, block_size, k_lo,
                                k_hi, n - 1, n - 1, c_log2, lds, oacc, m_run, l_tot);
    if (r >= H) return;
    if (hi == 0) { part[0] = m_run * c_log2; part[1] = l_tot; }
#pragma unroll
    for (int d = 0; d < NB; ++d)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq)
#pragma unroll
            for (int e = 0; e < 4; ++e) part[2 + 32 * d + 8 * rq + 4 * hi + e] = oacc[d][4 * rq + e];
}

__global__ void latent_decode_merge_kernel(const float* __restrict__ ws, unsigned short* __restrict__ o, int H, int R, int splits,
                                           int stride) {
    const size_t row = blockIdx.x;                          // b * H + h
    const size_t b = row / H, h = row % H;
    float M = -INFINITY;
    for (int s = 0; s < splits; ++s) {
        const float* p = ws + ((b * splits + s) * H + h) * stride;
        if (p[1] > 0.f) M = fmaxf(M, p[0]);
    }
    float L = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float* p = ws + ((b * splits + s) * H + h) * stride;
        if (p[1] > 0.f) L += __builtin_amdgcn_exp2f(p[0] - M) * p[1];
    }
    const float inv = 1.f / L;
    for (int c = threadIdx.x; c < R; c += blockDim.x) {
        float acc = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float* p = ws + ((b * splits + s) * H + h) * stride;
            if (p[1] > 0.f) acc += __builtin_amdgcn_exp2f(p[0] - M) * p[2 + c];
        }
        o[row * R + c] = __builtin_bit_cast(unsigned short, (bf16_t)(acc * inv));
    }
}

static int padded_nb(int R) {
    const int nb = (R + 31) / 32;
    return nb <= 4 ? nb : (nb <= 6 ? 6 : 8);
}

}  // namespace sm

using namespace sm;

extern "C" size_t sm_latent_decode_workspace_bytes(int64_t B, int H, int R, int splits) {
    if (B <= 0 || H <= 0 || R <= 0 || splits <= 0) return 0;
    return (size_t)B * splits * H * part_stride(padded_nb(R)) * sizeof(float);
}

extern "C" int sm_latent_attn_decode(const void* q, const void* cache, const int32_t* block_tables, const int32_t* ctx, void* o,
                                     float scale, int64_t B, int H, int R, int block_size, int max_blocks, int splits,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    if (B < 0 || H < 1 || R < 1 || block_size < 1 || max_blocks < 1 || splits < 1 ||
        (B > 0 && (!q || !cache || !block_tables || !ctx || !o || !workspace))) {
        set_error("sm_latent_attn_decode: bad argument");
        return SM_EINVAL;
    }
    if (R % 8 || R > 256 || block_size % 64 || H > 128 || B > 65535 || splits > 65535) {
        set_error("sm_latent_attn_decode: needs R %% 8 == 0, R <= 256, block_size %% 64 == 0, H <= 128");
        return SM_ESHAPE;
    }
    if (workspace_bytes < sm_latent_decode_workspace_bytes(B, H, R, splits)) {
        set_error("sm_latent_attn_decode: workspace too small");
        return SM_EWORKSPACE;
    }
    if (B == 0) return SM_OK;
    const int nb = padded_nb(R), waves = H <= 32 ? 1 : (H <= 64 ? 2 : 4);
    dim3 grid((unsigned)splits, (unsigned)B);
    const float c = scale * 1.4426950408889634f;
    hipStream_t s = as_stream(stream);
#define SM_DEC(NB_, W_)                                                                                                    \
    hipLaunchKernelGGL((latent_attn_decode_kernel<NB_, W_>), grid, dim3(64 * W_), 0, s, (const unsigned short*)q,          \
                       (const unsigned short*)cache, block_tables, ctx, (float*)workspace, c, H, R, block_size, max_blocks, splits)
#define SM_DEC_W(NB_) do { if (waves == 1) SM_DEC(NB_, 1); else if (waves == 2) SM_DEC(NB_, 2); else SM_DEC(NB_, 4); } while (0)
    switch (nb) {
        case 1: SM_DEC_W(1); break;
        case 2: SM_DEC_W(2); break;
        case 3: SM_DEC_W(3); break;
        case 4: SM_DEC_W(4); break;
        case 6: SM_DEC_W(6); break;
        default: SM_DEC_W(8); break;
    }
#undef SM_DEC_W
#undef SM_DEC
    SM_CHECK_LAUNCH("sm_latent_attn_decode");
    hipLaunchKernelGGL(latent_decode_merge_kernel, dim3((unsigned)(B * H)), dim3(64), 0, s, (const float*)workspace,
                       (unsigned short*)o, H, R, splits, part_stride(nb));
    SM_CHECK_LAUNCH("sm_latent_attn_decode (merge)");
    return SM_OK;
}
