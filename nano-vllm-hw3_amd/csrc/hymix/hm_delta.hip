// Generalized delta rule: S <- diag(w) S - (a u)(u^T S) + k v^T per head, o = S^T r, with a float32 state S [D, D] per
// (state slot, head).  Three launches: the float32 inputs of the recurrence from the mixer's merged product (parallel
// over tokens), the recurrence (sequential over a portion's tokens, parallel over sequences, heads and value channels),
// and the per-head norm and output gate (parallel over tokens).
#include <algorithm>

#include "hm_common.h"

namespace hm {

// One workgroup per (kPrepTokens consecutive tokens, head), one thread per key channel: a thread's row of w2 is read once
// for the tokens of the tile.  prep[t, h] = decay | a*u | u | k | r, D floats each.
constexpr int kPrepTokens = 8;

template <typename T>
__global__ void delta_prepare_kernel(const T* __restrict__ proj, int64_t row_stride, int r_off, int k_off, int a_off, int z_off,
                                     const T* __restrict__ w2, const T* __restrict__ w0, const T* __restrict__ a_bias, int rank,
                                     float decay_scale, float unit_eps, float* __restrict__ prep, int64_t T_, int H, int D) {
    extern __shared__ float tz[];              // kPrepTokens x rank floats: tanh of the decay's inner projection
    __shared__ float red[16];
    const int64_t t0 = (int64_t)blockIdx.x * kPrepTokens;
    const int nt = (int)min((int64_t)kPrepTokens, T_ - t0);
    const int hd = blockIdx.y, i = threadIdx.x;
    for (int e = threadIdx.x; e < nt * rank; e += blockDim.x) {
        const int tt = e / rank, j = e - tt * rank;
        tz[e] = tanhf(to_f(proj[(size_t)(t0 + tt) * row_stride + z_off + j]));
    }
    __syncthreads();
    const int c = hd * D + i;
    float acc[kPrepTokens];
#pragma unroll
    for (int tt = 0; tt < kPrepTokens; ++tt) acc[tt] = 0.f;
    float bias_a = 0.f, bias_w = 0.f;
    if (i < D) {
        const T* wr = w2 + (size_t)c * rank;
        struct alignas(sizeof(T) * 8) Pack { T v[8]; };
        int j = 0;
        if (rank % 8 == 0) {                   // 16-byte loads of the row (bf16); every token's sum runs over j = 0, 1, 2, ...
            for (; j < rank; j += 8) {
                const Pack pk = *(const Pack*)(wr + j);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float w = to_f(pk.v[e]);
#pragma unroll
                    for (int tt = 0; tt < kPrepTokens; ++tt) acc[tt] += w * tz[(tt < nt ? tt : 0) * rank + j + e];
                }
            }
        }
        for (; j < rank; ++j) {
            const float w = to_f(wr[j]);
#pragma unroll
            for (int tt = 0; tt < kPrepTokens; ++tt) acc[tt] += w * tz[(tt < nt ? tt : 0) * rank + j];
        }
        bias_a = to_f(a_bias[c]);
        bias_w = to_f(w0[c]);
    }
#pragma unroll
    for (int tt = 0; tt < kPrepTokens; ++tt) {
        if (tt >= nt) break;                   // (uniform over the workgroup)
        const T* row = proj + (size_t)(t0 + tt) * row_stride;
        float k = 0.f, r = 0.f, a = 0.f, decay = 0.f;
        if (i < D) {
            k = to_f(row[k_off + c]);
            r = to_f(row[r_off + c]);
            a = sigmoid_f(to_f(row[a_off + c]) + bias_a);
            decay = expf(-decay_scale * sigmoid_f(acc[tt] + bias_w));
        }
        const float ss = block_sum(k * k, red);
        if (i < D) {
            const float u = k / sqrtf(ss + unit_eps);
            float* out = prep + ((size_t)(t0 + tt) * H + hd) * 5 * D + i;
            out[0] = decay;
            out[D] = a * u;
            out[2 * D] = u;
            out[3 * D] = k;
            out[4 * D] = r;
        }
    }
}

// Sum over 8 neighbouring lanes with data-parallel-primitive moves (no LDS round trip): pairs, quads, then the mirrored
// half row; every lane of the group ends with the same total.
__device__ __forceinline__ float sum8(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // row_half_mirror
    return v;
}

// One workgroup of 256 threads per (sequence, head, 256 / SL value channels).  A column of S (one value channel, DK >= D
// key channels) is spread over SL neighbouring lanes, DK / SL channels each in registers; u^T S and S^T r are summed over
// those lanes with a butterfly, so every lane holds the total and the order of the sums is fixed by DK and SL alone.
// The per-token vectors (decay, a u, u, k, r and v, DK floats each, zero beyond D) are staged in LDS CH tokens at a time:
// the next chunk is requested from global memory before the current chunk's tokens run and written to the other buffer
// after them, so the recurrence itself waits for LDS only, with one barrier per chunk.
template <typename T, int DK, int SL, int CH>
__global__ __launch_bounds__(256) void delta_recurrence_kernel(const float* __restrict__ prep, const T* __restrict__ v,
                                                               int64_t v_stride, float* __restrict__ state,
                                                               const int32_t* __restrict__ qstart,
                                                               const int32_t* __restrict__ seq_pos0,
                                                               const int32_t* __restrict__ seq_slot, float* __restrict__ o,
                                                               int H, int D) {
    static_assert(SL == 8, "the lane sums are written for groups of 8");
    constexpr int KS = DK / SL, COLS = 256 / SL, TOK = 6 * DK, NR = (CH * TOK + 255) / 256;
    __shared__ __attribute__((aligned(16))) float buf[2][CH * TOK];
    const int b = blockIdx.x, hd = blockIdx.y;
    const int q0 = qstart[b], n = qstart[b + 1] - q0;
    if (n <= 0) return;
    const int tid = threadIdx.x, slice = tid % SL, col = tid / SL;
    const int j = blockIdx.z * COLS + col;
    const bool live = j < D;
    float* st = state + ((size_t)seq_slot[b] * H + hd) * (size_t)D * D;
    float s[KS];
    const bool fresh = seq_pos0[b] == 0;       // a sequence's first tokens: the state starts at zero, whatever the slot holds
#pragma unroll
    for (int ii = 0; ii < KS; ++ii) {
        const int i = slice * KS + ii;
        s[ii] = (!fresh && live && i < D) ? st[(size_t)i * D + j] : 0.f;
    }
    float regs[NR];
    auto request = [&](int tok0) {             // the vectors of tokens tok0 .. tok0 + CH - 1 into registers
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            const int e = tid + 256 * k;
            const int tc = e / TOK, rem = e - tc * TOK, part = rem / DK, i = rem - part * DK, tok = tok0 + tc;
            // beyond the portion's end a chunk is filled with the identity step (decay 1, everything else 0): every chunk
            // then runs CH steps of straight-line code and the state passes through the padding unchanged
            float val = part == 0 && tok >= n ? 1.f : 0.f;
            if (e < CH * TOK && tok < n && i < D) {
                const size_t row = (size_t)(q0 + tok);
                val = part < 5 ? prep[(row * H + hd) * 5 * D + (size_t)part * D + i] : to_f(v[row * v_stride + hd * D + i]);
            }
            regs[k] = val;
        }
    };
    auto deposit = [&](int which) {
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            const int e = tid + 256 * k;
            if (e < CH * TOK) buf[which][e] = regs[k];
        }
    };
    request(0);
    deposit(0);
    __syncthreads();
    int which = 0;
    for (int tok0 = 0; tok0 < n; tok0 += CH) {
        const bool more = tok0 + CH < n;
        if (more) request(tok0 + CH);
#pragma unroll
        for (int tc = 0; tc < CH; ++tc) {
            const float* p = buf[which] + tc * TOK + slice * KS;
            float dot = 0.f;
#pragma unroll
            for (int ii = 0; ii < KS; ++ii) dot += p[2 * DK + ii] * s[ii];
            dot = sum8(dot);
            const float vj = buf[which][tc * TOK + 5 * DK + min(j, DK - 1)];
            float out = 0.f;
#pragma unroll
            for (int ii = 0; ii < KS; ++ii) {
                s[ii] = p[ii] * s[ii] - p[DK + ii] * dot + p[3 * DK + ii] * vj;
                out += s[ii] * p[4 * DK + ii];
            }
            out = sum8(out);
            if (live && slice == 0 && tok0 + tc < n) o[((size_t)(q0 + tok0 + tc) * H + hd) * D + j] = out;
        }
        if (more) {
            deposit(which ^ 1);                // the other buffer was last read one chunk ago, before that chunk's barrier
            __syncthreads();
            which ^= 1;
        }
    }
    if (live) {
#pragma unroll
        for (int ii = 0; ii < KS; ++ii) {
            const int i = slice * KS + ii;
            if (i < D) st[(size_t)i * D + j] = s[ii];
        }
    }
}

// A head's D channels are spread over LPH lanes (a power of two, VEC consecutive channels per lane and round), so a wave
// covers 64 / LPH heads of one token at once; a workgroup of four waves walks the token's heads.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void delta_gate_norm_kernel(const float* __restrict__ o, const T* __restrict__ g,
                                                              int64_t g_stride, const T* __restrict__ norm_w, float eps,
                                                              T* __restrict__ out, int H, int D, int LPH) {
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int per_wave = 64 / LPH, sub = lane / LPH, li = lane % LPH;
    for (int hd = (blockIdx.y * 4 + wave) * per_wave + sub; hd < H + sub; hd += gridDim.y * 4 * per_wave) {
        const bool head = hd < H;              // lanes of a head beyond the last still take part in the shuffles
        const float* orow = o + ((size_t)t * H + (head ? hd : 0)) * D;
        float ss = 0.f;
        if (head)
            for (int i = li * VEC; i < D; i += LPH * VEC)
#pragma unroll
                for (int e = 0; e < VEC; ++e) ss += orow[i + e] * orow[i + e];
        for (int w = 1; w < LPH; w <<= 1) ss += __shfl_xor(ss, w);
        if (!head) continue;
        const float r = 1.f / sqrtf(ss / (float)D + eps);
        for (int i = li * VEC; i < D; i += LPH * VEC)
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const int c = hd * D + i + e;
                out[(size_t)t * H * D + c] = from_f<T>(orow[i + e] * r * to_f(norm_w[c]) * sigmoid_f(to_f(g[(size_t)t * g_stride + c])));
            }
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
    if (D > 256 || rank > 1024 || H > 65535) { set_error("hm_delta_prepare: dim <= 256, rank <= 1024, heads <= 65535"); return HM_ESHAPE; }
    if (T == 0) return HM_OK;
    dim3 grid((unsigned)((T + kPrepTokens - 1) / kPrepTokens), (unsigned)H);
    const int threads = (D + 63) / 64 * 64;
    HM_DISPATCH(dtype, "hm_delta_prepare",
                hipLaunchKernelGGL(delta_prepare_kernel<DT>, grid, dim3(threads), (size_t)rank * 4 * kPrepTokens, as_stream(stream),
                                   (const DT*)proj, row_stride, r_off, k_off, a_off, z_off, (const DT*)w2, (const DT*)w0,
                                   (const DT*)a_bias, rank, decay_scale, unit_eps, prep, T, H, D));
    HM_CHECK_LAUNCH("hm_delta_prepare");
    return HM_OK;
}

template <typename DT>
static int launch_recurrence(const float* prep, const void* v, int64_t v_stride, float* state, const int32_t* qstart,
                             const int32_t* seq_pos0, const int32_t* seq_slot, float* o, int B, int H, int D, int max_q,
                             hipStream_t s) {
    constexpr int SL = 8, COLS = 256 / SL;
    dim3 grid((unsigned)B, (unsigned)H, (unsigned)((D + COLS - 1) / COLS));
#define HM_RECUR(DK, CH)                                                                                                      \
    hipLaunchKernelGGL((delta_recurrence_kernel<DT, DK, SL, CH>), grid, dim3(256), 0, s, prep, (const DT*)v, v_stride, state, \
                       qstart, seq_pos0, seq_slot, o, H, D)
    // single tokens (decode): one token staged at a time, so that many small workgroups fit a CU; the sums are the same
    if (max_q <= 1) {
        if (D <= 32) HM_RECUR(32, 1);
        else if (D <= 64) HM_RECUR(64, 1);
        else if (D <= 128) HM_RECUR(128, 1);
        else HM_RECUR(256, 1);
    } else if (D <= 32) HM_RECUR(32, 8);
    else if (D <= 64) HM_RECUR(64, 8);
    else if (D <= 128) HM_RECUR(128, 8);
    else HM_RECUR(256, 4);
#undef HM_RECUR
    return 0;
}

extern "C" int hm_delta_recurrence(int dtype, const float* prep, const void* v, int64_t v_stride, float* state,
                                   const int32_t* qstart, const int32_t* seq_pos0, const int32_t* seq_slot, float* o, int B,
                                   int H, int D, int max_q, void* stream) {
    if (B < 0 || H < 1 || D < 1 || v_stride < (int64_t)H * D || (B > 0 && (!prep || !v || !state || !qstart || !seq_pos0 || !seq_slot || !o))) {
        set_error("hm_delta_recurrence: bad argument");
        return HM_EINVAL;
    }
    if (D > 256 || H > 65535) { set_error("hm_delta_recurrence: dim <= 256 and heads <= 65535"); return HM_ESHAPE; }
    if (B == 0) return HM_OK;
    HM_DISPATCH(dtype, "hm_delta_recurrence",
                launch_recurrence<DT>(prep, v, v_stride, state, qstart, seq_pos0, seq_slot, o, B, H, D, max_q, as_stream(stream)));
    HM_CHECK_LAUNCH("hm_delta_recurrence");
    return HM_OK;
}

extern "C" int hm_delta_gate_norm(int dtype, const float* o, const void* g, int64_t g_stride, const void* norm_w, float eps,
                                  void* out, int64_t T, int H, int D, void* stream) {
    if (T < 0 || H < 1 || D < 1 || g_stride < (int64_t)H * D || (T > 0 && (!o || !g || !norm_w || !out))) {
        set_error("hm_delta_gate_norm: bad argument");
        return HM_EINVAL;
    }
    if (T == 0) return HM_OK;
    const int vec = D % 4 == 0 ? 4 : 1;
    int lph = 1;
    while (lph < 64 && lph * vec < D) lph <<= 1;
    const int heads_per_block = 4 * (64 / lph);
    dim3 grid((unsigned)T, (unsigned)std::min(64, (H + heads_per_block - 1) / heads_per_block));
    HM_DISPATCH(dtype, "hm_delta_gate_norm",
                if (vec == 4)
                    hipLaunchKernelGGL((delta_gate_norm_kernel<DT, 4>), grid, dim3(256), 0, as_stream(stream), o, (const DT*)g,
                                       g_stride, (const DT*)norm_w, eps, (DT*)out, H, D, lph);
                else
                    hipLaunchKernelGGL((delta_gate_norm_kernel<DT, 1>), grid, dim3(256), 0, as_stream(stream), o, (const DT*)g,
                                       g_stride, (const DT*)norm_w, eps, (DT*)out, H, D, lph));
    HM_CHECK_LAUNCH("hm_delta_gate_norm");
    return HM_OK;
}
