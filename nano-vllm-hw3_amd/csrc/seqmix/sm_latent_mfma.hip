// Latent attention on the matrix cores (placeholder entry points until the tiled kernels land).
#include "sm_common.h"
using namespace sm;
extern "C" int sm_latent_attn_tiles(const void*, const void*, const int32_t*, const int32_t*, const int32_t*, void*, float, int,
                                    int, int, int, int, int, void*) {
    set_error("sm_latent_attn_tiles: not built");
    return SM_ESHAPE;
}
extern "C" size_t sm_latent_decode_workspace_bytes(int64_t, int, int, int) { return 0; }
extern "C" int sm_latent_attn_decode(const void*, const void*, const int32_t*, const int32_t*, void*, float, int64_t, int, int,
                                     int, int, int, void*, size_t, void*) {
    set_error("sm_latent_attn_decode: not built");
    return SM_ESHAPE;
}
