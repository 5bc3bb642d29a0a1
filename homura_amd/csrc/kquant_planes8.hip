#include "kquant_planes8.h"

namespace {

// get_scale_min_k4 (reference src/gguf.rs:847-862): scale and minimum factor of 32-wide sub-block j of a Q4_K block
__device__ __forceinline__ void q4k_scale_min(const uint8_t *raw, int j, int &sc, int &mn) {
    if (j < 4) {
        sc = raw[j] & 0x3F;
        mn = raw[4 + j] & 0x3F;
    } else {
        sc = (raw[4 + j] & 0x0F) | ((raw[j - 4] >> 6) << 4);
        mn = (raw[4 + j] >> 4) | ((raw[j] >> 6) << 4);
    }
}

// one thread per (row, 16-weight sub-block)
__global__ __launch_bounds__(256) void pack_k8_kernel(const uint8_t *__restrict__ blocks, int q6, int rows, int K,
                                                      uint8_t *__restrict__ plane, uint8_t *__restrict__ records, int row0,
                                                      int row_mult) {
    const int per_row = K / 16;
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (size_t)rows * per_row) return;
    const int r = (int)(id / per_row), s = (int)(id % per_row), b = s / 16, t = s % 16;
    const uint8_t *blk = blocks + ((size_t)r * (K / 256) + b) * (q6 ? 210 : 144);
    const size_t RS = (size_t)(K / 8 + K / 64);
    const size_t dst_row = (size_t)row0 + (size_t)r * row_mult;
    uint8_t *out = plane + dst_row * K + (size_t)s * 16;
    uint8_t *rec = records + dst_row * RS;
    int sc, mn;
    if (q6) {
        // reference dequant_q6_k (src/gguf.rs:886-917): weight w = 128 chunk + 32 grp + l
        for (int e = 0; e < 16; e++) {
            const int w = t * 16 + e, chunk = w / 128, rr = w % 128, l = rr % 32, grp = rr / 32;
            const uint8_t ql = blk[chunk * 64 + (grp & 1) * 32 + l];
            const int lo = grp >= 2 ? (ql >> 4) : (ql & 0x0F);
            const int hi = (blk[128 + chunk * 32 + l] >> (2 * grp)) & 3;
            out[e] = (uint8_t)(int8_t)((lo | (hi << 4)) - 32);
        }
        sc = (int8_t)blk[192 + t];
        mn = 0;
    } else {
        // reference dequant_q4_k (src/gguf.rs:835-882): pairs of 32-wide sub-blocks share 32 bytes, even = low nibbles
        const uint8_t *qs = blk + 16;
        for (int e = 0; e < 16; e++) {
            const int w = t * 16 + e, pair = w / 64, within = w % 64;
            const uint8_t byte = qs[pair * 32 + within % 32];
            out[e] = within < 32 ? (byte & 0x0F) : (byte >> 4);
        }
        q4k_scale_min(blk + 4, t / 2, sc, mn);
    }
    rec[s * 2] = (uint8_t)(int8_t)sc;
    rec[s * 2 + 1] = (uint8_t)mn;
    if (t == 0) {
        uint8_t *dd = rec + K / 8 + (size_t)b * 4;
        if (q6) {
            dd[0] = blk[208];
            dd[1] = blk[209];
            dd[2] = 0;
            dd[3] = 0;
        } else {
            dd[0] = blk[0];
            dd[1] = blk[1];
            dd[2] = blk[2];
            dd[3] = blk[3];
        }
    }
}

}  // namespace

int pack_k8_rows(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, int rows, int K, uint8_t *d_plane, uint8_t *d_records,
                 int row0, int row_mult) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, hm_dtype == HM_DTYPE_Q4_K || hm_dtype == HM_DTYPE_Q6_K, "pack_k8_rows: dtype %d is not a K-quant", hm_dtype);
    HM_REQUIRE(ctx, d_blocks && d_plane && d_records && rows > 0 && K > 0 && K % 256 == 0 && row0 >= 0 && row_mult >= 1,
               "pack_k8_rows: bad arguments (rows=%d K=%d)", rows, K);
    const size_t total = (size_t)rows * (K / 16);
    hipLaunchKernelGGL(pack_k8_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, d_blocks,
                       hm_dtype == HM_DTYPE_Q6_K ? 1 : 0, rows, K, d_plane, d_records, row0, row_mult);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}
