// Attention whose keys and values are made from one small latent a token ("latent attention").
//
// What is cached a token is one row [c (C channels) | k_rot (R channels)]: the normed latent and
// the rotated key part that all heads share.  Queries are brought into the latent's space (per
// head q_abs = W_uk^T q_unrotated, a product of its own), so a head's score over the cached row is
//     q_abs . c + q_rot . k_rot     = q_unrotated . (W_uk c) + q_rot . k_rot,
// attention runs as one key/value head of size C + R shared by all query heads, its value is the
// latent itself, and W_uv is applied to the attention's output.  k_latent_prepare does everything
// between the two down projections and the attention: the latent's RMSNorm, the rotation of the
// shared key part and of every head's rotated query channels (pairs (2i, 2i+1) of the first `dims`
// of the R channels, angle = position x inv_freq[i] formed in 32 bits), the write of the cached
// row into the key pages [page][0][slot][C + R] and, transposed, into the value pages
// [page][0][Dvc][slot] (Dvc = C, or C + R where the attention kernel wants values as long as
// keys), and the copy of the unrotated query channels in the compute type for the product that
// follows.  A workgroup a token.
#include "common.h"

template <typename TO>
__global__ __launch_bounds__(256) void k_latent_prepare(
    TO* __restrict__ qn_out, TO* __restrict__ q_out, TO* __restrict__ k_cache, TO* __restrict__ v_cache,
    const float* __restrict__ q_in, const float* __restrict__ kv_in, const float* __restrict__ c_w,
    const int* __restrict__ positions, const int* __restrict__ req_of_token, const int* __restrict__ block_table,
    const float* __restrict__ inv_freq, int table_stride, int H, int D, int R, int C, int Dvc, int dims, int ld_q, int ld_kv,
    int page_shift, int page_size, float eps) {
    __shared__ float part[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int pos = positions[t];
    const float* kv = kv_in + (size_t)t * ld_kv;
    // the latent's norm
    float ss = 0.f;
    for (int i = tid; i < C; i += 256) ss += kv[i] * kv[i];
    ss = wave_sum(ss);
    if ((tid & 63) == 0) part[tid >> 6] = ss;
    __syncthreads();
    const float rinv = 1.0f / sqrtf(((part[0] + part[1]) + (part[2] + part[3])) / (float)C + eps);
    const PageRef pr = page_of(block_table, table_stride, req_of_token[t], pos, page_shift, page_size - 1);
    const int DK = C + R;
    TO* krow = k_cache + ((size_t)pr.page * page_size + pr.off) * DK;
    TO* vpage = v_cache + (size_t)pr.page * Dvc * page_size + pr.off;
    for (int i = tid; i < C; i += 256) {
        const float c = kv[i] * rinv * c_w[i];
        st<TO>(krow, i, c);
        st<TO>(vpage, (size_t)i * page_size, c);
    }
    // the shared key part and every head's rotated query channels: unit u = 0 is the key, u = 1 + h head h
    const int half = dims >> 1, pairs_r = (R + 1) >> 1;       // a "pair" past `dims` is two channels that pass unchanged
    for (int w = tid; w < (H + 1) * pairs_r; w += 256) {
        const int u = w / pairs_r, i = w - u * pairs_r;
        const float* src = u == 0 ? kv + C : q_in + (size_t)t * ld_q + (size_t)(u - 1) * (D + R) + D;
        const int c0 = 2 * i, c1 = 2 * i + 1;
        float a = src[c0], b = c1 < R ? src[c1] : 0.f;
        if (i < half) {
            const float ang = (float)pos * inv_freq[i];
            const float cs = cosf(ang), sn = sinf(ang);
            const float ra = a * cs - b * sn, rb = b * cs + a * sn;
            a = ra;
            b = rb;
        }
        if (u == 0) {
            st<TO>(krow, C + c0, a);
            if (c1 < R) st<TO>(krow, C + c1, b);
            if (Dvc > C) {
                st<TO>(vpage, (size_t)(C + c0) * page_size, a);
                if (c1 < R) st<TO>(vpage, (size_t)(C + c1) * page_size, b);
            }
        } else {
            TO* dst = q_out + ((size_t)t * H + (u - 1)) * DK + C;
            st<TO>(dst, c0, a);
            if (c1 < R) st<TO>(dst, c1, b);
        }
    }
    // the unrotated query channels, head by head, for the product into the latent's space
    for (int w = tid; w < H * D; w += 256) {
        const int h = w / D, d = w - h * D;
        st<TO>(qn_out, (size_t)t * H * D + w, q_in[(size_t)t * ld_q + (size_t)h * (D + R) + d]);
    }
}

extern "C" int xr_latent_prepare(void* qn_out, void* q_out, void* k_cache, void* v_cache, const float* q_in, const float* kv_in,
                                 const float* c_w, const int* positions, const int* req_of_token, const int* block_table,
                                 int table_stride, const float* inv_freq, int T, int H, int D, int R, int C, int Dvc, int dims,
                                 int ld_q, int ld_kv, int page_size, float eps, int dtype, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && H > 0 && D > 0 && R >= 0 && C > 0, "latent_prepare: bad sizes T=%d H=%d D=%d R=%d C=%d", T, H, D, R, C);
    XR_REQUIRE(Dvc == C || Dvc == C + R, "latent_prepare: values of %d channels (the latent's %d, or %d with the rotated part)", Dvc, C, C + R);
    XR_REQUIRE(dims >= 0 && dims % 2 == 0 && dims <= R && (dims == 0 || inv_freq), "latent_prepare: %d rotated channels of %d", dims, R);
    XR_REQUIRE(ld_q >= H * (D + R) && ld_kv >= C + R, "latent_prepare: row strides %d, %d are too short", ld_q, ld_kv);
    const int shift = ilog2_exact(page_size);
    XR_REQUIRE(shift >= 0, "latent_prepare: page size %d is no power of two", page_size);
    if (T == 0) return XR_OK;
    if (dtype == XR_F32)
        k_latent_prepare<float><<<T, 256, 0, stream>>>((float*)qn_out, (float*)q_out, (float*)k_cache, (float*)v_cache, q_in, kv_in, c_w,
                                                       positions, req_of_token, block_table, inv_freq, table_stride, H, D, R, C, Dvc,
                                                       dims, ld_q, ld_kv, shift, page_size, eps);
    else if (dtype == XR_BF16)
        k_latent_prepare<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)qn_out, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, q_in, kv_in,
                                                        c_w, positions, req_of_token, block_table, inv_freq, table_stride, H, D, R, C,
                                                        Dvc, dims, ld_q, ld_kv, shift, page_size, eps);
    else { xr_set_error("latent_prepare: bad dtype %d", dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("latent_prepare");
    return XR_OK;
}
