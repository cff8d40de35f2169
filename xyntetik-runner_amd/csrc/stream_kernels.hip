// Kernels around the residual stream of a model that keeps several copies of it, and the
// embedding that starts it: a token's row plus a row of a hashed table of token pairs, normed;
// the mixing of the copies before and after a sublayer ("hyper-connections"), with the norm that
// the sublayer reads fused in.  All arithmetic is 32-bit float.
#include "common.h"

// sum over a workgroup of 256 threads (4 waves); every thread gets the total, in one fixed order
__device__ inline float block_sum_256(float v, float* part) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();            // `part` may still be read from a call before
    if (lane == 0) part[wave] = v;
    __syncthreads();
    return (part[0] + part[1]) + (part[2] + part[3]);
}

// ---------------------------------------------------------------- embedding with a hashed pair table
// x[t] = table[id_t] + pairs[r_t], then RMSNorm with weight w (w null: no norm).
// r_t = (prev_t * mul_prev + id_t * mul_cur) mod buckets; the token at position 0, which has none
// before it, reads row `buckets` (the table has buckets + 1 rows).  prev_t is the row before in
// the same request's portion, or, for a portion's first row, the request's last token of the step
// before, kept in last_token[slot].  The workgroup of a portion's first row is the only one that
// touches the request's entry: it reads it, and then writes the portion's last token there.
// An id outside [0, V) reads row 0 of `table` (and hashes as it is).
template <typename TW>
__global__ __launch_bounds__(256) void k_embedding_pairs(float* __restrict__ out, const TW* __restrict__ table,
                                                         const TW* __restrict__ pairs, const float* __restrict__ w,
                                                         const int* __restrict__ ids, const int* __restrict__ positions,
                                                         const int* __restrict__ req_of_token, const int* __restrict__ cu_q,
                                                         const int* __restrict__ slots, int* __restrict__ last_token,
                                                         int E, int V, int buckets, long long mul_prev, long long mul_cur,
                                                         float eps) {
    __shared__ float part[4];
    __shared__ int s_prev;
    const int t = blockIdx.x;
    const int id = ids[t];
    const int req = req_of_token[t];
    const int first = cu_q[req];
    if (pairs && threadIdx.x == 0) {
        s_prev = (t == first) ? last_token[slots[req]] : ids[t - 1];
    }
    __syncthreads();
    if (pairs && t == first && threadIdx.x == 0) last_token[slots[req]] = ids[cu_q[req + 1] - 1];
    const TW* row = table + (size_t)((id < 0 || id >= V) ? 0 : id) * E;
    const TW* prow = nullptr;
    if (pairs) {
        long long r = buckets;
        if (positions[t] != 0) {
            r = (((long long)s_prev % buckets) * mul_prev + ((long long)id % buckets) * mul_cur) % (long long)buckets;
            if (r < 0) r += buckets;
        }
        prow = pairs + (size_t)r * E;
    }
    float* o = out + (size_t)t * E;
    float ss = 0.f;
    for (int i = threadIdx.x; i < E; i += 256) {
        float v = ld<TW>(row, i);
        if (prow) v += ld<TW>(prow, i);
        o[i] = v;
        ss += v * v;
    }
    if (!w) return;
    const float rinv = 1.0f / sqrtf(block_sum_256(ss, part) / (float)E + eps);
    for (int i = threadIdx.x; i < E; i += 256) o[i] = o[i] * rinv * w[i];
}

extern "C" int xr_embedding_pairs(float* out, const void* table, const void* pairs, const float* norm_w, const int* ids,
                                  const int* positions, const int* req_of_token, const int* cu_q, const int* slots,
                                  int* last_token, int T, int E, int V, int buckets, int mul_prev, int mul_cur, float eps,
                                  int table_dtype, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && E > 0 && V > 0, "embedding_pairs: bad sizes T=%d E=%d V=%d", T, E, V);
    XR_REQUIRE(table_dtype == XR_F32 || table_dtype == XR_BF16, "embedding_pairs: bad dtype %d", table_dtype);
    XR_REQUIRE(!pairs || (buckets > 0 && mul_prev >= 0 && mul_cur >= 0 && last_token && slots && cu_q && req_of_token && positions),
               "embedding_pairs: a pair table needs buckets > 0, multipliers >= 0 and the step's rows");
    if (T == 0) return XR_OK;
    if (table_dtype == XR_F32)
        k_embedding_pairs<float><<<T, 256, 0, stream>>>(out, (const float*)table, (const float*)pairs, norm_w, ids, positions,
                                                        req_of_token, cu_q, slots, last_token, E, V, buckets, mul_prev, mul_cur, eps);
    else
        k_embedding_pairs<bf16_t><<<T, 256, 0, stream>>>(out, (const bf16_t*)table, (const bf16_t*)pairs, norm_w, ids, positions,
                                                         req_of_token, cu_q, slots, last_token, E, V, buckets, mul_prev, mul_cur, eps);
    XR_CHECK_LAUNCH("embedding_pairs");
    return XR_OK;
}

// ---------------------------------------------------------------- several residual streams
#define HC_MAX_STREAMS 8

// xs [S][T][E] <- x [T][E] in every copy
__global__ void k_streams_expand(float* __restrict__ xs, const float* __restrict__ x, size_t n, int S) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = x[i];
    for (int s = 0; s < S; ++s) xs[(size_t)s * n + i] = v;
}

// x [T][E] <- sum over the copies, in ascending order
__global__ void k_streams_sum(float* __restrict__ x, const float* __restrict__ xs, size_t n, int S) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = xs[i];
    for (int s = 1; s < S; ++s) v += xs[(size_t)s * n + i];
    x[i] = v;
}

extern "C" int xr_streams_expand(float* xs, const float* x, int T, int E, int S, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && E > 0 && S >= 1, "streams_expand: bad sizes T=%d E=%d S=%d", T, E, S);
    const size_t n = (size_t)T * E;
    if (n == 0) return XR_OK;
    k_streams_expand<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(xs, x, n, S);
    XR_CHECK_LAUNCH("streams_expand");
    return XR_OK;
}

extern "C" int xr_streams_sum(float* x, const float* xs, int T, int E, int S, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && E > 0 && S >= 1, "streams_sum: bad sizes T=%d E=%d S=%d", T, E, S);
    const size_t n = (size_t)T * E;
    if (n == 0) return XR_OK;
    k_streams_sum<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, xs, n, S);
    XR_CHECK_LAUNCH("streams_sum");
    return XR_OK;
}

// One step of the streams around a sublayer, a workgroup a row, both halves optional:
//   write (y given):  xs_t <- sum_s mix[s][t] xs_s + out_w[t] * y     for all t at once, from the old copies
//   read (h given):   u = sum_s in_w[s] xs_s;  h = u / sqrt(mean(u^2) + eps) * norm_w   (norm_w null: h = u)
// With both, the read sees the copies the write has just made (the write of one sublayer and the
// read of the next in one pass over the row).  A thread owns the columns i = tid, tid + 256, ...
// in both halves, so the read needs no barrier after the write.
template <typename TO>
__global__ __launch_bounds__(256) void k_streams_step(float* __restrict__ xs, const float* __restrict__ y,
                                                      const float* __restrict__ mix, const float* __restrict__ out_w,
                                                      const float* __restrict__ in_w, const float* __restrict__ norm_w,
                                                      TO* __restrict__ h, int T, int E, int S, float eps) {
    __shared__ float part[4];
    __shared__ float c_mix[HC_MAX_STREAMS * HC_MAX_STREAMS], c_out[HC_MAX_STREAMS], c_in[HC_MAX_STREAMS];
    const int t = blockIdx.x;
    if (threadIdx.x < S * S && y) c_mix[threadIdx.x] = mix[threadIdx.x];
    if (threadIdx.x < S) {
        if (y) c_out[threadIdx.x] = out_w[threadIdx.x];
        if (h) c_in[threadIdx.x] = in_w[threadIdx.x];
    }
    __syncthreads();
    const size_t plane = (size_t)T * E, base = (size_t)t * E;
    float ss = 0.f;
    for (int i = threadIdx.x; i < E; i += 256) {
        float v[HC_MAX_STREAMS];
#pragma unroll
        for (int s = 0; s < HC_MAX_STREAMS; ++s) v[s] = s < S ? xs[(size_t)s * plane + base + i] : 0.f;
        if (y) {
            const float yi = y[base + i];
            float nv[HC_MAX_STREAMS];
#pragma unroll
            for (int to = 0; to < HC_MAX_STREAMS; ++to) {
                float a = 0.f;
                if (to < S) {
                    for (int s = 0; s < S; ++s) a += c_mix[s * S + to] * v[s];
                    a += c_out[to] * yi;
                    xs[(size_t)to * plane + base + i] = a;
                }
                nv[to] = a;
            }
#pragma unroll
            for (int s = 0; s < HC_MAX_STREAMS; ++s) v[s] = nv[s];
        }
        if (h) {
            float u = 0.f;
            for (int s = 0; s < S; ++s) u += c_in[s] * v[s];
            ss += u * u;
            if (!norm_w) st<TO>(h, base + i, u);
        }
    }
    if (!h || !norm_w) return;
    const float rinv = 1.0f / sqrtf(block_sum_256(ss, part) / (float)E + eps);
    for (int i = threadIdx.x; i < E; i += 256) {
        float u = 0.f;
        for (int s = 0; s < S; ++s) u += c_in[s] * xs[(size_t)s * plane + base + i];
        st<TO>(h, base + i, u * rinv * norm_w[i]);
    }
}

// The same for rows whose width is a multiple of 4 (up to 4 * 256 * NV): a thread handles float4 pieces,
// and keeps u in registers between the sum and the scaling.
template <typename TO> __device__ inline void hc_store4(TO* p, size_t i, float a, float b, float c, float d);
template <> __device__ inline void hc_store4<float>(float* p, size_t i, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(p + i) = make_float4(a, b, c, d);
}
template <> __device__ inline void hc_store4<bf16_t>(bf16_t* p, size_t i, float a, float b, float c, float d) {
    uint2 w;
    w.x = pack_bf16x2(a, b);
    w.y = pack_bf16x2(c, d);
    *reinterpret_cast<uint2*>(p + i) = w;
}

template <typename TO, int NV>
__global__ __launch_bounds__(256) void k_streams_step_v4(float* __restrict__ xs, const float* __restrict__ y,
                                                         const float* __restrict__ mix, const float* __restrict__ out_w,
                                                         const float* __restrict__ in_w, const float* __restrict__ norm_w,
                                                         TO* __restrict__ h, int T, int E, int S, float eps) {
    __shared__ float part[4];
    __shared__ float c_mix[HC_MAX_STREAMS * HC_MAX_STREAMS], c_out[HC_MAX_STREAMS], c_in[HC_MAX_STREAMS];
    const int t = blockIdx.x;
    if (threadIdx.x < S * S && y) c_mix[threadIdx.x] = mix[threadIdx.x];
    if (threadIdx.x < S) {
        if (y) c_out[threadIdx.x] = out_w[threadIdx.x];
        if (h) c_in[threadIdx.x] = in_w[threadIdx.x];
    }
    __syncthreads();
    const size_t plane = (size_t)T * E, base = (size_t)t * E;
    const int n4 = E >> 2;
    float4 u[NV];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int c = threadIdx.x + j * 256;
        u[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c >= n4) continue;
        const size_t at = base + (size_t)c * 4;
        float4 v[HC_MAX_STREAMS];
#pragma unroll
        for (int s = 0; s < HC_MAX_STREAMS; ++s)
            if (s < S) v[s] = *reinterpret_cast<const float4*>(xs + (size_t)s * plane + at);
        if (y) {
            const float4 yi = *reinterpret_cast<const float4*>(y + at);
            float4 nv[HC_MAX_STREAMS];
#pragma unroll
            for (int to = 0; to < HC_MAX_STREAMS; ++to) {
                if (to >= S) continue;
                float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int s = 0; s < HC_MAX_STREAMS; ++s) {
                    if (s >= S) continue;
                    const float m = c_mix[s * S + to];
                    a.x += m * v[s].x; a.y += m * v[s].y; a.z += m * v[s].z; a.w += m * v[s].w;
                }
                const float ow = c_out[to];
                a.x += ow * yi.x; a.y += ow * yi.y; a.z += ow * yi.z; a.w += ow * yi.w;
                *reinterpret_cast<float4*>(xs + (size_t)to * plane + at) = a;
                nv[to] = a;
            }
#pragma unroll
            for (int s = 0; s < HC_MAX_STREAMS; ++s)
                if (s < S) v[s] = nv[s];
        }
        if (h) {
            float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int s = 0; s < HC_MAX_STREAMS; ++s) {
                if (s >= S) continue;
                const float m = c_in[s];
                a.x += m * v[s].x; a.y += m * v[s].y; a.z += m * v[s].z; a.w += m * v[s].w;
            }
            u[j] = a;
            ss += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
            if (!norm_w) hc_store4<TO>(h, at, a.x, a.y, a.z, a.w);
        }
    }
    if (!h || !norm_w) return;
    const float rinv = 1.0f / sqrtf(block_sum_256(ss, part) / (float)E + eps);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int c = threadIdx.x + j * 256;
        if (c >= n4) continue;
        const float4 w4 = *reinterpret_cast<const float4*>(norm_w + (size_t)c * 4);
        hc_store4<TO>(h, base + (size_t)c * 4, u[j].x * rinv * w4.x, u[j].y * rinv * w4.y, u[j].z * rinv * w4.z, u[j].w * rinv * w4.w);
    }
}

template <typename TO>
static void launch_streams_step(float* xs, const float* y, const float* mix, const float* out_w, const float* in_w,
                                const float* norm_w, TO* h, int T, int E, int S, float eps, hipStream_t stream) {
    const bool al = ((uintptr_t)xs % 16) == 0 && ((uintptr_t)y % 16) == 0 && ((uintptr_t)h % 16) == 0 && ((uintptr_t)norm_w % 16) == 0;
    if (al && E % 4 == 0 && E <= 4 * 256 * 8) {
        if (E <= 1024) k_streams_step_v4<TO, 1><<<T, 256, 0, stream>>>(xs, y, mix, out_w, in_w, norm_w, h, T, E, S, eps);
        else if (E <= 2048) k_streams_step_v4<TO, 2><<<T, 256, 0, stream>>>(xs, y, mix, out_w, in_w, norm_w, h, T, E, S, eps);
        else if (E <= 4096) k_streams_step_v4<TO, 4><<<T, 256, 0, stream>>>(xs, y, mix, out_w, in_w, norm_w, h, T, E, S, eps);
        else k_streams_step_v4<TO, 8><<<T, 256, 0, stream>>>(xs, y, mix, out_w, in_w, norm_w, h, T, E, S, eps);
    } else {
        k_streams_step<TO><<<T, 256, 0, stream>>>(xs, y, mix, out_w, in_w, norm_w, h, T, E, S, eps);
    }
}

extern "C" int xr_streams_step(float* xs, const float* y, const float* mix, const float* out_w, const float* in_w,
                               const float* norm_w, void* h, int T, int E, int S, float eps, int h_dtype, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && E > 0 && S >= 1 && S <= HC_MAX_STREAMS, "streams_step: bad sizes T=%d E=%d S=%d (at most %d streams)", T, E, S,
               HC_MAX_STREAMS);
    XR_REQUIRE(!y || (mix && out_w), "streams_step: the write needs mix and out weights");
    XR_REQUIRE(!h || in_w, "streams_step: the read needs in weights");
    XR_REQUIRE(y || h, "streams_step: nothing to do");
    if (T == 0) return XR_OK;
    if (!h || h_dtype == XR_F32)
        launch_streams_step<float>(xs, y, mix, out_w, in_w, norm_w, (float*)h, T, E, S, eps, stream);
    else if (h_dtype == XR_BF16)
        launch_streams_step<bf16_t>(xs, y, mix, out_w, in_w, norm_w, (bf16_t*)h, T, E, S, eps, stream);
    else { xr_set_error("streams_step: bad dtype %d", h_dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("streams_step");
    return XR_OK;
}
