// Linear recurrences over time with a matrix of state per request and head, in 32-bit floats:
//
//   retention:   S <- decay_h S + k v^T;                            o = S^T q
//   delta rule:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//
// S is [D, Dv] and its columns never meet: column c only needs v[c], so a thread group of four
// lanes owns one column (lane r the rows r, r+4, r+8, ...), keeps it in registers over the whole
// portion and the two sums over D are a few fused multiply-adds and two lane exchanges a token.
// A workgroup is 64 columns of one (request, head); queries and keys of a few tokens at a time
// are staged in LDS, rows of a lane side by side so that they are read four at a time.
// The same kernel runs a prompt's portion and a decoded token (a portion of one).
//
// State in memory: [slot][head][J = ceil(D/4)][Dv][4], i.e. S[4 j + r][c] at ((j * Dv) + c) * 4 + r:
// a wave's loads and stores are contiguous.  Rows past D (when D is no multiple of 4) stay zero.
#include "common.h"

#define REC_COLS 64          // columns of S a workgroup owns
#define REC_TOKENS 8         // tokens staged at a time
#define XR_REC_RETENTION 0
#define XR_REC_DELTA 1

struct RecArgs {
    float* out;              // [T, H, Dv]
    const float* q;          // [T, ld] at the first query head; G heads of D
    const float* k;
    const float* v;          // H heads of Dv
    const float* beta;       // [T, ld_g] at head 0 (delta rule)
    const float* gate;       // [T, ld_g] at head 0: the decay of every token and head (delta rule)
    const float* decay;      // [H] (retention)
    float* state;
    const int* cu_q;
    const int* slots;
    int H, G, D, Dv, ld, ld_g;   // row strides of q/k/v and of beta/gate
};

template <int MODE, int DPER>
__global__ __launch_bounds__(256) void k_recurrence(RecArgs a) {
    __shared__ float4 qs[REC_TOKENS][DPER];        // [token][r * (DPER/4) + j/4] as lanes read them
    __shared__ float4 ks[REC_TOKENS][DPER];
    __shared__ float vs[REC_TOKENS][REC_COLS];
    __shared__ float bs[REC_TOKENS], gs[REC_TOKENS];
    const int b = blockIdx.z, h = blockIdx.y, tid = threadIdx.x;
    const int cl = tid >> 2, r = tid & 3;
    const int col = blockIdx.x * REC_COLS + cl;
    const bool live = col < a.Dv;
    const int row0 = a.cu_q[b], n = a.cu_q[b + 1] - row0;
    if (n <= 0) return;
    const int kvh = h / (a.H / a.G);
    const int J = (a.D + 3) >> 2;
    float* sp = a.state + (((size_t)a.slots[b] * a.H + h) * J) * a.Dv * 4;
    float S[DPER];
#pragma unroll
    for (int j = 0; j < DPER; ++j) S[j] = (live && j < J) ? sp[((size_t)j * a.Dv + col) * 4 + r] : 0.f;
    const float dec = MODE == XR_REC_RETENTION ? a.decay[h] : 1.f;
    float* qf = reinterpret_cast<float*>(&qs[0][0]);
    float* kf = reinterpret_cast<float*>(&ks[0][0]);

    for (int c0 = 0; c0 < n; c0 += REC_TOKENS) {
        const int nt = n - c0 < REC_TOKENS ? n - c0 : REC_TOKENS;
        __syncthreads();
        // element d = 4 j + rr of a token goes to place rr * DPER + j; places past D hold zero
        for (int idx = tid; idx < nt * 4 * DPER; idx += 256) {
            const int tt = idx / (4 * DPER), e = idx - tt * 4 * DPER;
            const int rr = e / DPER, j = e - rr * DPER, d = 4 * j + rr;
            const size_t row = (size_t)(row0 + c0 + tt) * a.ld + (size_t)kvh * a.D;
            qf[idx] = d < a.D ? a.q[row + d] : 0.f;
            kf[idx] = d < a.D ? a.k[row + d] : 0.f;
        }
        for (int idx = tid; idx < nt * REC_COLS; idx += 256) {
            const int tt = idx / REC_COLS, c = idx - tt * REC_COLS;
            const int cc = blockIdx.x * REC_COLS + c;
            vs[tt][c] = cc < a.Dv ? a.v[(size_t)(row0 + c0 + tt) * a.ld + (size_t)h * a.Dv + cc] : 0.f;
        }
        if (MODE == XR_REC_DELTA && tid < nt) {
            bs[tid] = a.beta[(size_t)(row0 + c0 + tid) * a.ld_g + h];
            gs[tid] = a.gate[(size_t)(row0 + c0 + tid) * a.ld_g + h];
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float4* kq = &ks[tt][r * (DPER / 4)];
            const float4* qq = &qs[tt][r * (DPER / 4)];
            const float vv = vs[tt][cl];
            float o = 0.f;
            if (MODE == XR_REC_DELTA) {
                const float g = gs[tt];
                float dot = 0.f;
#pragma unroll
                for (int j = 0; j < DPER; j += 4) {
                    const float4 kk = kq[j >> 2];
                    S[j] *= g; S[j + 1] *= g; S[j + 2] *= g; S[j + 3] *= g;
                    dot = fmaf(S[j], kk.x, dot); dot = fmaf(S[j + 1], kk.y, dot);
                    dot = fmaf(S[j + 2], kk.z, dot); dot = fmaf(S[j + 3], kk.w, dot);
                }
                dot += __shfl_xor(dot, 1, 64);
                dot += __shfl_xor(dot, 2, 64);
                const float u = bs[tt] * (vv - dot);
#pragma unroll
                for (int j = 0; j < DPER; j += 4) {
                    const float4 kk = kq[j >> 2];
                    const float4 q4 = qq[j >> 2];
                    S[j] = fmaf(kk.x, u, S[j]); S[j + 1] = fmaf(kk.y, u, S[j + 1]);
                    S[j + 2] = fmaf(kk.z, u, S[j + 2]); S[j + 3] = fmaf(kk.w, u, S[j + 3]);
                    o = fmaf(S[j], q4.x, o); o = fmaf(S[j + 1], q4.y, o);
                    o = fmaf(S[j + 2], q4.z, o); o = fmaf(S[j + 3], q4.w, o);
                }
            } else {
#pragma unroll
                for (int j = 0; j < DPER; j += 4) {
                    const float4 kk = kq[j >> 2];
                    const float4 q4 = qq[j >> 2];
                    S[j] = fmaf(dec, S[j], kk.x * vv); S[j + 1] = fmaf(dec, S[j + 1], kk.y * vv);
                    S[j + 2] = fmaf(dec, S[j + 2], kk.z * vv); S[j + 3] = fmaf(dec, S[j + 3], kk.w * vv);
                    o = fmaf(S[j], q4.x, o); o = fmaf(S[j + 1], q4.y, o);
                    o = fmaf(S[j + 2], q4.z, o); o = fmaf(S[j + 3], q4.w, o);
                }
            }
            o += __shfl_xor(o, 1, 64);
            o += __shfl_xor(o, 2, 64);
            if (live && r == 0) a.out[((size_t)(row0 + c0 + tt) * a.H + h) * a.Dv + col] = o;
        }
    }
    if (live) {
#pragma unroll
        for (int j = 0; j < DPER; ++j)
            if (j < J) sp[((size_t)j * a.Dv + col) * 4 + r] = S[j];
    }
}

extern "C" int xr_state_rows_per_head(int D) { return (D + 3) / 4; }

extern "C" int xr_linear_recurrence(float* out, const float* q, const float* k, const float* v, const float* beta,
                                    const float* gate, const float* decay, float* state, const int* cu_q,
                                    const int* slots, int B, int H, int G, int D, int Dv, int ld, int ld_g, int mode,
                                    hipStream_t stream) {
    XR_REQUIRE(B >= 0 && H > 0 && G > 0 && H % G == 0, "recurrence: %d heads over %d key heads", H, G);
    XR_REQUIRE(D > 0 && D <= 256 && Dv > 0, "recurrence: key size %d (1 to 256), value size %d", D, Dv);
    XR_REQUIRE(mode == XR_REC_RETENTION || mode == XR_REC_DELTA, "recurrence: mode %d", mode);
    XR_REQUIRE(mode == XR_REC_RETENTION ? decay != nullptr : (beta != nullptr && gate != nullptr),
               "recurrence: the mode's gates are missing");
    XR_REQUIRE(out && q && k && v && state && cu_q && slots, "recurrence: a pointer is missing");
    if (B == 0) return XR_OK;
    RecArgs a{out, q, k, v, beta, gate, decay, state, cu_q, slots, H, G, D, Dv, ld, ld_g};
    dim3 grid((Dv + REC_COLS - 1) / REC_COLS, H, B);
    const int per = (D + 3) / 4;
#define REC(M)                                                                          \
    do {                                                                                \
        if (per <= 8) k_recurrence<M, 8><<<grid, 256, 0, stream>>>(a);                  \
        else if (per <= 16) k_recurrence<M, 16><<<grid, 256, 0, stream>>>(a);           \
        else if (per <= 32) k_recurrence<M, 32><<<grid, 256, 0, stream>>>(a);           \
        else k_recurrence<M, 64><<<grid, 256, 0, stream>>>(a);                          \
    } while (0)
    if (mode == XR_REC_DELTA) REC(XR_REC_DELTA);
    else REC(XR_REC_RETENTION);
#undef REC
    XR_CHECK_LAUNCH("linear_recurrence");
    return XR_OK;
}
