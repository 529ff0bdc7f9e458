// A short causal convolution over time on each channel of the 32-bit stream, added to its input:
//   out_t = x_t + sum_{k=0}^{taps-1} w[:, taps-1-k] * x_(t-k)        (zeros before a request's start)
// over a flat batch of portions of several requests.  What lies before a portion comes from the
// request's state: its last taps - 1 inputs, state[slot][j] being the input at position
// (tokens so far) - (taps - 1) + j, zeros where that is negative (the state of a new request is
// cleared by the step function).
//
// The rows of one request are consecutive and no request comes twice in a step, so a row finds its
// place inside its portion by looking back: row t - k belongs to the same request exactly if its
// table row (tok_seq) is the same.  No list of portions is needed, and a recorded step's rows that
// only fill it up (all on the tables' spare row) are taken as one portion.
#include "common.h"

template <typename TA>
__global__ void short_conv_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                  const float* __restrict__ state, const int* __restrict__ tok_seq,
                                  TA* __restrict__ out, int T, int H, int taps) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const long t = blockIdx.y;
    if (c >= H) return;
    const int n1 = taps - 1;
    const int s = tok_seq[t];
    int before = 0;                                   // rows of the same request right before this one, up to n1
    while (before < n1 && t - 1 - before >= 0 && tok_seq[t - 1 - before] == s) ++before;
    const float* wc = w + (long)c * taps;
    const float xt = x[t * H + c];
    float acc = xt;
    for (int k = n1; k >= 0; --k) {                   // oldest input first: the same order however the request was cut
        float v;
        if (k <= before) v = x[(t - k) * H + c];
        else v = state[((long)s * n1 + (n1 - k + before)) * H + c];
        acc = fmaf(wc[n1 - k], v, acc);
    }
    Elem<TA>::store(out + t * H + c, acc);
}

// After the convolution: the state takes the portion's last taps - 1 inputs.  A portion shorter than
// that moves the state's old entries up first; its first row's thread does all of it, so that no
// thread reads what another writes.
__global__ void short_conv_update_kernel(const float* __restrict__ x, float* __restrict__ state,
                                         const int* __restrict__ tok_seq, int T, int H, int taps) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const long t = blockIdx.y;
    if (c >= H) return;
    const int n1 = taps - 1;
    const int s = tok_seq[t];
    int before = 0, after = 0;
    while (before < n1 && t - 1 - before >= 0 && tok_seq[t - 1 - before] == s) ++before;
    while (after < n1 && t + 1 + after < T && tok_seq[t + 1 + after] == s) ++after;
    float* st = state + (long)s * n1 * H + c;
    if (before + after + 1 < n1) {                    // the whole portion is shorter than the state
        if (before != 0) return;
        const int q = after + 1;
        for (int j = 0; j + q < n1; ++j) st[(long)j * H] = st[(long)(j + q) * H];
        for (int m = 0; m < q; ++m) st[(long)(n1 - q + m) * H] = x[(t + m) * H + c];
    } else if (after < n1) {
        st[(long)(n1 - 1 - after) * H] = x[t * H + c];
    }
}

// Every row the only row of its request (single new tokens): the convolution and the state's shift in one launch;
// a thread reads its channel's state, forms the output and writes the state back moved up by one.
template <typename TA>
__global__ void short_conv_single_kernel(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ state,
                                         const int* __restrict__ tok_seq, TA* __restrict__ out, int H, int taps) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const long t = blockIdx.y;
    if (c >= H) return;
    const int n1 = taps - 1;
    float* st = state + (long)tok_seq[t] * n1 * H + c;
    const float* wc = w + (long)c * taps;
    const float xt = x[t * H + c];
    float acc = xt;
    for (int j = 0; j < n1; ++j) {                    // oldest input first, as in short_conv_kernel
        const float v = st[(long)j * H];
        acc = fmaf(wc[j], v, acc);
        if (j > 0) st[(long)(j - 1) * H] = v;
    }
    acc = fmaf(wc[n1], xt, acc);
    st[(long)(n1 - 1) * H] = xt;
    Elem<TA>::store(out + t * H + c, acc);
}

// update 2: the caller knows that every row is the only row of its request
extern "C" int qe_short_conv(const float* x, const float* w, float* state, const int* tok_seq, void* out,
                             int dt_a, int T, int H, int taps, int update, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && H > 0 && taps >= 1, "short_conv: bad sizes T=%d H=%d taps=%d", T, H, taps);
    QE_REQUIRE(taps == 1 || state, "short_conv: %d taps need a state", taps);
    QE_REQUIRE(T <= 65535, "short_conv: more than 65535 rows in a step");
    if (T == 0) return 0;
    const int threads = H >= 256 ? 256 : 64;
    dim3 grid(qe_cdiv(H, threads), T);                // (blockIdx.y is the row)
    if (update == 2 && taps > 1) {
        if (dt_a == QE_F32) short_conv_single_kernel<float><<<grid, threads, 0, stream>>>(x, w, state, tok_seq, (float*)out, H, taps);
        else if (dt_a == QE_BF16) short_conv_single_kernel<bf16_t><<<grid, threads, 0, stream>>>(x, w, state, tok_seq, (bf16_t*)out, H, taps);
        else QE_REQUIRE(false, "short_conv: unknown output type %d", dt_a);
        QE_LAUNCH_CHECK();
        return 0;
    }
    if (dt_a == QE_F32)
        short_conv_kernel<float><<<grid, threads, 0, stream>>>(x, w, state, tok_seq, (float*)out, T, H, taps);
    else if (dt_a == QE_BF16)
        short_conv_kernel<bf16_t><<<grid, threads, 0, stream>>>(x, w, state, tok_seq, (bf16_t*)out, T, H, taps);
    else
        QE_REQUIRE(false, "short_conv: unknown output type %d", dt_a);
    QE_LAUNCH_CHECK();
    if (update && taps > 1) {
        short_conv_update_kernel<<<grid, threads, 0, stream>>>(x, state, tok_seq, T, H, taps);
        QE_LAUNCH_CHECK();
    }
    return 0;
}
