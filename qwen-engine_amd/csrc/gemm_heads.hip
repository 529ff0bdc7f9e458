// A matrix product per head: out[t, h, :] = W_h x[t, h, :], W [H, N, K], for all heads in one launch.
// x and out are addressed with a row and a head stride of their own (in elements), so the product can
// read a part of each head of a wider tensor and write into a part of each head of another (the
// unrotated part of the queries into the packed queries).  With ``gate`` ([T, H * N], the activation
// type) the result is multiplied by sigmoid(gate) before it is stored.
//
// Any sizes, every multiply-add in IEEE 32-bit, each output summed over k in ascending order whatever
// T is.  64x64 output tile per block of 256 threads, 4x4 outputs per thread, K in steps of 16 through
// shared memory; blockIdx.z is the head.
#include "common.h"

#define HT 64
#define HK 16

template <typename TA, typename TW>
__global__ __launch_bounds__(256) void gemm_heads_kernel(
    const TA* __restrict__ x, long xs_t, long xs_h, const TW* __restrict__ w, TA* __restrict__ out, long os_t,
    long os_h, const TA* __restrict__ gate, int T, int N, int K) {
    __shared__ float xs[HK][HT + 4];
    __shared__ float ws[HK][HT + 4];
    const int tid = threadIdx.x;
    const int h = blockIdx.z;
    const int m0 = blockIdx.y * HT, n0 = blockIdx.x * HT;
    const int lr = tid >> 2;
    const int lk = (tid & 3) * 4;
    const int ty = tid >> 4, tx = tid & 15;
    const TA* xh = x + h * xs_h;
    const TW* wh = w + (long)h * N * K;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < K; k0 += HK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int m = m0 + lr, n = n0 + lr;
            xs[lk + i][lr] = (m < T && k < K) ? Elem<TA>::load(xh + (long)m * xs_t + k) : 0.f;
            ws[lk + i][lr] = (n < N && k < K) ? Elem<TW>::load(wh + (long)n * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < HK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
    const int H = gridDim.z;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= T) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (gate) {
                const float g = Elem<TA>::load(gate + ((long)m * H + h) * N + n);
                v = v / (1.f + expf(-g));
            }
            Elem<TA>::store(out + (long)m * os_t + h * os_h + n, v);
        }
    }
}

extern "C" int qe_gemm_heads(const void* x, long xs_t, long xs_h, const void* w, void* out, long os_t, long os_h,
                             const void* gate, int T, int H, int N, int K, int dt_a, int dt_w, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && H > 0 && N > 0 && K > 0, "gemm_heads: bad sizes T=%d H=%d N=%d K=%d", T, H, N, K);
    QE_REQUIRE(H <= 65535 && qe_cdiv(T, HT) <= 65535, "gemm_heads: too many heads or rows for one launch");
    if (T == 0) return 0;
    dim3 grid(qe_cdiv(N, HT), qe_cdiv(T, HT), H);
#define QE_GH(TA_, TW_) gemm_heads_kernel<TA_, TW_><<<grid, 256, 0, stream>>>((const TA_*)x, xs_t, xs_h, (const TW_*)w, (TA_*)out, os_t, os_h, (const TA_*)gate, T, N, K)
    if (dt_a == QE_F32 && dt_w == QE_F32) QE_GH(float, float);
    else if (dt_a == QE_BF16 && dt_w == QE_BF16) QE_GH(bf16_t, bf16_t);
    else if (dt_a == QE_BF16 && dt_w == QE_F32) QE_GH(bf16_t, float);
    else QE_REQUIRE(false, "gemm_heads: no kernel for element types x=%d w=%d", dt_a, dt_w);
#undef QE_GH
    QE_LAUNCH_CHECK();
    return 0;
}
