// What stands between the q|k|v projection and the attention of a mixer whose projected queries, keys
// and values each pass a short causal convolution over time before the rotation:
//
//   y_t[c] = sum_{j=0}^{taps-1} w[c][j] u_(t - taps + 1 + j)[c]        (zeros before a request's start)
//
// on every channel c of the packed row u = [q heads | k heads | v heads], then the half-split rotation
// of the first rot_dims numbers of every q and k head (the pair (i, i + rot_dims / 2) turned by
// position * inv_freq[i], angle, sine and cosine formed in 32-bit), then q to q_out and k and v into the
// paged cache at the token's slot.  Key and value heads may have different sizes (Dk, Dv): q_out and
// the cache use one head size Dc >= both, and what lies beyond a head's own numbers is written as
// zeros (a zero adds nothing to a score, and the rows of the output projection beyond Dv meet zeros).
//
// What lies before a portion comes from the request's state: its last taps - 1 projected rows,
// state[slot][j] being the row at position (tokens so far) - (taps - 1) + j.  The rows of one request are
// consecutive, so a row finds its place in its portion by looking back along tok_seq.  The sum runs
// oldest input first: the same order however the request was cut.
//
// A thread owns one channel, or the two channels of a rotated pair (the thread of the pair's first
// number does both, the thread of the second leaves): every channel's state is read by one thread only,
// which in a step of single new tokens also moves it up by one (one launch for everything).
//
// cache of one layer: [page][2 (k, v)][Hkv][P * Dc]; a key tile is [P][Dc], a value tile [Dc][P].
#include "common.h"

template <typename TA>
struct ConvArgs {
    const TA* u;              // [T, C]
    const float* w;           // [C, taps]
    float* state;             // [slots, taps - 1, C]
    const int* tok_seq;
    int T, C, taps;
};

// the convolution of channel c at row t; with SHIFT the state of the channel is moved up by one as well
template <typename TA, bool SHIFT>
__device__ __forceinline__ float conv_channel(const ConvArgs<TA>& a, long t, int c, int s, int before) {
    const int n1 = a.taps - 1;
    const float* wc = a.w + (long)c * a.taps;
    float acc = 0.f;
    if (SHIFT) {
        float* st = a.state + (long)s * n1 * a.C + c;
        for (int j = 0; j < n1; ++j) {
            const float v = st[(long)j * a.C];
            acc = fmaf(wc[j], v, acc);
            if (j > 0) st[(long)(j - 1) * a.C] = v;
        }
        const float ut = Elem<TA>::load(a.u + t * a.C + c);
        if (n1 > 0) st[(long)(n1 - 1) * a.C] = ut;
        return fmaf(wc[n1], ut, acc);
    }
    for (int k = n1; k >= 0; --k) {
        float v;
        if (k <= before) v = Elem<TA>::load(a.u + (t - k) * a.C + c);
        else v = a.state[((long)s * n1 + (n1 - k + before)) * a.C + c];
        acc = fmaf(wc[n1 - k], v, acc);
    }
    return acc;
}

template <typename TA, bool SHIFT>
__global__ void qkv_conv_rope_store_kernel(ConvArgs<TA> a, const int* __restrict__ positions,
                                           const float* __restrict__ inv_freq, const int* __restrict__ slots,
                                           TA* __restrict__ q_out, TA* __restrict__ cache,
                                           int Hq, int Hkv, int Dk, int Dv, int Dc, int P, int rot_dims) {
    const int x = blockIdx.x * blockDim.x + threadIdx.x;      // a coordinate of the padded row [Hq + 2 Hkv][Dc]
    const long t = blockIdx.y;
    if (x >= (Hq + 2 * Hkv) * Dc) return;
    const int hh = x / Dc, d = x % Dc;
    const int half = rot_dims / 2;
    const bool is_q = hh < Hq, is_k = !is_q && hh < Hq + Hkv;
    const int own = is_q || is_k ? Dk : Dv;                   // the head's own numbers
    const bool rotated = (is_q || is_k) && d < rot_dims;
    if (rotated && d >= half) return;                         // the pair's first thread does both
    const int s = a.tok_seq[t];
    const int slot = slots ? slots[t] : -1;
    // where the coordinate goes: q_out, or the cache (a key row, a value column)
    TA* dst = nullptr;
    long step = 1;                                            // distance of the pair's second number
    if (is_q) {
        dst = q_out + (t * Hq + hh) * Dc + d;
    } else if (slot >= 0) {
        const long page = slot / P;
        const int off = slot % P;
        const long page_stride = 2L * Hkv * P * Dc;
        if (is_k) dst = cache + page * page_stride + ((long)(hh - Hq) * P + off) * Dc + d;
        else { dst = cache + page * page_stride + ((long)(hh - Hq) * P) * Dc + (long)d * P + off; step = P; }
    }
    if (d >= own) {                                           // beyond the head's own numbers
        if (dst) Elem<TA>::store(dst, 0.f);
        return;
    }
    const int c = is_q ? hh * Dk + d : (is_k ? Hq * Dk + (hh - Hq) * Dk + d : (Hq + Hkv) * Dk + (hh - Hq - Hkv) * Dv + d);
    int before = 0;                                           // rows of the same request right before this one, up to taps - 1
    if (!SHIFT)
        while (before < a.taps - 1 && t - 1 - before >= 0 && a.tok_seq[t - 1 - before] == s) ++before;
    float y0 = conv_channel<TA, SHIFT>(a, t, c, s, before);
    if (rotated) {
        float y1 = conv_channel<TA, SHIFT>(a, t, c + half, s, before);
        const float angle = (float)positions[t] * inv_freq[d];
        float sn, cs;
        sincosf(angle, &sn, &cs);
        rotate_pair(cs, sn, y0, y1);
        if (dst) Elem<TA>::store(dst + half * step, y1);
    }
    if (dst) Elem<TA>::store(dst, y0);
}

// After the convolution: the state takes the portion's last taps - 1 rows.  A portion shorter than
// that moves the state's old entries up first; its first row's thread does all of it, so that no
// thread reads what another writes.
template <typename TA>
__global__ void qkv_conv_state_kernel(ConvArgs<TA> a) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const long t = blockIdx.y;
    if (c >= a.C) return;
    const int n1 = a.taps - 1;
    const int s = a.tok_seq[t];
    int before = 0, after = 0;
    while (before < n1 && t - 1 - before >= 0 && a.tok_seq[t - 1 - before] == s) ++before;
    while (after < n1 && t + 1 + after < a.T && a.tok_seq[t + 1 + after] == s) ++after;
    float* st = a.state + (long)s * n1 * a.C + c;
    if (before + after + 1 < n1) {                            // the whole portion is shorter than the state
        if (before != 0) return;
        const int q = after + 1;
        for (int j = 0; j + q < n1; ++j) st[(long)j * a.C] = st[(long)(j + q) * a.C];
        for (int m = 0; m < q; ++m) st[(long)(n1 - q + m) * a.C] = Elem<TA>::load(a.u + (t + m) * a.C + c);
    } else if (after < n1) {
        st[(long)(n1 - 1 - after) * a.C] = Elem<TA>::load(a.u + t * a.C + c);
    }
}

template <typename TA>
static int launch_conv_rope_store(const void* u, const float* w, float* state, const int* tok_seq, const int* positions,
                                  const float* inv_freq, const int* slots, void* q_out, void* cache, int T, int Hq,
                                  int Hkv, int Dk, int Dv, int Dc, int P, int taps, int rot_dims, int single,
                                  hipStream_t stream) {
    ConvArgs<TA> a{(const TA*)u, w, state, tok_seq, T, Hq * Dk + Hkv * (Dk + Dv), taps};
    const int width = (Hq + 2 * Hkv) * Dc;
    const int threads = width >= 256 ? 256 : 64;
    dim3 grid(qe_cdiv(width, threads), T);
    if (single && taps > 1) {
        qkv_conv_rope_store_kernel<TA, true><<<grid, threads, 0, stream>>>(a, positions, inv_freq, slots, (TA*)q_out,
                                                                            (TA*)cache, Hq, Hkv, Dk, Dv, Dc, P, rot_dims);
        return 0;
    }
    qkv_conv_rope_store_kernel<TA, false><<<grid, threads, 0, stream>>>(a, positions, inv_freq, slots, (TA*)q_out,
                                                                         (TA*)cache, Hq, Hkv, Dk, Dv, Dc, P, rot_dims);
    if (taps > 1) {
        const int th = a.C >= 256 ? 256 : 64;
        qkv_conv_state_kernel<TA><<<dim3(qe_cdiv(a.C, th), T), th, 0, stream>>>(a);
    }
    return 0;
}

// u [T, Hq Dk + Hkv Dk + Hkv Dv] in the activation type; w float [that many, taps]; state float [slots, taps - 1,
// that many] (row tok_seq[t]; null when taps is 1); inv_freq float [rot_dims / 2] (null when rot_dims is 0);
// slots [T] (negative: the row's key and value go nowhere), or null; q_out [T, Hq, Dc]; cache [pages, 2, Hkv, P, Dc].
// single: the caller knows that no two rows belong to the same request.
extern "C" int qe_qkv_conv_rope_store(const void* u, const float* w, float* state, const int* tok_seq,
                                      const int* positions, const float* inv_freq, const int* slots, void* q_out,
                                      void* cache, int T, int Hq, int Hkv, int Dk, int Dv, int Dc, int P, int taps,
                                      int rot_dims, int single, int dt_a, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && Hq > 0 && Hkv > 0 && Dk > 0 && Dv > 0 && P > 0 && taps >= 1, "qkv_conv_rope_store: bad sizes");
    QE_REQUIRE(Dc >= Dk && Dc >= Dv, "qkv_conv_rope_store: the common head size %d is smaller than %d or %d", Dc, Dk, Dv);
    QE_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= Dk, "qkv_conv_rope_store: %d rotated numbers of %d", rot_dims, Dk);
    QE_REQUIRE(taps == 1 || state, "qkv_conv_rope_store: %d taps need a state", taps);
    QE_REQUIRE(rot_dims == 0 || (inv_freq && positions), "qkv_conv_rope_store: a rotation needs positions and frequencies");
    QE_REQUIRE(!slots || cache, "qkv_conv_rope_store: slots without a cache");
    QE_REQUIRE(T <= 65535, "qkv_conv_rope_store: more than 65535 rows in a step");
    if (T == 0) return 0;
    int rc;
    if (dt_a == QE_F32)
        rc = launch_conv_rope_store<float>(u, w, state, tok_seq, positions, inv_freq, slots, q_out, cache, T, Hq, Hkv, Dk, Dv,
                                           Dc, P, taps, rot_dims, single, stream);
    else if (dt_a == QE_BF16)
        rc = launch_conv_rope_store<bf16_t>(u, w, state, tok_seq, positions, inv_freq, slots, q_out, cache, T, Hq, Hkv, Dk,
                                            Dv, Dc, P, taps, rot_dims, single, stream);
    else
        QE_REQUIRE(false, "qkv_conv_rope_store: unknown element type %d", dt_a);
    if (rc) return rc;
    QE_LAUNCH_CHECK();
    return 0;
}

__global__ void scale_kernel(float* __restrict__ x, long n, float s) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] *= s;
}

// x *= s on a 32-bit tensor (an embedding's scale, on the stream)
extern "C" int qe_scale_f32(float* x, long n, float s, hipStream_t stream) {
    QE_REQUIRE(n >= 0, "scale: bad size");
    if (n == 0) return 0;
    scale_kernel<<<qe_cdiv(n, 256), 256, 0, stream>>>(x, n, s);
    QE_LAUNCH_CHECK();
    return 0;
}
