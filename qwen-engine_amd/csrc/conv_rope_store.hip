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

// The same sum (oldest input first) for up to CONV_UNROLL taps, with all of a channel's loads issued before the
// first is used: a loop over a number of taps known only at run time waits for every load in turn, and a thread's
// few coordinates then cost a trip to memory each and per tap.
#define CONV_UNROLL 8
template <typename TA>
__device__ __forceinline__ float conv_channel_ahead(const ConvArgs<TA>& a, long t, int c, int s, int before) {
    const int n1 = a.taps - 1;
    if (n1 >= CONV_UNROLL) return conv_channel<TA, false>(a, t, c, s, before);
    const float* wc = a.w + (long)c * a.taps;
    float v[CONV_UNROLL], wv[CONV_UNROLL];
#pragma unroll
    for (int j = 0; j < CONV_UNROLL; ++j) {                   // the j-th oldest input lies k = n1 - j rows back
        const int k = n1 - j;
        v[j] = 0.f;
        wv[j] = 0.f;
        if (k >= 0) {
            wv[j] = wc[j];
            if (k <= before) v[j] = Elem<TA>::load(a.u + (t - k) * a.C + c);
            else v[j] = a.state[((long)s * n1 + (j + before)) * a.C + c];
        }
    }
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < CONV_UNROLL; ++j)
        if (j <= n1) acc = fmaf(wv[j], v[j], acc);
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

// Many rows (portions of prompts): a block per (16 consecutive rows of the batch, head).  Every row's place in its
// portion is looked up once, the cosines and sines of its position once per pair; query and key heads are
// written as they are computed (whole rows of a head side by side); a value head is first turned round in shared
// memory, because the cache holds value tiles as [Dc][P]: where eight of the block's rows lie side by side in one
// page (rows of one request do), their eight values of a feature are one store of 16 or 32 bytes instead of eight
// stores of one number each, 32 bytes apart.  (A thread per coordinate with its own look-back, its own sine and
// single stores took 58 + 25 us for 2048 rows of 3072 coordinates.)
#define CT_ROWS 16
template <typename TA>
__global__ __launch_bounds__(256) void qkv_conv_rope_store_tile_kernel(
    ConvArgs<TA> a, const int* __restrict__ positions, const float* __restrict__ inv_freq,
    const int* __restrict__ slots, TA* __restrict__ q_out, TA* __restrict__ cache, int Hq, int Hkv, int Dk, int Dv,
    int Dc, int P, int rot_dims) {
    extern __shared__ float tile_lds[];                       // [CT_ROWS][rot_dims] cos | sin, or the value tile [Dv][CT_ROWS + 1]
    __shared__ int before_lds[CT_ROWS], seq_lds[CT_ROWS], slot_lds[CT_ROWS], off_lds[CT_ROWS];
    __shared__ long page_lds[CT_ROWS];                        // elements from the cache's start to the row's page; -1: no slot
    const long t0 = (long)blockIdx.x * CT_ROWS;
    const int rows = a.T - t0 < CT_ROWS ? (int)(a.T - t0) : CT_ROWS;
    const int hh = blockIdx.y;
    const int half = rot_dims / 2;
    const bool is_q = hh < Hq, is_k = !is_q && hh < Hq + Hkv;
    const int own = is_q || is_k ? Dk : Dv;
    const int c0 = is_q ? hh * Dk : (is_k ? Hq * Dk + (hh - Hq) * Dk : (Hq + Hkv) * Dk + (hh - Hq - Hkv) * Dv);
    const long page_stride = 2L * Hkv * P * Dc;
    if (threadIdx.x < rows) {
        const long t = t0 + threadIdx.x;
        const int s = a.tok_seq[t];
        int before = 0;                                       // rows of the same request right before this one, up to taps - 1
        while (before < a.taps - 1 && t - 1 - before >= 0 && a.tok_seq[t - 1 - before] == s) ++before;
        before_lds[threadIdx.x] = before;
        seq_lds[threadIdx.x] = s;
        const int slot = slots ? slots[t] : -1;
        slot_lds[threadIdx.x] = slot;
        page_lds[threadIdx.x] = slot >= 0 ? (long)(slot / P) * page_stride : -1;
        off_lds[threadIdx.x] = slot >= 0 ? slot % P : 0;
    }
    // (divisions by sizes known only at run time cost dozens of instructions each: one per thread here, none per item.
    // A thread keeps its feature d and walks the rows r, r + r_step, ...; heads wider than the block walk d as well.)
    const int r_first = Dc <= (int)blockDim.x ? threadIdx.x / Dc : 0;
    const int d_first = Dc <= (int)blockDim.x ? threadIdx.x - r_first * Dc : threadIdx.x;
    const int r_step = Dc <= (int)blockDim.x ? blockDim.x / Dc : 1;
    const int d_step = Dc <= (int)blockDim.x ? Dc : blockDim.x;       // (Dc: one pass over d)
    const bool idle = Dc <= (int)blockDim.x && r_first >= r_step;    // threads beyond the last whole row of a pass
    if ((is_q || is_k) && half > 0 && !idle) {
        for (int r = r_first; r < rows; r += r_step) {
            const float pos = (float)positions[t0 + r];
            for (int j = d_first; j < half; j += d_step) {
                float sn, cv;
                sincosf(pos * inv_freq[j], &sn, &cv);
                tile_lds[r * rot_dims + j] = cv;
                tile_lds[r * rot_dims + half + j] = sn;
            }
        }
    }
    __syncthreads();
    if (is_q || is_k) {
        if (idle) return;
        for (int r = r_first; r < rows; r += r_step) {
            const long t = t0 + r;
            TA* row_dst = nullptr;
            if (is_q) row_dst = q_out + (t * Hq + hh) * Dc;
            else if (page_lds[r] >= 0) row_dst = cache + page_lds[r] + ((long)(hh - Hq) * P + off_lds[r]) * Dc;
            for (int d = d_first; d < Dc; d += d_step) {
                const bool rotated = d < rot_dims;
                if (rotated && d >= half) continue;           // the pair's first thread does both
                if (d >= own) {
                    if (row_dst) Elem<TA>::store(row_dst + d, 0.f);
                    continue;
                }
                float y0 = conv_channel_ahead<TA>(a, t, c0 + d, seq_lds[r], before_lds[r]);
                if (rotated) {
                    float y1 = conv_channel_ahead<TA>(a, t, c0 + d + half, seq_lds[r], before_lds[r]);
                    rotate_pair(tile_lds[r * rot_dims + d], tile_lds[r * rot_dims + half + d], y0, y1);
                    if (row_dst) Elem<TA>::store(row_dst + d + half, y1);
                }
                if (row_dst) Elem<TA>::store(row_dst + d, y0);
            }
        }
        return;
    }
    // a value head: the convolution into shared memory, turned round ([feature][row], rows of 17 words)
    if (!idle) {
        for (int r = r_first; r < rows; r += r_step)
            for (int d = d_first; d < Dv; d += d_step)
                tile_lds[d * (CT_ROWS + 1) + r] = conv_channel_ahead<TA>(a, t0 + r, c0 + d, seq_lds[r], before_lds[r]);
    }
    __syncthreads();
    // every (feature, half of the rows) is a work item: eight rows that lie side by side in one page, from a slot
    // that is a multiple of eight, go out as one piece; else number by number
    const long vhead = ((long)(hh - Hq) * P) * Dc;           // (hh - Hq is Hkv + the key/value head)
    for (int i = threadIdx.x; i < Dc * 2; i += blockDim.x) {
        const int d = i >> 1, r0 = (i & 1) * 8;
        if (r0 >= rows) continue;
        const int n = rows - r0 < 8 ? rows - r0 : 8;
        const int sl = slot_lds[r0];
        bool run = n == 8 && sl >= 0 && (sl & 7) == 0 && (P & 7) == 0;
        if (run)
            for (int j = 1; j < 8; ++j) run = run && slot_lds[r0 + j] == sl + j;
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (d < Dv && j < n) ? tile_lds[d * (CT_ROWS + 1) + r0 + j] : 0.f;
        if (run) {
            TA* dst = cache + page_lds[r0] + vhead + (long)d * P + off_lds[r0];
            Vec4<TA>::store(dst, *(const float(*)[4])v);
            Vec4<TA>::store(dst + 4, *(const float(*)[4])(v + 4));
        } else {
            for (int j = 0; j < n; ++j)
                if (page_lds[r0 + j] >= 0) Elem<TA>::store(cache + page_lds[r0 + j] + vhead + (long)d * P + off_lds[r0 + j], v[j]);
        }
    }
}

// The same tile with eight neighbouring features a thread (heads, and the halves of their rotated part, in whole
// groups of eight): a wave's load of two bytes a lane costs the memory pipeline what a load of sixteen costs, and
// the thread-per-feature form was bound by the number of its loads (48 to 61 us for 2048 rows of 3072 coordinates,
// whatever else was changed).  wt: the convolution's weights transposed, [taps][C], so that a tap's weights for eight
// neighbouring channels are two loads.
template <typename TA>
__device__ __forceinline__ void load8(const TA* p, float (&v)[8]) {
    Vec4<TA>::load(p, *(float(*)[4])v);
    Vec4<TA>::load(p + 4, *(float(*)[4])(v + 4));
}
template <typename TA>
__device__ __forceinline__ void store8(TA* p, const float (&v)[8]) {
    Vec4<TA>::store(p, *(const float(*)[4])v);
    Vec4<TA>::store(p + 4, *(const float(*)[4])(v + 4));
}

// y[e] = the convolution of channel c + e at row t, e < 8 (oldest input first, all loads issued before the first use)
template <typename TA, int UN>      // UN: at least the number of taps
__device__ __forceinline__ void conv8(const ConvArgs<TA>& a, const float* __restrict__ wt, long t, int c, int s, int before,
                                      float (&y)[8]) {
    const int n1 = a.taps - 1;
    float v[UN][8], wv[UN][8];
#pragma unroll
    for (int j = 0; j < UN; ++j) {                   // the j-th oldest input lies k = n1 - j rows back
        const int k = n1 - j;
        if (k >= 0) {
            load8<float>(wt + (long)j * a.C + c, wv[j]);
            if (k <= before) load8<TA>(a.u + (t - k) * a.C + c, v[j]);
            else load8<float>(a.state + ((long)s * n1 + (j + before)) * a.C + c, v[j]);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = 0.f;
#pragma unroll
    for (int j = 0; j < UN; ++j)
        if (j <= n1) {
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = fmaf(wv[j][e], v[j][e], y[e]);
        }
}

// (A block's time is its chain of trips to memory, some microseconds whatever it computes, and the chip holds few
// blocks of many registers: so the look-back's loads, the slots', the positions' and the frequencies' are all asked
// for at once, and the taps are unrolled four deep where four are enough.)
template <typename TA, int UN>
__global__ __launch_bounds__(256) void qkv_conv_rope_store_tile8_kernel(
    ConvArgs<TA> a, const float* __restrict__ wt, const int* __restrict__ positions, const float* __restrict__ inv_freq,
    const int* __restrict__ slots, TA* __restrict__ q_out, TA* __restrict__ cache, int Hq, int Hkv, int Dk, int Dv,
    int Dc, int P, int rot_dims) {
    extern __shared__ float tile_lds[];                       // [CT_ROWS][rot_dims] cos | sin, or the value tile [Dc][CT_ROWS + 1]
    __shared__ int before_lds[CT_ROWS], seq_lds[CT_ROWS], slot_lds[CT_ROWS], off_lds[CT_ROWS];
    __shared__ long page_lds[CT_ROWS];
    const long t0 = (long)blockIdx.x * CT_ROWS;
    const int rows = a.T - t0 < CT_ROWS ? (int)(a.T - t0) : CT_ROWS;
    const int hh = blockIdx.y;
    const int half = rot_dims / 2;
    const bool is_q = hh < Hq, is_k = !is_q && hh < Hq + Hkv;
    const int own = is_q || is_k ? Dk : Dv;
    const int c0 = is_q ? hh * Dk : (is_k ? Hq * Dk + (hh - Hq) * Dk : (Hq + Hkv) * Dk + (hh - Hq - Hkv) * Dv);
    const long page_stride = 2L * Hkv * P * Dc;
    if (threadIdx.x < rows) {
        const long t = t0 + threadIdx.x;
        const int s = a.tok_seq[t];
        int back[UN];                                         // the rows before this one: all loads at once
#pragma unroll
        for (int k = 1; k < UN; ++k) back[k] = (k < a.taps && t - k >= 0) ? a.tok_seq[t - k] : -1;
        int before = 0;
        bool same = true;
#pragma unroll
        for (int k = 1; k < UN; ++k) {
            same = same && k < a.taps && t - k >= 0 && back[k] == s;
            before += same ? 1 : 0;
        }
        before_lds[threadIdx.x] = before;
        seq_lds[threadIdx.x] = s;
        const int slot = slots ? slots[t] : -1;
        slot_lds[threadIdx.x] = slot;
        page_lds[threadIdx.x] = slot >= 0 ? (long)(slot / P) * page_stride : -1;
        off_lds[threadIdx.x] = slot >= 0 ? slot % P : 0;
    }
    if ((is_q || is_k) && half > 0) {
        for (int i = threadIdx.x; i < CT_ROWS * half; i += blockDim.x) {
            const int r = i / half, j = i - r * half;
            if (r < rows) {
                float sn, cv;
                sincosf((float)positions[t0 + r] * inv_freq[j], &sn, &cv);
                tile_lds[r * rot_dims + j] = cv;
                tile_lds[r * rot_dims + half + j] = sn;
            }
        }
    }
    __syncthreads();
    const int groups = Dc >> 3;                               // groups of eight features in a head of the common size
    const int r_step = blockDim.x / groups;                   // (the host makes sure that a head has at most 256 / 1 groups)
    const int r_first = threadIdx.x / groups, g8 = threadIdx.x - r_first * groups;
    const int d = g8 * 8;
    const bool idle = r_first >= r_step;
    if (is_q || is_k) {
        if (idle) return;
        const bool rotated = d < rot_dims;
        if (rotated && d >= half) return;                     // the group of the pairs' first numbers does both
        for (int r = r_first; r < rows; r += r_step) {
            const long t = t0 + r;
            TA* row_dst = nullptr;
            if (is_q) row_dst = q_out + (t * Hq + hh) * Dc;
            else if (page_lds[r] >= 0) row_dst = cache + page_lds[r] + ((long)(hh - Hq) * P + off_lds[r]) * Dc;
            float y0[8];
            if (d >= own) {
#pragma unroll
                for (int e = 0; e < 8; ++e) y0[e] = 0.f;
                if (row_dst) store8<TA>(row_dst + d, y0);
                continue;
            }
            conv8<TA, UN>(a, wt, t, c0 + d, seq_lds[r], before_lds[r], y0);
            if (rotated) {
                float y1[8];
                conv8<TA, UN>(a, wt, t, c0 + d + half, seq_lds[r], before_lds[r], y1);
#pragma unroll
                for (int e = 0; e < 8; ++e) rotate_pair(tile_lds[r * rot_dims + d + e], tile_lds[r * rot_dims + half + d + e], y0[e], y1[e]);
                if (row_dst) store8<TA>(row_dst + d + half, y1);
            }
            if (row_dst) store8<TA>(row_dst + d, y0);
        }
        return;
    }
    // a value head: the convolution into shared memory, turned round ([feature][row], rows of 17 words)
    if (!idle) {
        for (int r = r_first; r < rows; r += r_step) {
            float y[8];
            if (d < own) conv8<TA, UN>(a, wt, t0 + r, c0 + d, seq_lds[r], before_lds[r], y);
            else {
#pragma unroll
                for (int e = 0; e < 8; ++e) y[e] = 0.f;
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) tile_lds[(d + e) * (CT_ROWS + 1) + r] = y[e];
        }
    }
    __syncthreads();
    const long vhead = ((long)(hh - Hq) * P) * Dc;           // (hh - Hq is Hkv + the key/value head)
    for (int i = threadIdx.x; i < Dc * 2; i += blockDim.x) {
        const int dd = i >> 1, r0 = (i & 1) * 8;
        if (r0 >= rows) continue;
        const int n = rows - r0 < 8 ? rows - r0 : 8;
        const int sl = slot_lds[r0];
        bool run = n == 8 && sl >= 0 && (sl & 7) == 0 && (P & 7) == 0;
        if (run)
            for (int j = 1; j < 8; ++j) run = run && slot_lds[r0 + j] == sl + j;
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = j < n ? tile_lds[dd * (CT_ROWS + 1) + r0 + j] : 0.f;
        if (run) {
            store8<TA>(cache + page_lds[r0] + vhead + (long)dd * P + off_lds[r0], v);
        } else {
            for (int j = 0; j < n; ++j)
                if (page_lds[r0 + j] >= 0) Elem<TA>::store(cache + page_lds[r0 + j] + vhead + (long)dd * P + off_lds[r0 + j], v[j]);
        }
    }
}

// After the convolution: the state takes the portion's last taps - 1 rows.  A portion shorter than
// that moves the state's old entries up first; its first row's thread does all of it, so that no
// thread reads what another writes.  A block looks at 64 rows of the batch and a piece of the channels: the
// rows that are among their portion's last taps - 1 (rows of a request are consecutive: a row is not, if the row
// taps - 1 further on is the same request's) are found by 64 lanes at once, and only those are walked.
template <typename TA>
__global__ void qkv_conv_state_kernel(ConvArgs<TA> a) {
    __shared__ unsigned long long cand_lds;
    const long tb = (long)blockIdx.y * 64;
    const int n1 = a.taps - 1;
    if (threadIdx.x < 64) {
        const long t = tb + threadIdx.x;
        bool last = false;
        if (t < a.T) last = !(t + n1 < a.T && a.tok_seq[t + n1] == a.tok_seq[t]);
        const unsigned long long m = __ballot(last);
        if (threadIdx.x == 0) cand_lds = m;
    }
    __syncthreads();
    unsigned long long m = cand_lds;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= a.C) return;
    while (m) {
        const long t = tb + (__ffsll((long long)m) - 1);
        m &= m - 1;
        const int s = a.tok_seq[t];
        int before = 0, after = 0;
        while (before < n1 && t - 1 - before >= 0 && a.tok_seq[t - 1 - before] == s) ++before;
        while (after < n1 && t + 1 + after < a.T && a.tok_seq[t + 1 + after] == s) ++after;
        float* st = a.state + (long)s * n1 * a.C + c;
        if (before + after + 1 < n1) {                        // the whole portion is shorter than the state
            if (before != 0) continue;
            const int q = after + 1;
            for (int j = 0; j + q < n1; ++j) st[(long)j * a.C] = st[(long)(j + q) * a.C];
            for (int i = 0; i < q; ++i) st[(long)(n1 - q + i) * a.C] = Elem<TA>::load(a.u + (t + i) * a.C + c);
        } else if (after < n1) {
            st[(long)(n1 - 1 - after) * a.C] = Elem<TA>::load(a.u + t * a.C + c);
        }
    }
}

template <typename TA>
static int launch_conv_rope_store(const void* u, const float* w, const float* wt, float* state, const int* tok_seq, const int* positions,
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
    // eight features a thread where heads, and the halves of their rotated parts, are whole groups of eight
    const bool by_eight = wt && taps <= CONV_UNROLL && Dk % 8 == 0 && Dv % 8 == 0 && (rot_dims / 2) % 8 == 0 && Dc % 8 == 0 &&
                          Dc / 8 <= 256;
    if (T > 16 && by_eight) {
        const size_t rot_bytes = (size_t)CT_ROWS * rot_dims * sizeof(float), val_bytes = (size_t)Dc * (CT_ROWS + 1) * sizeof(float);
        const dim3 tgrid(qe_cdiv(T, CT_ROWS), Hq + 2 * Hkv);
        const size_t lds = rot_bytes > val_bytes ? rot_bytes : val_bytes;
        if (taps <= 4)
            qkv_conv_rope_store_tile8_kernel<TA, 4><<<tgrid, 256, lds, stream>>>(
                a, wt, positions, inv_freq, slots, (TA*)q_out, (TA*)cache, Hq, Hkv, Dk, Dv, Dc, P, rot_dims);
        else
            qkv_conv_rope_store_tile8_kernel<TA, CONV_UNROLL><<<tgrid, 256, lds, stream>>>(
                a, wt, positions, inv_freq, slots, (TA*)q_out, (TA*)cache, Hq, Hkv, Dk, Dv, Dc, P, rot_dims);
    } else if (T > 16) {
        const size_t rot_bytes = (size_t)CT_ROWS * rot_dims * sizeof(float), val_bytes = (size_t)Dv * (CT_ROWS + 1) * sizeof(float);
        qkv_conv_rope_store_tile_kernel<TA><<<dim3(qe_cdiv(T, CT_ROWS), Hq + 2 * Hkv), 256, rot_bytes > val_bytes ? rot_bytes : val_bytes, stream>>>(
            a, positions, inv_freq, slots, (TA*)q_out, (TA*)cache, Hq, Hkv, Dk, Dv, Dc, P, rot_dims);
    }
    else
        qkv_conv_rope_store_kernel<TA, false><<<grid, threads, 0, stream>>>(a, positions, inv_freq, slots, (TA*)q_out,
                                                                             (TA*)cache, Hq, Hkv, Dk, Dv, Dc, P, rot_dims);
    if (taps > 1) {
        const int th = a.C >= 256 ? 256 : 64;
        qkv_conv_state_kernel<TA><<<dim3(qe_cdiv(a.C, th), qe_cdiv(T, 64)), th, 0, stream>>>(a);
    }
    return 0;
}

// u [T, Hq Dk + Hkv Dk + Hkv Dv] in the activation type; w float [that many, taps]; state float [slots, taps - 1,
// that many] (row tok_seq[t]; null when taps is 1); inv_freq float [rot_dims / 2] (null when rot_dims is 0);
// slots [T] (negative: the row's key and value go nowhere), or null; q_out [T, Hq, Dc]; cache [pages, 2, Hkv, P, Dc].
// single: the caller knows that no two rows belong to the same request.
// wt: null, or the same weights transposed, float [taps, that many] (the kernel for many rows then takes eight
// channels a thread where the sizes are whole groups of eight).
extern "C" int qe_qkv_conv_rope_store(const void* u, const float* w, const float* wt, float* state, const int* tok_seq,
                                      const int* positions, const float* inv_freq, const int* slots, void* q_out,
                                      void* cache, int T, int Hq, int Hkv, int Dk, int Dv, int Dc, int P, int taps,
                                      int rot_dims, int single, int dt_a, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && Hq > 0 && Hkv > 0 && Dk > 0 && Dv > 0 && P > 0 && taps >= 1, "qkv_conv_rope_store: bad sizes");
    QE_REQUIRE(Dc >= Dk && Dc >= Dv, "qkv_conv_rope_store: the common head size %d is smaller than %d or %d", Dc, Dk, Dv);
    QE_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= Dk, "qkv_conv_rope_store: %d rotated numbers of %d", rot_dims, Dk);
    QE_REQUIRE(taps == 1 || state, "qkv_conv_rope_store: %d taps need a state", taps);
    QE_REQUIRE(rot_dims == 0 || (inv_freq && positions), "qkv_conv_rope_store: a rotation needs positions and frequencies");
    QE_REQUIRE(!slots || cache, "qkv_conv_rope_store: slots without a cache");
    QE_REQUIRE(T <= 65535 && Hq + 2 * Hkv <= 65535, "qkv_conv_rope_store: more than 65535 rows in a step, or heads");
    QE_REQUIRE(Dk <= 512 && Dv <= 512, "qkv_conv_rope_store: heads of more than 512 numbers");
    if (T == 0) return 0;
    int rc;
    if (dt_a == QE_F32)
        rc = launch_conv_rope_store<float>(u, w, wt, state, tok_seq, positions, inv_freq, slots, q_out, cache, T, Hq, Hkv, Dk, Dv,
                                           Dc, P, taps, rot_dims, single, stream);
    else if (dt_a == QE_BF16)
        rc = launch_conv_rope_store<bf16_t>(u, w, wt, state, tok_seq, positions, inv_freq, slots, q_out, cache, T, Hq, Hkv, Dk,
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
