// kr_serve_ops.hip -- row kernels of the batched serving step (gfx950, wave64): embedding, layer / RMS norm, rotary table, query / key preparation with
// the paged cache append, sliding-window attention with a sink over the paged cache, group-limited top-k router, expert row sort, gated activations,
// the parallel-block residual sum, argmax.
//
// Every f32 reduction here is a lane / wave tree; sums written as a * b + c may be contracted (explicit __builtin_fmaf): the serving path states a
// tolerance against an f32 restatement, not a bit pattern.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include <type_traits>

#include "kr_device.h"
#include "kr_serve_ops.h"

namespace {
__device__ __forceinline__ float sv_ld(const float* p) { return *p; }
__device__ __forceinline__ float sv_ld(const uint16_t* p) { return kr_bf16_to_f32(*p); }
__device__ __forceinline__ void sv_st(float* p, float v) { *p = v; }
__device__ __forceinline__ void sv_st(uint16_t* p, float v) { *p = kr_f32_to_bf16(v); }

// wave-wide sum / maximum, every lane receives it: four DPP steps inside each row of 16 lanes, then the four rows through scalar reads
#define SV_DPPF(v, ctrl) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), (ctrl), 0xF, 0xF, false))
#define SV_LANE(v, i) __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), (i)))
__device__ __forceinline__ float sv_wave_sum(float v) {
    v += SV_DPPF(v, KR_DPP_XOR1); v += SV_DPPF(v, KR_DPP_XOR2); v += SV_DPPF(v, KR_DPP_HALF_MIRROR); v += SV_DPPF(v, KR_DPP_MIRROR);
    return (SV_LANE(v, 0) + SV_LANE(v, 16)) + (SV_LANE(v, 32) + SV_LANE(v, 48));
}
__device__ __forceinline__ float sv_wave_max(float v) {
    v = fmaxf(v, SV_DPPF(v, KR_DPP_XOR1)); v = fmaxf(v, SV_DPPF(v, KR_DPP_XOR2)); v = fmaxf(v, SV_DPPF(v, KR_DPP_HALF_MIRROR)); v = fmaxf(v, SV_DPPF(v, KR_DPP_MIRROR));
    return fmaxf(fmaxf(SV_LANE(v, 0), SV_LANE(v, 16)), fmaxf(SV_LANE(v, 32), SV_LANE(v, 48)));
}
// sum over a workgroup of NW waves; every thread receives it
template <int NW>
__device__ __forceinline__ float sv_block_sum(float v, float* red) {
    v = sv_wave_sum(v);
    if constexpr (NW == 1) return v;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; w++) s += red[w];
    return s;
}

template <typename T>
__global__ void __launch_bounds__(256) sv_embed_kernel(const T* __restrict__ table, const int* __restrict__ tokens, float* __restrict__ x, T* __restrict__ h_out, int width,
                                                       float scale, const T* __restrict__ table2, const int* __restrict__ rows2) {
    const int t = blockIdx.x;
    const T* row = table + (size_t)tokens[t] * width;
    const T* row2 = table2 ? table2 + (size_t)rows2[t] * width : nullptr;
    for (int c = threadIdx.x; c < width; c += 256) {
        float v = sv_ld(row + c) * scale;
        if (row2) v += sv_ld(row2 + c);
        x[(size_t)t * width + c] = v;
        if (h_out) sv_st(h_out + (size_t)t * width + c, v);
    }
}

// statistics of `groups` equal consecutive parts of a row (LDS or global): st[2 g] = mean (0 for an RMS norm), st[2 g + 1] = 1 / sqrt(variance + eps).
// Wave w of the NW takes the parts w, w + NW, ...; the caller makes the row visible before and synchronises after.
template <int KIND, int NW = 4>
__device__ __forceinline__ void sv_group_stats(const float* xr, int width, int groups, float eps, float* st) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, gw = width / groups;
    for (int g = wave; g < groups; g += NW) {
        const float* xg = xr + (size_t)g * gw;
        float mean = 0.0f;
        if constexpr (KIND == KR_SV_NORM_LAYER) {
            float s = 0.0f;
            for (int c = lane; c < gw; c += 64) s += xg[c];
            mean = sv_wave_sum(s) / (float)gw;
        }
        float q = 0.0f;
        for (int c = lane; c < gw; c += 64) { const float d = xg[c] - mean; q = __builtin_fmaf(d, d, q); }
        q = sv_wave_sum(q);
        if (lane == 0) { st[2 * g] = mean; st[2 * g + 1] = 1.0f / sqrtf(q / (float)gw + eps); }
    }
}

template <typename T, int KIND>
__global__ void __launch_bounds__(256) sv_norm_kernel(const float* __restrict__ x, const int* __restrict__ rows, const float* __restrict__ w, const float* __restrict__ b,
                                                      T* __restrict__ out, int width, float eps, int groups, float* __restrict__ out32) {
    __shared__ float red[4];
    extern __shared__ float gst[];            // [2 * groups] when the row is normed in parts
    const int r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : r) * width;
    if (groups > 1) {
        sv_group_stats<KIND>(xr, width, groups, eps, gst);
        __syncthreads();
        const int gw = width / groups;
        for (int c = threadIdx.x; c < width; c += 256) {
            const int g = c / gw;
            float v = (xr[c] - gst[2 * g]) * gst[2 * g + 1] * w[c];
            if (b) v += b[c];
            sv_st(out + (size_t)r * width + c, v);
            if (out32) out32[(size_t)r * width + c] = v;
        }
        return;
    }
    float mean = 0.0f;
    if constexpr (KIND == KR_SV_NORM_LAYER) {
        float s = 0.0f;
        for (int c = threadIdx.x; c < width; c += 256) s += xr[c];
        mean = sv_block_sum<4>(s, red) / (float)width;
    }
    float q = 0.0f;
    for (int c = threadIdx.x; c < width; c += 256) { const float d = xr[c] - mean; q = __builtin_fmaf(d, d, q); }
    const float var = sv_block_sum<4>(q, red) / (float)width;
    const float inv = 1.0f / sqrtf(var + eps);
    for (int c = threadIdx.x; c < width; c += 256) {
        float v = (xr[c] - mean) * inv * w[c];
        if (b) v += b[c];
        sv_st(out + (size_t)r * width + c, v);
        if (out32) out32[(size_t)r * width + c] = v;
    }
}

// input convolution over positions (KrSvCanon): one thread per (token, channel)
template <typename T>
__global__ void __launch_bounds__(256) sv_canon_kernel(const KrSvCanon a, T* __restrict__ out) {
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= a.width) return;
    const int p = a.pos[t], sl = a.slot[t], K = a.taps - 1;
    const float* w = a.w + (size_t)c * a.taps;
    float acc = a.h32[(size_t)t * a.width + c];
    acc = __builtin_fmaf(w[K], acc, acc);                     // the tap on the token itself
    for (int d = 1; d <= K; d++) {                            // d positions back
        const int q = p - d;
        if (q < 0) break;
        float hv;
        if (t - d >= 0 && a.slot[t - d] == sl) hv = a.h32[(size_t)(t - d) * a.width + c];
        else hv = a.state[((size_t)sl * K + q % K) * a.width + c];
        acc = __builtin_fmaf(w[K - d], hv, acc);
    }
    sv_st(out + (size_t)t * a.width + c, acc);
}

// the stream itself (kr_sv_stream_norm): a vector joins the row, and / or the row is normed -- in place, or into the next sublayer's input
template <typename T, int KIND>
__global__ void __launch_bounds__(256) sv_stream_norm_kernel(float* __restrict__ x, const float* __restrict__ add, const float* __restrict__ w, const float* __restrict__ b, int in_place,
                                                             T* __restrict__ out, int width, float eps, int groups) {
    extern __shared__ float xr[];            // [width] | [2 * groups]
    __shared__ float red[4];
    const size_t t = blockIdx.x;
    float* xp = x + t * width;
    float* gst = xr + width;
    float s1 = 0.0f;
    for (int c = threadIdx.x; c < width; c += 256) {
        float v = xp[c];
        if (add) { v += add[c]; xp[c] = v; }
        xr[c] = v; s1 += v;
    }
    if (!w) return;
    float mean = 0.0f, inv = 0.0f;
    if (groups > 1) { __syncthreads(); sv_group_stats<KIND, 4>(xr, width, groups, eps, gst); __syncthreads(); }
    else {
        if constexpr (KIND == KR_SV_NORM_LAYER) mean = sv_block_sum<4>(s1, red) / (float)width;
        float q = 0.0f;
        for (int c = threadIdx.x; c < width; c += 256) { const float dv = xr[c] - mean; q = __builtin_fmaf(dv, dv, q); }
        inv = 1.0f / sqrtf(sv_block_sum<4>(q, red) / (float)width + eps);
    }
    const int gw = groups > 1 ? width / groups : width;
    for (int c = threadIdx.x; c < width; c += 256) {
        if (groups > 1) { mean = gst[2 * (c / gw)]; inv = gst[2 * (c / gw) + 1]; }
        float v = (xr[c] - mean) * inv * w[c];
        if (b) v += b[c];
        if (in_place) xp[c] = v; else sv_st(out + t * width + c, v);
    }
}

// short convolution on the channels of a projection (KrSvChanConv): one thread per (token, channel)
__global__ void __launch_bounds__(256) sv_chan_conv_kernel(const KrSvChanConv a) {
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= a.C) return;
    const int p = a.pos[t], sl = a.slot[t], K = a.taps - 1;
    const float* w = a.w + (size_t)c * a.taps;
    const float ib = a.in_bias ? a.in_bias[c] : 0.0f;
    float acc = a.cb ? a.cb[c] : 0.0f;
    acc = __builtin_fmaf(w[K], a.in[(size_t)t * a.ld_in + c] + ib, acc);
    for (int d = 1; d <= K; d++) {            // d positions back
        const int q = p - d;
        if (q < 0) break;
        float u;
        if (t - d >= 0 && a.slot[t - d] == sl) u = a.in[(size_t)(t - d) * a.ld_in + c] + ib;
        else u = a.state[((size_t)sl * K + q % K) * a.C + c];
        acc = __builtin_fmaf(w[K - d], u, acc);
    }
    if (a.act == 1) acc = acc / (1.0f + expf(-acc));
    a.out[(size_t)t * a.ld_out + c] = acc;
}
// the last taps - 1 inputs of every portion -> the request's ring
__global__ void __launch_bounds__(256) sv_chan_conv_save_kernel(const KrSvChanConv a) {
    const int e = blockIdx.x, i = blockIdx.y, c = blockIdx.z * 256 + threadIdx.x, K = a.taps - 1;
    if (c >= a.C) return;
    const int t = a.ent_off[e + 1] - 1 - i;
    if (t < a.ent_off[e]) return;
    const float ib = a.in_bias ? a.in_bias[c] : 0.0f;
    a.state[((size_t)a.slot[t] * K + a.pos[t] % K) * a.C + c] = a.in[(size_t)t * a.ld_in + c] + ib;
}
__global__ void sv_scale_kernel(float* __restrict__ p, size_t n, float scale) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] *= scale;
}

// unit_norm == 3: 1 / rms over the whole q row (part 0) and the whole k row (part 1) of every token, biases included
__global__ void __launch_bounds__(256) sv_qk_rms_kernel(const KrSvAttn a) {
    __shared__ float red[4];
    const int t = blockIdx.x, part = blockIdx.y;
    const int n = (part ? a.kv_heads : a.heads) * a.dim;
    const float* z = a.qkv + (size_t)t * a.ldq + (part ? a.heads * a.dim : 0);
    const float* b = part ? a.k_bias : a.q_bias;
    float q = 0.0f;
    for (int c = threadIdx.x; c < n; c += 256) { const float v = b ? z[c] + b[c] : z[c]; q = __builtin_fmaf(v, v, q); }
    q = sv_block_sum<4>(q, red);
    if (threadIdx.x == 0) a.inv_rms_out[(size_t)t * 2 + part] = 1.0f / sqrtf(q / (float)n + a.eps);
}

__global__ void sv_rope_table_kernel(const int* __restrict__ pos, const double* __restrict__ inv_freq, float2* __restrict__ cs, int T, int half, float mult) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= T * half) return;
    const int t = i / half, j = i - t * half;
    const double a = (double)pos[t] * inv_freq[j];
    cs[i] = make_float2((float)cos(a) * mult, (float)sin(a) * mult);
}

// one wave per (token, head): the head vector is staged in LDS, rotated and normed there; q heads are written back in place, k heads go to the
// cache page of (slot, position), v heads are copied there
template <typename T>
__global__ void __launch_bounds__(64) sv_qk_prep_kernel(const KrSvAttn a) {
    extern __shared__ float hv[];            // [dim]
    const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
    const int H = a.heads, G = a.kv_heads;
    const int p = a.pos[t], sl = a.slot[t];
    float* row = a.qkv + (size_t)t * a.ldq;
    size_t prow = 0;
    if (hh >= H) {
        const size_t page = (size_t)a.page_table[(size_t)sl * a.table_ld + p / a.page_tokens];
        prow = page * a.page_tokens + (p % a.page_tokens);
    }
    if (hh >= H + G) {                       // value head (never launched when the values are the keys): copy, or blend with the values an earlier layer formed for this token
        const int g = hh - H - G;
        const float* v = row + (size_t)H * a.dim + (size_t)G * a.dim + (size_t)g * a.vdim;
        T* dst = (T*)a.vpool + prow * a.ldv + (size_t)g * a.vdim;
        float* vf = a.v_mix ? a.v_first + ((size_t)t * G + g) * a.vdim : nullptr;
        const float lam = a.v_mix == 2 ? *a.v_lambda : 0.0f;
        const float* vb = a.v_bias ? a.v_bias + (size_t)g * a.vdim : nullptr;
        for (int d = lane; d < a.vdim; d += 64) {
            float val = vb ? v[d] + vb[d] : v[d];
            if (a.v_mix == 1) vf[d] = val;
            else if (a.v_mix == 2) val = (1.0f - lam) * val + lam * vf[d];
            sv_st(dst + d, val);
        }
        return;
    }
 float* v = row + (size_t)hh * a.dim;
    {
        const float* bias = hh < H ? a.q_bias : a.k_bias;
        if (bias) bias += (size_t)(hh < H ? hh : hh - H) * a.dim;
        for (int d = lane; d < a.dim; d += 64) hv[d] = bias ? v[d] + bias[d] : v[d];
    }
    __syncthreads();
    if (a.v_from_k && hh >= H) {             // the value row of this key head: the key as projected
        T* dst = (T*)a.vpool + prow * a.ldv + (size_t)(hh - H) * a.dim;
        for (int d = lane; d < a.dim; d += 64) sv_st(dst + d, hv[d]);
    }
    if (a.unit_norm == 3) {                  // one statistic for the whole row, a weight per coordinate of the row
        const float inv3 = a.inv_rms[(size_t)t * 2 + (hh < H ? 0 : 1)];
        const float* w = hh < H ? a.q_norm_w + (size_t)hh * a.dim : a.k_norm_w + (size_t)(hh - H) * a.dim;
        for (int d = lane; d < a.dim; d += 64) hv[d] = hv[d] * inv3 * w[d];
        __syncthreads();
    }
    if (a.unit_norm == 2) {                  // weighted, before the rotation
        const float* w = hh < H ? a.q_norm_w : a.k_norm_w;
        float s2 = 0.0f;
        for (int d = lane; d < a.dim; d += 64) s2 = __builtin_fmaf(hv[d], hv[d], s2);
        s2 = sv_wave_sum(s2);
        const float inv2 = 1.0f / sqrtf(s2 / (float)a.dim + a.eps);
        for (int d = lane; d < a.dim; d += 64) hv[d] = hv[d] * inv2 * w[d];
        __syncthreads();
    }
    const int half = a.rot_dims / 2;
    const float2* cs = a.cs + (size_t)t * half;
    float ss = 0.0f;
    for (int i = lane; i < half; i += 64) {  // a lane owns whole rotation pairs; the tail past rot_dims passes unchanged
        const int i0 = a.rot_interleaved ? 2 * i : i, i1 = a.rot_interleaved ? 2 * i + 1 : i + half;
        const float u = hv[i0], w = hv[i1];
        const float2 c = cs[i];
        const float r0 = u * c.x - w * c.y, r1 = w * c.x + u * c.y;
        hv[i0] = r0; hv[i1] = r1;
        ss = __builtin_fmaf(r0, r0, ss); ss = __builtin_fmaf(r1, r1, ss);
    }
    for (int d = a.rot_dims + lane; d < a.dim; d += 64) ss = __builtin_fmaf(hv[d], hv[d], ss);
    ss = sv_wave_sum(ss);
    const float inv = a.unit_norm == 1 ? 1.0f / sqrtf(ss / (float)a.dim + a.eps) : 1.0f;
    __syncthreads();
    if (hh < H) {
        for (int d = lane; d < a.dim; d += 64) v[d] = hv[d] * inv;
    } else {
        const int g = hh - H;
        T* dst = (T*)a.kpool + prow * a.ldk + (size_t)g * a.dim;
        for (int d = lane; d < a.dim; d += 64) sv_st(dst + d, hv[d] * inv);
    }
}

// Windowed attention with a sink over the paged cache.  One workgroup (four waves) per (token, key / value head, batch of RM query heads of that
// head's group): a cache row is fetched once for all query heads that share it.  The visible keys [max(0, p - window + 1), p] are walked in blocks of
// 64, block b by wave b % 4; lane j scores key j for every head (f32 dot of the pre-scaled query, held in LDS, with the 16-byte pieces of its key row),
// the wave updates each head's running maximum / denominator (online softmax, f32) and the lanes then own value columns for p.v.  The four waves'
// partial states are merged through LDS in wave order; the sink joins the denominator there, once.
typedef uint32_t sv_u4 __attribute__((ext_vector_type(4)));
#ifdef KR_SV_STAMPS      // probe build: shader-clock stamps of the first wave of the first workgroup (kr_sv_read_stamps)
__device__ long long sv_stamps[16];
#define SV_STAMP(i) do { if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0) sv_stamps[i] = __builtin_readcyclecounter(); } while (0)
#else
#define SV_STAMP(i) do { } while (0)
#endif
template <typename T, int RM, int VC>
__global__ void __launch_bounds__(256) sv_attn_group_kernel(const KrSvAttn a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int VEC = 16 / sizeof(T);
    const int G = a.kv_heads, R = a.heads / G, dim = a.dim, vdim = a.vdim;
    const int sp = blockIdx.z % a.nsplit;
    const int t = blockIdx.x, g = blockIdx.y, r0 = (blockIdx.z / a.nsplit) * RM, nr = min(RM, R - r0), h0 = g * R + r0;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float* qs = lds;                                       // [RM][dim]
    float* pw = qs + RM * dim + wave * 64 * RM;            // this wave's weights [RM][64]
    float* ml = qs + RM * dim + 4 * 64 * RM;               // [4][RM][2]
    float* accs = ml + 4 * RM * 2;                         // [RM][vdim]
    const int p = a.pos[t], sl = a.slot[t];
    const int* table = a.page_table + (size_t)sl * a.table_ld;
    const float* q = a.qkv + (size_t)t * a.ldq + (size_t)h0 * dim;
    // heads past the group's last one are computed on zero queries and dropped: the loops below carry no per-head branches, so the loads of a block of
    // keys are all in flight before the first product needs them
    SV_STAMP(0);
    for (int i = tid; i < RM * dim; i += 256) qs[i] = i < nr * dim ? q[i] * a.scale : 0.0f;
    __syncthreads();
    SV_STAMP(1);
    const int lo = a.window > 0 ? max(0, p - a.window + 1) : (a.chunk > 0 ? p - p % a.chunk : 0);
    float slope[RM];
#pragma unroll
    for (int r = 0; r < RM; r++) slope[r] = (a.slopes && r < nr) ? a.slopes[h0 + r] : 0.0f;
    float m[RM], l[RM], acc[RM][VC];
#pragma unroll
    for (int r = 0; r < RM; r++) {
        m[r] = -INFINITY; l[r] = 0.0f;
#pragma unroll
        for (int c = 0; c < VC; c++) acc[r][c] = 0.0f;
    }
    const T* kp = (const T*)a.kpool; const T* vp = (const T*)a.vpool;
    const bool vec = ((size_t)dim * sizeof(T)) % 16 == 0 && ((size_t)a.ldk * sizeof(T)) % 16 == 0;
    const int npiece = dim / VEC;
    auto widen = [](const sv_u4& kv, float* kf) {
        if constexpr (sizeof(T) == 2) {
#pragma unroll
            for (int i = 0; i < 4; i++) { kf[2 * i] = __uint_as_float(kv[i] << 16); kf[2 * i + 1] = __uint_as_float(kv[i] & 0xFFFF0000u); }
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) kf[i] = __uint_as_float(kv[i]);
        }
    };
    // blocks of 64 keys: this workgroup's share [c0, c1) of the token's blocks (all of them when the launch is not split), block c by wave (c - c0) % 4
    const int nch = (p - lo) / 64 + 1, cps = (nch + a.nsplit - 1) / a.nsplit;
    const int c0 = sp * cps, c1 = min(nch, c0 + cps);
    for (int cb = c0 + wave; cb < c1; cb += 4) {
        const int j0 = lo + 64 * cb;
        const int j = j0 + lane;
        const bool live = j <= p;
        const int jc = min(j, p);                            // lanes past the last key score it again; their weight is set to 0
        const int prow = table[jc / a.page_tokens] * a.page_tokens + (jc % a.page_tokens);
        const T* k = kp + (size_t)prow * a.ldk + (size_t)g * dim;
        constexpr int U = 16 / VC;                           // keys whose value rows are requested together
        const int nk = min(64, p - j0 + 1);
        float va[U][VC], vb[U][VC];
        auto fetch_v = [&](int jb, float (&vv)[U][VC]) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int pr = __builtin_amdgcn_readlane(prow, min(jb + u, 63));
                const T* vr = vp + (size_t)pr * a.ldv + (size_t)g * vdim;
#pragma unroll
                for (int c = 0; c < VC; c++) { const int d = lane + 64 * c; vv[u][c] = d < vdim ? sv_ld(vr + d) : 0.0f; }
            }
        };
        SV_STAMP(2);
        fetch_v(0, va);                                      // in flight behind the key rows, consumed after the softmax
        float s[RM];
#pragma unroll
        for (int r = 0; r < RM; r++) s[r] = 0.0f;
        if (vec) {
            int pc = 0;
            auto block = [&](auto PBc) {                     // PB 16-byte pieces of the key row in flight, then their products with every head's query
                constexpr int PB = decltype(PBc)::value;
                sv_u4 kv[PB];
#pragma unroll
                for (int u = 0; u < PB; u++) kv[u] = *reinterpret_cast<const sv_u4*>(k + (pc + u) * VEC);
#pragma unroll
                for (int u = 0; u < PB; u++) {
                    float kf[VEC];
                    widen(kv[u], kf);
#pragma unroll
                    for (int r = 0; r < RM; r++) {
                        const float4* qp = reinterpret_cast<const float4*>(qs + r * dim + (pc + u) * VEC);
#pragma unroll
                        for (int v4 = 0; v4 < VEC / 4; v4++) {
                            const float4 qa = qp[v4];
                            s[r] = __builtin_fmaf(qa.x, kf[4 * v4], s[r]); s[r] = __builtin_fmaf(qa.y, kf[4 * v4 + 1], s[r]);
                            s[r] = __builtin_fmaf(qa.z, kf[4 * v4 + 2], s[r]); s[r] = __builtin_fmaf(qa.w, kf[4 * v4 + 3], s[r]);
                        }
                    }
                }
                pc += PB;
            };
            while (pc + 16 <= npiece) block(std::integral_constant<int, 16>{});
            if (pc + 8 <= npiece) block(std::integral_constant<int, 8>{});
            if (pc + 4 <= npiece) block(std::integral_constant<int, 4>{});
            for (; pc < npiece; pc++) {
                const sv_u4 kv = *reinterpret_cast<const sv_u4*>(k + pc * VEC);
                float kf[VEC];
                widen(kv, kf);
#pragma unroll
                for (int r = 0; r < RM; r++)
#pragma unroll
                    for (int i = 0; i < VEC; i++) s[r] = __builtin_fmaf(qs[r * dim + pc * VEC + i], kf[i], s[r]);
            }
        } else {
            for (int d = 0; d < dim; d++) {
                const float kd = sv_ld(k + d);
#pragma unroll
                for (int r = 0; r < RM; r++) s[r] = __builtin_fmaf(qs[r * dim + d], kd, s[r]);
            }
        }
        SV_STAMP(3);
#pragma unroll
        for (int r = 0; r < RM; r++) {
            const float sc = a.softcap > 0.0f ? a.softcap * tanhf(s[r] / a.softcap) : s[r];
            const float sr = live ? sc - slope[r] * (float)(p - j) : -INFINITY;
            const float mn = fmaxf(m[r], sv_wave_max(sr));
            const float alpha = expf(m[r] - mn);               // first block of this wave: exp(-inf) = 0
            const float pj = live ? expf(sr - mn) : 0.0f;
            l[r] = l[r] * alpha + sv_wave_sum(pj);
            m[r] = mn;
#pragma unroll
            for (int c = 0; c < VC; c++) acc[r][c] *= alpha;
            pw[r * 64 + lane] = pj;
        }
        // the wave's own LDS writes are read back by its own lanes below: a wave executes in lock step, only the LDS counter has to drain
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        SV_STAMP(4);
        // groups of U keys: a group's products run while the next group's value rows are in flight (the first group's were requested before the scores);
        // keys past nk inside the last group carry weight 0 and read the last key's row
        auto products = [&](int jb, float (&vv)[U][VC]) {
#pragma unroll
            for (int r = 0; r < RM; r++) {
                if constexpr (U % 4 == 0) {      // four keys' weights per LDS read (jb is a multiple of U: the read is 16-byte aligned and stays inside the block)
#pragma unroll
                    for (int u4 = 0; u4 < U / 4; u4++) {
                        const float4 w4 = *reinterpret_cast<const float4*>(&pw[r * 64 + jb + 4 * u4]);
#pragma unroll
                        for (int c = 0; c < VC; c++) {
                            acc[r][c] = __builtin_fmaf(w4.x, vv[4 * u4][c], acc[r][c]); acc[r][c] = __builtin_fmaf(w4.y, vv[4 * u4 + 1][c], acc[r][c]);
                            acc[r][c] = __builtin_fmaf(w4.z, vv[4 * u4 + 2][c], acc[r][c]); acc[r][c] = __builtin_fmaf(w4.w, vv[4 * u4 + 3][c], acc[r][c]);
                        }
                    }
                } else {
#pragma unroll
                    for (int u = 0; u < U; u++) {
                        const float w = pw[r * 64 + min(jb + u, 63)];
#pragma unroll
                        for (int c = 0; c < VC; c++) acc[r][c] = __builtin_fmaf(w, vv[u][c], acc[r][c]);
                    }
                }
            }
        };
        for (int jb = 0; jb < nk; jb += 2 * U) {
            if (jb + U < nk) fetch_v(jb + U, vb);
            products(jb, va);
            if (jb + 2 * U < nk) fetch_v(jb + 2 * U, va);
            if (jb + U < nk) products(jb + U, vb);
        }
        SV_STAMP(5);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < RM; r++) if (r < nr) { ml[(wave * RM + r) * 2] = m[r]; ml[(wave * RM + r) * 2 + 1] = l[r]; }
    }
    __syncthreads();
    SV_STAMP(6);
    const bool last = a.nsplit == 1;                         // an unsplit launch finishes here: sink, normalisation, output; a split one leaves partial states
    float f[RM];
#pragma unroll
    for (int r = 0; r < RM; r++) {
        f[r] = 0.0f;
        if (r < nr) {
            float M = -INFINITY;
            for (int w = 0; w < 4; w++) M = fmaxf(M, ml[(w * RM + r) * 2]);
            if (last && a.sink) M = fmaxf(M, a.sink[h0 + r]);
            f[r] = m[r] == -INFINITY ? 0.0f : expf(m[r] - M);
        }
    }
    for (int w = 0; w < 4; w++) {
        if (wave == w) {
#pragma unroll
            for (int r = 0; r < RM; r++) {
                if (r < nr) {
#pragma unroll
                    for (int c = 0; c < VC; c++) {
                        const int d = lane + 64 * c;
                        if (d < vdim) accs[r * vdim + d] = (w == 0 ? 0.0f : accs[r * vdim + d]) + acc[r][c] * f[r];
                    }
                }
            }
        }
        __syncthreads();
    }
    T* o = (T*)a.out + (size_t)t * (a.out_ld ? a.out_ld : a.heads * vdim) + (size_t)h0 * vdim;
    const float osc = a.out_scale != 0.0f ? a.out_scale : 1.0f;
    for (int i = tid; i < nr * vdim; i += 256) {
        const int r = i / vdim;
        float M = -INFINITY;
        for (int w = 0; w < 4; w++) M = fmaxf(M, ml[(w * RM + r) * 2]);
        if (last && a.sink) M = fmaxf(M, a.sink[h0 + r]);
        float L = (last && a.sink) ? expf(a.sink[h0 + r] - M) : 0.0f;
        for (int w = 0; w < 4; w++) { const float mw = ml[(w * RM + r) * 2]; if (mw != -INFINITY) L += ml[(w * RM + r) * 2 + 1] * expf(mw - M); }
        if (last) {
            const float gt = a.out_gate ? 1.0f / (1.0f + expf(-a.out_gate[(size_t)t * a.ld_gate + (a.gate_elem ? (size_t)h0 * vdim + i : (size_t)(h0 + r))])) : 1.0f;
            sv_st(o + i, accs[i] / L * gt * osc);
        }
        else {
            const size_t slot = ((size_t)t * a.heads + h0 + r) * a.nsplit + sp;
            a.part_acc[slot * vdim + (i - r * vdim)] = accs[i];
            if (i == r * vdim) { a.part_ml[slot * 2] = M; a.part_ml[slot * 2 + 1] = L; }
        }
    }
    SV_STAMP(7);
}

// Prompt-sized steps: the same attention on the f32 matrix instruction (v_mfma_f32_16x16x4_f32: every product and sum stays f32).  A workgroup owns 16
// query ROWS that share one key / value head -- the heads of its group for one token, or for 16 / R consecutive tokens of one request when the group has
// fewer than 16 heads (a row carries its own position, so the causal and window masks are per row) -- and its four waves split the blocks of 64 keys.
// Both products are formed TRANSPOSED so that nothing is shuffled between them:
//   S^T[key][row] = K Q^T   (A = key rows, B = the rows' queries, held in registers for the whole launch)
//   O^T[d][row]  += V^T P^T (A = value columns, B = the weights exactly where the first product left them: lane = row, register = key)
// so a lane's accumulators all belong to ONE row and the online-softmax rescale is a per-lane scalar.  The reduction index of an MFMA is spread over the
// four 16-lane groups; group q takes the CONTIGUOUS quarter q of a key row (dim / 4 elements, 16-byte loads) and the keys 4 q .. 4 q + 3 of a 16-key block.
typedef float sv_f4 __attribute__((ext_vector_type(4)));
template <typename T, int DQ, int DB, int NKB = 4>      // DQ = dim / 4 query elements per lane, DB = vdim / 16 value columns per lane, NKB = blocks of 16 keys a wave takes at a time
__global__ void __launch_bounds__(256) sv_attn_mfma_kernel(const KrSvAttn a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int VEC = 16 / sizeof(T);
    const int G = a.kv_heads, R = a.heads / G, dim = DQ * 4, vdim = DB * 16;
    const int Rb = R < 16 ? R : 16, TQ = a.tq;             // tokens per workgroup: 16 / Rb for prompt portions, 1 for decode-shaped steps (rows past TQ * Rb idle)
    const int sp = blockIdx.z % a.nsplit, hb = blockIdx.z / a.nsplit;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, row = lane & 15, qd = lane >> 4;
    const int g = blockIdx.y, h_row = g * R + hb * 16 + (row % Rb), t0 = blockIdx.x * TQ, tq_row = row / Rb;
    float* ml = lds;                    // [4 waves][16 rows][2]
    float* mf = lds + 4 * 16 * 2;       // [16 rows][2]: the merged maximum and 1 / denominator (or the denominator itself in a split launch)
    // [16 rows][AS]: a row is vdim + 65 floats long and the column block of lane group qd starts 16 floats late, so that the 64 lanes of a wave, which hold the
    // same column of 16 rows x 4 groups, fall into distinct LDS banks (rows of exactly vdim floats put all of them into ONE bank)
    float* accs = mf + 16 * 2;
    constexpr int AS = DB * 16 + 65;
    auto acc_at = [](int r, int c) { return r * AS + c + (c / (4 * DB)) * 16; };
    const T* kp = (const T*)a.kpool; const T* vp = (const T*)a.vpool;
    for (int base = 0; base < TQ && t0 + base < a.T;) {
        // the run of tokens [base, end) of this group that continue one request (same slot, consecutive positions)
        const int sl = a.slot[t0 + base], p0 = a.pos[t0 + base];
        int end = base + 1;
        while (end < TQ && t0 + end < a.T && a.slot[t0 + end] == sl && a.pos[t0 + end] == p0 + (end - base)) end++;
        const bool rv = tq_row >= base && tq_row < end;
        const int p_row = rv ? p0 + (tq_row - base) : -1;
        const int lo_row = a.window > 0 ? max(0, p_row - a.window + 1) : (a.chunk > 0 && rv ? p_row - p_row % a.chunk : 0);
        const int hi = p0 + (end - base - 1), lo = a.window > 0 ? max(0, p0 - a.window + 1) : (a.chunk > 0 ? p0 - p0 % a.chunk : 0);
        const float slope_row = (a.slopes && rv) ? a.slopes[h_row] : 0.0f;
        const int* table = a.page_table + (size_t)sl * a.table_ld;
        float q[DQ];
        {
            const float* qp = a.qkv + (size_t)(t0 + (rv ? tq_row : base)) * a.ldq + (size_t)h_row * dim + qd * DQ;
#pragma unroll
            for (int i = 0; i < DQ; i++) q[i] = rv ? qp[i] * a.scale : 0.0f;
        }
        float m = -INFINITY, l = 0.0f;
        sv_f4 acc[DB];
#pragma unroll
        for (int d = 0; d < DB; d++) acc[d] = sv_f4{0.0f, 0.0f, 0.0f, 0.0f};
        constexpr int KEYS = 16 * NKB;
        const int nch = (hi - lo) / KEYS + 1, cps = (nch + a.nsplit - 1) / a.nsplit, c0 = sp * cps, c1 = min(nch, c0 + cps);
        for (int cb = c0 + wave; cb < c1; cb += 4) {
            const int j0 = lo + KEYS * cb;
            // ---- S^T: NKB blocks of 16 keys
            sv_f4 st[NKB];
            int prow[NKB];
#pragma unroll
            for (int kb = 0; kb < NKB; kb++) {
                const int key = min(j0 + kb * 16 + row, hi);         // keys past the last one are fetched again and masked
                prow[kb] = table[key / a.page_tokens] * a.page_tokens + (key % a.page_tokens);
            }
#pragma unroll
            for (int kb = 0; kb < NKB; kb++) {
                const T* k = kp + (size_t)prow[kb] * a.ldk + (size_t)g * dim + qd * DQ;
                // a key row's quarter in batches of at most PB 16-byte pieces: long rows (a latent cache row) must not hold all of it in registers at once
                constexpr int NP = DQ / VEC, PB = NP <= 8 ? NP : 6;
                sv_f4 c = sv_f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int u0 = 0; u0 < NP; u0 += PB) {
                    sv_u4 kv[PB];
#pragma unroll
                    for (int u = 0; u < PB; u++) if (u0 + u < NP) kv[u] = *reinterpret_cast<const sv_u4*>(k + (u0 + u) * VEC);
#pragma unroll
                    for (int u = 0; u < PB; u++) {
                        if (u0 + u >= NP) continue;
                        float kf[VEC];
                        if constexpr (sizeof(T) == 2) {
#pragma unroll
                            for (int i = 0; i < 4; i++) { kf[2 * i] = __uint_as_float(kv[u][i] << 16); kf[2 * i + 1] = __uint_as_float(kv[u][i] & 0xFFFF0000u); }
                        } else {
#pragma unroll
                            for (int i = 0; i < 4; i++) kf[i] = __uint_as_float(kv[u][i]);
                        }
#pragma unroll
                        for (int i = 0; i < VEC; i++) c = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[i], q[(u0 + u) * VEC + i], c, 0, 0, 0);
                    }
                }
                st[kb] = c;
            }
            // ---- masks and the online softmax of this lane's row (its 16 keys here, the other 48 in the three lanes 16 apart)
            float cm = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < NKB; kb++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int key = j0 + kb * 16 + 4 * qd + i;
                    const bool ok = rv && key <= p_row && key >= lo_row;
                    const float sc = a.softcap > 0.0f ? a.softcap * tanhf(st[kb][i] / a.softcap) : st[kb][i];
                    st[kb][i] = ok ? sc - slope_row * (float)(p_row - key) : -INFINITY;
                    cm = fmaxf(cm, st[kb][i]);
                }
            cm = fmaxf(cm, __shfl_xor(cm, 16)); cm = fmaxf(cm, __shfl_xor(cm, 32));
            const float mn = fmaxf(m, cm);
            const float alpha = mn == -INFINITY ? 1.0f : expf(m - mn);       // a row that has seen no key yet keeps its zero state
            float ps = 0.0f;
#pragma unroll
            for (int kb = 0; kb < NKB; kb++)
#pragma unroll
                for (int i = 0; i < 4; i++) { const float pj = st[kb][i] == -INFINITY ? 0.0f : expf(st[kb][i] - mn); st[kb][i] = pj; ps += pj; }
            ps += __shfl_xor(ps, 16); ps += __shfl_xor(ps, 32);
            l = l * alpha + ps; m = mn;
#pragma unroll
            for (int d = 0; d < DB; d++) acc[d] *= alpha;
            // ---- O^T += V^T P^T: key (kb, 4 qd + i) -> this lane reads its DB value columns of that key's row
            // wide values (DB > 16) go through in column batches of DC, so that one batch of four keys' values is in registers at a time
            constexpr int DC = DB <= 16 ? DB : 8;
#pragma unroll
            for (int kb = 0; kb < NKB; kb++) {
                int prk[4];
#pragma unroll
                for (int i = 0; i < 4; i++) prk[i] = __shfl(prow[kb], 4 * qd + i);
#pragma unroll
                for (int d0 = 0; d0 < DB; d0 += DC) {
                    float vf[4][DC];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const T* vr = vp + (size_t)prk[i] * a.ldv + (size_t)g * vdim + row * DB + d0;
                        if constexpr ((DC * sizeof(T)) % 16 == 0 && (DB * sizeof(T)) % 16 == 0) {
#pragma unroll
                            for (int u = 0; u < DC / VEC; u++) {
                                const sv_u4 vv = *reinterpret_cast<const sv_u4*>(vr + u * VEC);
                                if constexpr (sizeof(T) == 2) {
#pragma unroll
                                    for (int e = 0; e < 4; e++) { vf[i][u * VEC + 2 * e] = __uint_as_float(vv[e] << 16); vf[i][u * VEC + 2 * e + 1] = __uint_as_float(vv[e] & 0xFFFF0000u); }
                                } else {
#pragma unroll
                                    for (int e = 0; e < 4; e++) vf[i][u * VEC + e] = __uint_as_float(vv[e]);
                                }
                            }
                        } else {
#pragma unroll
                            for (int e = 0; e < DC; e++) vf[i][e] = sv_ld(vr + e);
                        }
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++)
#pragma unroll
                        for (int d = 0; d < DC; d++) acc[d0 + d] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[i][d], st[kb][i], acc[d0 + d], 0, 0, 0);
                }
            }
        }
        // ---- the four waves' states -> one, in wave order; an unsplit launch adds the sink and writes the output, a split one leaves (maximum, denominator, sums)
        const bool last = a.nsplit == 1;
        __syncthreads();
        if (qd == 0) { ml[(wave * 16 + row) * 2] = m; ml[(wave * 16 + row) * 2 + 1] = l; }
        __syncthreads();
        if (tid < 16) {
            const int h = g * R + hb * 16 + (tid % Rb);
            float Mr = -INFINITY;
            for (int w = 0; w < 4; w++) Mr = fmaxf(Mr, ml[(w * 16 + tid) * 2]);
            if (last && a.sink) Mr = fmaxf(Mr, a.sink[h]);
            float L = (last && a.sink) ? expf(a.sink[h] - Mr) : 0.0f;
            for (int w = 0; w < 4; w++) { const float mw = ml[(w * 16 + tid) * 2]; if (mw != -INFINITY) L += ml[(w * 16 + tid) * 2 + 1] * expf(mw - Mr); }
            mf[tid * 2] = Mr; mf[tid * 2 + 1] = last ? 1.0f / L : L;
        }
        __syncthreads();
        const float f = m == -INFINITY ? 0.0f : expf(m - mf[row * 2]);
        for (int w = 0; w < 4; w++) {
            if (wave == w) {
#pragma unroll
                for (int d = 0; d < DB; d++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int col = (4 * qd + i) * DB + d;
                        accs[acc_at(row, col)] = (w == 0 ? 0.0f : accs[acc_at(row, col)]) + acc[d][i] * f;
                    }
            }
            __syncthreads();
        }
        for (int i = tid; i < 16 * vdim; i += 256) {
            const int r = i / vdim, tq = r / Rb;
            if (tq < base || tq >= end) continue;
            const int h = g * R + hb * 16 + (r % Rb);
            const float av = accs[acc_at(r, i - r * vdim)];
            if (last) {
                const float gt = a.out_gate ? 1.0f / (1.0f + expf(-a.out_gate[(size_t)(t0 + tq) * a.ld_gate + (a.gate_elem ? (size_t)h * vdim + (i - r * vdim) : (size_t)h)])) : 1.0f;
                sv_st((T*)a.out + (size_t)(t0 + tq) * (a.out_ld ? a.out_ld : a.heads * vdim) + (size_t)h * vdim + (i - r * vdim), av * mf[r * 2 + 1] * gt * (a.out_scale != 0.0f ? a.out_scale : 1.0f));
            }
            else {
                const size_t slot = ((size_t)(t0 + tq) * a.heads + h) * a.nsplit + sp;
                a.part_acc[slot * vdim + (i - r * vdim)] = av;
                if (i == r * vdim) { a.part_ml[slot * 2] = mf[r * 2]; a.part_ml[slot * 2 + 1] = mf[r * 2 + 1]; }
            }
        }
        __syncthreads();
        base = end;
    }
}

// the partial states of a split launch -> output: one workgroup per (token, head).  The splits' weights exp(m_s - M) are formed once (LDS); a thread then owns
// value columns and its loads over the splits do not depend on one another
template <typename T>
__global__ void __launch_bounds__(256) sv_attn_merge_kernel(const KrSvAttn a) {
    extern __shared__ float wsp[];           // [nsplit] weight of every split, then 1 / denominator
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const size_t base = ((size_t)t * a.heads + h) * a.nsplit;
    float M = a.sink ? a.sink[h] : -INFINITY;
    for (int s = 0; s < a.nsplit; s++) M = fmaxf(M, a.part_ml[(base + s) * 2]);
    for (int s = tid; s < a.nsplit; s += 256) { const float ms = a.part_ml[(base + s) * 2]; wsp[s] = ms == -INFINITY ? 0.0f : expf(ms - M); }
    __syncthreads();
    if (tid == 0) {
        float L = a.sink ? expf(a.sink[h] - M) : 0.0f;
        for (int s = 0; s < a.nsplit; s++) if (wsp[s] != 0.0f) L = __builtin_fmaf(a.part_ml[(base + s) * 2 + 1], wsp[s], L);
        wsp[a.nsplit] = 1.0f / L;
    }
    __syncthreads();
    const float inv = wsp[a.nsplit] * ((a.out_gate && !a.gate_elem) ? 1.0f / (1.0f + expf(-a.out_gate[(size_t)t * a.ld_gate + h])) : 1.0f) * (a.out_scale != 0.0f ? a.out_scale : 1.0f);
    T* o = (T*)a.out + (size_t)t * (a.out_ld ? a.out_ld : a.heads * a.vdim) + (size_t)h * a.vdim;
    for (int d = tid; d < a.vdim; d += 256) {
        float v = 0.0f;
#pragma unroll 8
        for (int s = 0; s < a.nsplit; s++) { const float w = wsp[s], p = a.part_acc[(base + s) * a.vdim + d]; v = __builtin_fmaf(w != 0.0f ? p : 0.0f, w, v); }      // a split without keys counts as zeros
        if (a.out_gate && a.gate_elem) v *= 1.0f / (1.0f + expf(-a.out_gate[(size_t)t * a.ld_gate + (size_t)h * a.vdim + d]));
        sv_st(o + d, v * inv);
    }
}

// selection: one wave per token; the scores of the E experts live in LDS
// z holds the logits as `parts` column blocks of E that are added (a gate stored as two bf16 terms gives two)
__global__ void __launch_bounds__(64) sv_router_select_kernel(const float* __restrict__ z, int ld, int parts, const float* __restrict__ bias, int bias_mode, int score_kind,
                                                              int group_kind, int E, int top, int groups, int keep, int renorm, int* __restrict__ ids, float* __restrict__ wts) {
    extern __shared__ float lds[];           // s[E] scores | c[E] choice scores | gscore[groups] | allowed flags as floats [groups]
    float* s = lds; float* cs = lds + E; float* gs = cs + E; float* gok = gs + groups;
    const int t = blockIdx.x, lane = threadIdx.x;
    for (int e = lane; e < E; e += 64) {
        float v = z[(size_t)t * ld + e];
        for (int q = 1; q < parts; q++) v += z[(size_t)t * ld + (size_t)q * E + e];
        s[e] = (bias && bias_mode == 1) ? v + bias[e] : v;
    }
    __syncthreads();
    if (score_kind == 1) {
        for (int e = lane; e < E; e += 64) s[e] = 1.0f / (1.0f + expf(-s[e]));
    } else {
        float mx = -INFINITY;
        for (int e = lane; e < E; e += 64) mx = fmaxf(mx, s[e]);
        mx = sv_wave_max(mx);
        float sum = 0.0f;
        for (int e = lane; e < E; e += 64) { const float v = expf(s[e] - mx); s[e] = v; sum += v; }
        __syncthreads();
        sum = sv_wave_sum(sum);
        const float inv = 1.0f / sum;
        for (int e = lane; e < E; e += 64) s[e] *= inv;
    }
    for (int e = lane; e < E; e += 64) cs[e] = (bias && bias_mode == 2) ? s[e] + bias[e] : s[e];
    __syncthreads();
    const int per = E / groups;
    for (int gi = lane; gi < groups; gi += 64) {
        float v = -INFINITY, v2 = -INFINITY;       // the two largest of the group
        for (int e = gi * per; e < (gi + 1) * per; e++) { const float c = cs[e]; if (c > v) { v2 = v; v = c; } else if (c > v2) v2 = c; }
        gs[gi] = (group_kind == 1 && per > 1) ? v + v2 : v; gok[gi] = groups == keep ? 1.0f : 0.0f;
    }
    __syncthreads();
    if (keep < groups) {
        for (int r = 0; r < keep; r++) {         // r-th best group: largest score, lowest index among equals
            float bv = -INFINITY; int bi = 0x7fffffff;
            for (int gi = lane; gi < groups; gi += 64) if (gok[gi] == 0.0f && (gs[gi] > bv || (gs[gi] == bv && gi < bi))) { bv = gs[gi]; bi = gi; }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float ov = __shfl_xor(bv, o); const int oi = __shfl_xor(bi, o);
                if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
            }
            __syncthreads();
            if (lane == 0 && bi != 0x7fffffff) gok[bi] = 1.0f;
            __syncthreads();
        }
    }
    float wsum = 0.0f;
    for (int r = 0; r < top; r++) {
        float bv = -INFINITY; int bi = 0x7fffffff;
        for (int e = lane; e < E; e += 64) {
            const float v = cs[e];
            if (v != -INFINITY && gok[e / per] != 0.0f && (v > bv || (v == bv && e < bi))) { bv = v; bi = e; }      // a taken expert is marked by minus infinity
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o); const int oi = __shfl_xor(bi, o);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        __syncthreads();
        float wv;
        if (bi == 0x7fffffff) { bi = 0; wv = 0.0f; }      // fewer allowed experts than `top` (refused on the host): a zero-weight slot
        else { wv = s[bi]; if (lane == 0) cs[bi] = -INFINITY; }
        if (lane == 0) { ids[(size_t)t * top + r] = bi; wts[(size_t)t * top + r] = wv; }
        wsum += wv;
        __syncthreads();
    }
    if (renorm) {
        const float rinv = 1.0f / (wsum + 1e-20f);
        for (int r = lane; r < top; r += 64) wts[(size_t)t * top + r] *= rinv;
    }
}

__global__ void sv_fill_int_kernel(int* p, int n, int v) { const int i = blockIdx.x * blockDim.x + threadIdx.x; if (i < n) p[i] = v; }
__global__ void sv_moe_count_kernel(const int* __restrict__ ids, int n, int* __restrict__ counts) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) atomicAdd(&counts[ids[i]], 1);
}
__global__ void sv_moe_scan_kernel(const int* __restrict__ counts, int E, int* __restrict__ seg, int* __restrict__ cursor) {
    if (threadIdx.x == 0) {
        int o = 0;
        for (int e = 0; e < E; e++) { seg[e] = o; cursor[e] = 0; o += counts[e]; }
        seg[E] = o;
    }
}
__global__ void sv_moe_fill_kernel(const int* __restrict__ ids, int n, int top, const int* __restrict__ seg, int* __restrict__ cursor, int* __restrict__ src_row,
                                   int* __restrict__ row_group, int* __restrict__ pair_pos) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int e = ids[i];
    const int pos = seg[e] + atomicAdd(&cursor[e], 1);
    src_row[pos] = i / top; row_group[pos] = e; pair_pos[i] = pos;
}

// the three launches above as one workgroup, for decode-sized batches (n pairs <= 1024, E counters in LDS)
__global__ void __launch_bounds__(256) sv_moe_sort_small_kernel(const int* __restrict__ ids, int n, int top, int E, int* __restrict__ seg, int* __restrict__ src_row,
                                                                int* __restrict__ row_group, int* __restrict__ pair_pos) {
    extern __shared__ int cnt[];             // counts[E] | start[E]
    int* start = cnt + E;
    for (int e = threadIdx.x; e < E; e += 256) cnt[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += 256) atomicAdd(&cnt[ids[i]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int o = 0;
        for (int e = 0; e < E; e++) { start[e] = o; seg[e] = o; o += cnt[e]; cnt[e] = 0; }
        seg[E] = o;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += 256) {
        const int e = ids[i];
        const int pos = start[e] + atomicAdd(&cnt[e], 1);
        src_row[pos] = i / top; row_group[pos] = e; pair_pos[i] = pos;
    }
}

template <typename T>
__global__ void sv_act_kernel(const float* __restrict__ gu, int ld, T* __restrict__ y, int M, int F, int kind, float limit, float alpha) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)M * F) return;
    const size_t r = i / F; const int c = (int)(i - r * F);
    float g = gu[r * ld + c], u = kind == KR_SV_ACT_RELU2 ? 0.0f : gu[r * ld + F + c], v;
    if (kind == KR_SV_ACT_RELU2) {
        g = fmaxf(g, 0.0f); v = g * g;
    } else if (kind == KR_SV_ACT_GELU_TANH) {
        const float in = 0.7978845608028654f * (g + 0.044715f * g * g * g);
        v = 0.5f * g * (1.0f + tanhf(in)) * u;
    } else if (kind == KR_SV_ACT_CLAMPED_SWIGLU) {
        g = fminf(g, limit); u = fminf(fmaxf(u, -limit), limit);
        v = g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
    } else {
        v = g / (1.0f + expf(-g)) * u;
    }
    sv_st(y + i, v);
}

// one workgroup per token: the sublayers' output row is formed in LDS, normed there when the design norms sublayer outputs, gated when the design gates
// them, added to the residual row, and the new row is written back and handed on in the storage type -- normed for the next sublayer (norm_w) or as it is
// NT threads: 256 for prompt-sized steps (many rows), 1024 for decode-sized ones, where a row's workgroup is alone on its compute unit and the
// per-thread chain of columns is what the launch waits for
template <typename T, int KIND, int NT>
__global__ void __launch_bounds__(NT) sv_residual_norm_kernel(const KrSvResidual a, T* __restrict__ h_out) {
    extern __shared__ float xr[];            // [width] | [2 * groups]
    __shared__ float red[NT / 64];
    __shared__ int pp_s[64]; __shared__ float w_s[64];      // the token's expert rows and weights, read once (top <= 64; more fall back to global reads)
    const size_t t = blockIdx.x;
    const int width = a.width, top = a.top;
    float* gst = xr + width;
    const float* __restrict__ rows = a.rows; const float* __restrict__ mix = a.mix; const float* __restrict__ dense = a.dense; const float* __restrict__ shared = a.shared;
    float* __restrict__ x = a.x;
    if (a.canon_state) {                     // the mixer's un-convolved input of this token is kept when it is among the last canon_keep of its portion
        const int K = a.canon_keep, sl = a.slot[t];
        if ((int)t + K >= a.T || a.slot[t + K] != sl) {
            float* dst = a.canon_state + ((size_t)sl * K + a.pos[t] % K) * width;
            for (int c = threadIdx.x; c < width; c += NT) dst[c] = a.h32_in[t * width + c];
        }
    }
    const bool staged = rows && top <= 64;
    if (staged && threadIdx.x < top) { pp_s[threadIdx.x] = a.pair_pos[t * top + threadIdx.x]; w_s[threadIdx.x] = a.wts[t * top + threadIdx.x]; }
    if (rows) __syncthreads();
    auto gate_at = [&](int c) {
        const float z = a.gate[t * a.ld_gate + c] + (a.gate_b ? a.gate_b[c] : 0.0f);
        return 1.0f / (1.0f + expf(-z));
    };
    float s1 = 0.0f;
    for (int c = threadIdx.x; c < width; c += NT) {
        const size_t i = t * width + c;
        float ff = 0.0f; bool any = false;
        if (rows) {
            if (staged) {
#pragma unroll 4
                for (int s = 0; s < top; s++) ff = __builtin_fmaf(w_s[s], rows[(size_t)pp_s[s] * width + c], ff);
            } else {
                for (int s = 0; s < top; s++) ff = __builtin_fmaf(a.wts[t * top + s], rows[(size_t)a.pair_pos[t * top + s] * width + c], ff);
            }
            any = true;
        }
        if (shared) { ff = any ? ff + shared[i] : shared[i]; any = true; }
        if (dense) { ff = any ? ff + dense[i] : dense[i]; any = true; }
        float d = mix ? mix[i] : 0.0f;
        if (mix && a.mix_bias) d += a.mix_bias[c];
        if (any) d = mix ? d + ff : ff;
        if (a.post_w) { xr[c] = d; s1 += d; continue; }      // the sum waits for its norm
        if (a.gate) d *= gate_at(c);
        const float v = x[i] + a.mult * d;
        x[i] = v; xr[c] = v; s1 += v;
    }
    if (a.post_w) {
        float mean = 0.0f, inv = 0.0f;
        if (a.groups > 1) { __syncthreads(); sv_group_stats<KIND, NT / 64>(xr, width, a.groups, a.eps, gst); __syncthreads(); }
        else {
            if constexpr (KIND == KR_SV_NORM_LAYER) mean = sv_block_sum<NT / 64>(s1, red) / (float)width;
            float q = 0.0f;
            for (int c = threadIdx.x; c < width; c += NT) { const float dv = xr[c] - mean; q = __builtin_fmaf(dv, dv, q); }
            inv = 1.0f / sqrtf(sv_block_sum<NT / 64>(q, red) / (float)width + a.eps);
        }
        const int gw = a.groups > 1 ? width / a.groups : width;
        s1 = 0.0f;
        for (int c = threadIdx.x; c < width; c += NT) {
            const size_t i = t * width + c;
            if (a.groups > 1) { mean = gst[2 * (c / gw)]; inv = gst[2 * (c / gw) + 1]; }
            float y = (xr[c] - mean) * inv * a.post_w[c];
            if (a.post_b) y += a.post_b[c];
            if (a.gate) y *= gate_at(c);
            const float v = x[i] + a.mult * y;
            x[i] = v; xr[c] = v; s1 += v;
        }
    }
    if (!h_out) return;
    if (!a.norm_w) {
        for (int c = threadIdx.x; c < width; c += NT) { sv_st(h_out + t * width + c, xr[c]); if (a.h32_out) a.h32_out[t * width + c] = xr[c]; }
        return;
    }
    float mean = 0.0f, inv = 0.0f;
    if (a.groups > 1) { __syncthreads(); sv_group_stats<KIND, NT / 64>(xr, width, a.groups, a.eps, gst); __syncthreads(); }
    else {
        if constexpr (KIND == KR_SV_NORM_LAYER) mean = sv_block_sum<NT / 64>(s1, red) / (float)width;
        float q = 0.0f;
        for (int c = threadIdx.x; c < width; c += NT) { const float dv = xr[c] - mean; q = __builtin_fmaf(dv, dv, q); }      // a thread re-reads its own columns
        inv = 1.0f / sqrtf(sv_block_sum<NT / 64>(q, red) / (float)width + a.eps);
    }
    const int gw = a.groups > 1 ? width / a.groups : width;
    for (int c = threadIdx.x; c < width; c += NT) {
        if (a.groups > 1) { mean = gst[2 * (c / gw)]; inv = gst[2 * (c / gw) + 1]; }
        float v = (xr[c] - mean) * inv * a.norm_w[c];
        if (a.norm_b) v += a.norm_b[c];
        sv_st(h_out + t * width + c, v);
        if (a.h32_out) a.h32_out[t * width + c] = v;
    }
}

// ---- latent mixer
// one workgroup per (token, part): part 0 norms the query latent, part 1 norms the key / value latent into the cache row and turns the shared key part
template <typename T>
__global__ void __launch_bounds__(256) sv_latent_prep_kernel(const KrSvLatent a) {
    __shared__ float red[4];
    const int t = blockIdx.x, part = blockIdx.y;
    const float* z = a.dz + (size_t)t * a.ld + (part ? a.q_rank : 0);
    const int n = part ? a.kv_rank : a.q_rank;
    const float* w = part ? a.dkv_norm_w : a.dq_norm_w;
    T* dst;
    if (part) {
        const int p = a.pos[t];
        const size_t page = (size_t)a.page_table[(size_t)a.slot[t] * a.table_ld + p / a.page_tokens];
        dst = (T*)a.pool + (page * a.page_tokens + (p % a.page_tokens)) * (size_t)(a.kv_rank + a.rot);
    } else dst = (T*)a.cq + (size_t)t * a.q_rank;
    float q = 0.0f;
    for (int c = threadIdx.x; c < n; c += 256) q = __builtin_fmaf(z[c], z[c], q);
    const float inv = 1.0f / sqrtf(sv_block_sum<4>(q, red) / (float)n + a.eps);
    for (int c = threadIdx.x; c < n; c += 256) sv_st(dst + c, z[c] * inv * w[c]);
    if (part) {
        const float2* cs = a.cs + (size_t)t * (a.rot / 2);
        for (int i = threadIdx.x; i < a.rot / 2; i += 256) {
            const float u = z[n + 2 * i], v = z[n + 2 * i + 1];
            const float2 c = cs[i];
            sv_st(dst + n + 2 * i, u * c.x - v * c.y); sv_st(dst + n + 2 * i + 1, v * c.x + u * c.y);
        }
    }
}
// one wave per (token, head)
template <typename T>
__global__ void __launch_bounds__(64) sv_latent_q_kernel(const KrSvLatent a, const float* __restrict__ q2, T* __restrict__ qn, float* __restrict__ qe) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* q = q2 + ((size_t)t * a.heads + h) * (a.dim + a.rot);
    T* n = qn + ((size_t)t * a.heads + h) * a.dim;
    for (int d = lane; d < a.dim; d += 64) sv_st(n + d, q[d]);
    float* e = qe + ((size_t)t * a.heads + h) * (a.kv_rank + a.rot) + a.kv_rank;
    const float2* cs = a.cs + (size_t)t * (a.rot / 2);
    for (int i = lane; i < a.rot / 2; i += 64) {
        const float u = q[a.dim + 2 * i], v = q[a.dim + 2 * i + 1];
        const float2 c = cs[i];
        e[2 * i] = u * c.x - v * c.y; e[2 * i + 1] = v * c.x + u * c.y;
    }
}
__global__ void sv_head_rows_kernel(int T, int heads, int* __restrict__ seg, int* __restrict__ rows, int* __restrict__ group) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i <= heads) seg[i] = i * T;
    if (i >= T * heads) return;
    const int h = i / T, t = i - h * T;
    rows[i] = t * heads + h; group[i] = h;
}

// ---- recurrent mixers (KrSvLin)
// One WAVE per (request of the step, head, block of 16 value columns): lane = 4 * column + part, and a lane keeps the rows [part * dpr, (part + 1) * dpr) of
// its column of S in registers for the whole portion (dpr = ceil(dim / 4) <= DP).  The tokens of the portion are walked in order; TB of them at a time are
// staged in LDS (q and k of the head with the rotation and the scales applied, the 16 value columns, the two gates), so the serial loop reads LDS only.
// Per token a lane does dpr updates S <- a S + (b v) k and dpr products for o, and the four parts of a column meet through two lane exchanges.
#define SV_WAVE_SYNC() do { __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront"); } while (0)
template <int KIND, int DP>
__global__ void __launch_bounds__(64) sv_lin_scan_kernel(const KrSvLin a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int TB = 8;
    constexpr bool ML = KIND == 3, GLA = KIND == 4, SSD = KIND == 5;
    const int e = blockIdx.x, h = blockIdx.y, cb = blockIdx.z, lane = threadIdx.x;
    const int part = lane & 3, cl = lane >> 2, col = cb * 16 + cl;
    const int dim = a.dim, vdim = a.vdim, H = a.heads, ncb = (vdim + 15) / 16;
    const int dpr = (dim + 3) / 4, dimp = 4 * dpr;
    const int t0 = a.ent_off[e], t1 = a.ent_off[e + 1], sl = a.ent_slot[e];
    const bool fresh = a.pos[t0] == 0, cv = col < vdim;
    float* Sg = a.state + (size_t)sl * a.state_stride + ((size_t)h * vdim + (cv ? col : 0)) * dim + part * dpr;
    float* nmg = a.nm + (size_t)sl * a.nm_stride + ((size_t)h * ncb + cb) * (dim + 4);
    float S[DP], n[DP];
#pragma unroll
    for (int r = 0; r < DP; r++) {
        const int row = part * dpr + r;
        const bool ok = r < dpr && row < dim && !fresh;
        S[r] = (ok && cv) ? Sg[r] : 0.0f;
        n[r] = (ML && ok) ? nmg[row] : 0.0f;
    }
    float m = (ML && !fresh) ? nmg[dim] : 0.0f;
    const float decay = KIND == 2 ? a.decay[h] : 0.0f;
    float* qs = lds; float* ks = qs + TB * dimp; float* vs = ks + TB * dimp; float* gs = vs + TB * 16; float* as = gs + TB * 2;      // as [TB * dimp]: per-channel decays (gla)
    const int half = a.rot_dims / 2;
    for (int tb = t0; tb < t1; tb += TB) {
        const int nt = min(TB, t1 - tb);
        if constexpr (GLA || SSD) {
            const int hq = h / a.qk_group;
            for (int idx = lane; idx < nt * dimp; idx += 64) {
                const int tt = idx / dimp, d = idx - tt * dimp;
                const size_t r = (size_t)(tb + tt) * a.src_ld + (size_t)hq * dim + d;
                qs[idx] = d < dim ? a.qsrc[r] * a.q_scale : 0.0f;
                ks[idx] = d < dim ? a.ksrc[r] * a.k_scale : 0.0f;
                if constexpr (GLA) {
                    float al = 0.0f;
                    if (d < dim) {
                        const float z = a.gz[(size_t)(tb + tt) * a.gz_ld + (size_t)h * dim + d] + a.gz_bias[(size_t)h * dim + d];
                        al = expf((fminf(z, 0.0f) - log1pf(expf(-fabsf(z)))) * a.inv_tau);      // sigmoid(z)^(1 / tau)
                    }
                    as[idx] = al;
                }
            }
            for (int idx = lane; idx < nt * 16; idx += 64) {
                const int tt = idx >> 4, c = cb * 16 + (idx & 15);
                vs[idx] = c < vdim ? a.vsrc[(size_t)(tb + tt) * a.src_ld + (size_t)h * vdim + c] : 0.0f;
            }
            if (SSD && lane < nt) {
                const float z = a.dtz[(size_t)(tb + lane) * a.dtz_ld + h] + a.dt_bias[h];
                const float dt = fmaxf(z, 0.0f) + log1pf(expf(-fabsf(z)));                      // softplus
                gs[2 * lane] = dt; gs[2 * lane + 1] = -expf(a.a_log[h]) * dt;
            }
        } else {
        for (int idx = lane; idx < nt * dimp; idx += 64) {
            const int tt = idx / dimp, d = idx - tt * dimp;
            const float* zr = a.z + (size_t)(tb + tt) * a.ld + (size_t)h * dim;
            qs[idx] = d < dim ? zr[d] * a.q_scale : 0.0f;
            ks[idx] = d < dim ? zr[(size_t)H * dim + d] * a.k_scale : 0.0f;
        }
        for (int idx = lane; idx < nt * 16; idx += 64) {
            const int tt = idx >> 4, c = cb * 16 + (idx & 15);
            vs[idx] = c < vdim ? a.z[(size_t)(tb + tt) * a.ld + (size_t)2 * H * dim + (size_t)h * vdim + c] : 0.0f;
        }
        if (ML && lane < nt) {
            const float* zg = a.z + (size_t)(tb + lane) * a.ld + (size_t)2 * H * dim + (size_t)2 * H * vdim;
            float zi = zg[h] + a.i_bias[h], zf = zg[H + h] + a.f_bias[h];
            if (a.gate_cap > 0.0f) { zi = a.gate_cap * tanhf(zi / a.gate_cap); zf = a.gate_cap * tanhf(zf / a.gate_cap); }
            gs[2 * lane] = zi;
            gs[2 * lane + 1] = fminf(zf, 0.0f) - log1pf(expf(-fabsf(zf)));      // log sigmoid
        }
        }
        SV_WAVE_SYNC();
        if (half > 0) {
            for (int idx = lane; idx < nt * half; idx += 64) {
                const int tt = idx / half, i = idx - tt * half;
                const float2 c = a.cs[(size_t)(tb + tt) * half + i];
                float* qp = qs + tt * dimp; float* kp = ks + tt * dimp;
                const float qu = qp[i], qv = qp[i + half], ku = kp[i], kv = kp[i + half];
                qp[i] = qu * c.x - qv * c.y; qp[i + half] = qv * c.x + qu * c.y;
                kp[i] = ku * c.x - kv * c.y; kp[i + half] = kv * c.x + ku * c.y;
            }
            SV_WAVE_SYNC();
        }
        for (int tt = 0; tt < nt; tt++) {
            const float* qp = qs + tt * dimp + part * dpr; const float* kp = ks + tt * dimp + part * dpr;
            const float v = vs[tt * 16 + cl];
            float av, bv;
            if constexpr (ML) {
                const float ig = gs[2 * tt], fg = gs[2 * tt + 1];
                const float mn = fmaxf(fg + m, ig);
                av = expf(fg + m - mn); bv = expf(ig - mn); m = mn;
            } else if constexpr (SSD) { bv = gs[2 * tt]; av = expf(gs[2 * tt + 1]); }
            else { av = decay; bv = 1.0f; }
            const float* ap = as + tt * dimp + part * dpr;
            const float bvv = bv * v;
            float po = 0.0f, pn = 0.0f;
#pragma unroll
            for (int r = 0; r < DP; r++) {
                if (r < dpr) {
                    const float kr = kp[r], qr = qp[r];
                    if constexpr (GLA) S[r] = __builtin_fmaf(kr, bvv, ap[r] * S[r]);
                    else S[r] = __builtin_fmaf(kr, bvv, av * S[r]);
                    po = __builtin_fmaf(S[r], qr, po);
                    if constexpr (ML) { n[r] = __builtin_fmaf(bv, kr, av * n[r]); pn = __builtin_fmaf(n[r], qr, pn); }
                }
            }
            po += __shfl_xor(po, 1); po += __shfl_xor(po, 2);
            if constexpr (ML) {
                pn += __shfl_xor(pn, 1); pn += __shfl_xor(pn, 2);
                po = po / (fmaxf(fabsf(pn), expf(-m)) + 1e-6f);
            }
            if (part == 0 && cv) a.o[(size_t)(tb + tt) * H * vdim + (size_t)h * vdim + col] = po;
        }
        SV_WAVE_SYNC();
    }
#pragma unroll
    for (int r = 0; r < DP; r++) {
        const int row = part * dpr + r;
        if (r < dpr && row < dim) {
            if (cv) Sg[r] = S[r];
            if (ML && cl == 0) nmg[row] = n[r];
        }
    }
    if (ML && lane == 0) nmg[dim] = m;
}

// Prompt portions of the gla and state-space mixers (kinds 4, 5): the same recurrence, token by token, laid out for the length of the serial chain:
// what a portion waits for is the instructions ONE wave issues per token, so a head's state is spread over as many lanes as the chip has to spare.
// One WORKGROUP of four waves per (request, head, block of 8 value columns); a wave owns 2 columns, lane = 32 * column + part, and a lane keeps the rows
// [part * dpr, (part + 1) * dpr) of its column of S in registers (dpr = ceil(dim / 32) <= DP): a token costs a lane dpr updates and dpr products, and the
// thirty-two parts of a column meet in four exchanges inside their rows of 16 lanes and one across the two rows.  Tokens are staged 16 at a time in one
// of two LDS buffers: the loads of the next 16 are issued before the current 16 are walked and land in registers meanwhile (one barrier per 16
// tokens); the walk itself has no branch and no store (the 16 outputs of a lane leave together afterwards), so the LDS reads of the following tokens
// are in flight while one is worked on.  a.gz holds the decays themselves (sv_gla_decay_kernel).
// PIPE: the walk as an explicit pipeline (the next token's rows are read before the current one is worked on, the lane exchanges of all 16 tokens are done
// together afterwards) -- shorter when a workgroup has its compute unit to itself; with several workgroups per compute unit the plain walk (token after
// token, each with its own exchanges) leaves more of the issue slots to the others and the launch is over sooner.
template <int KIND, int DP, bool PIPE>
__global__ void __launch_bounds__(256) sv_lin_scanw_kernel(const KrSvLin a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int TB = 16, NC = 8;           // tokens per batch, value columns per workgroup
    constexpr bool GLA = KIND == 4, SSD = KIND == 5;
    const int e = blockIdx.x, h = blockIdx.y, cb = blockIdx.z, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int part = lane & 31, cl = wave * 2 + (lane >> 5), col = cb * NC + cl;
    const int dim = a.dim, vdim = a.vdim, H = a.heads;
    // a lane's dpr rows stand together in LDS, the parts of a token `pitch` floats apart: dpr + 4 where dpr is a multiple of 8, so that the 16-byte reads of
    // neighbouring parts fall into distinct banks
    const int dpr = (dim + 31) / 32, pitch = (dpr % 8 == 0) ? dpr + 4 : dpr, dimp = 32 * pitch;
    const int t0 = a.ent_off[e], t1 = a.ent_off[e + 1], sl = a.ent_slot[e];
    const bool fresh = a.pos[t0] == 0, cv = col < vdim;
    float* Sg = a.state + (size_t)sl * a.state_stride + ((size_t)h * vdim + (cv ? col : 0)) * dim + part * dpr;
    float S[DP];
#pragma unroll
    for (int r = 0; r < DP; r++) S[r] = (r < dpr && part * dpr + r < dim && !fresh && cv) ? Sg[r] : 0.0f;
    const int per = (GLA ? 3 : 2) * TB * dimp + TB * NC + TB * 2;      // floats of one buffer: q | k | (decays) | v | gates
    const int hq = h / a.qk_group;
    // staging: thread (token tid / 16 of the batch, row tid % 16 + 16 j of the head) -- 2 dpr elements of q, of k and of the decays per thread and batch.
    // fetch() is loads and nothing else (clamped addresses, no use of a loaded value), so that no wait stands between it and the walk over the current
    // batch; scales, masks and the gates' functions are applied when the registers go to LDS
    float pq[2 * DP], pk[2 * DP], pa[2 * DP], pv = 0.0f, pg = 0.0f;
    const int ft = tid >> 4, fd = tid & 15;
    int gd[2 * DP], li[2 * DP];              // per staged element: its column in the head's row (clamped) and its place in an LDS buffer
    unsigned real = 0;                       // bit j: the element exists (rows past dim are staged as zeros)
#pragma unroll
    for (int j = 0; j < 2 * DP; j++) {
        const int d = fd + 16 * j, pp = dpr == DP ? d / DP : d / dpr;
        gd[j] = min(d, dim - 1); li[j] = ft * dimp + pp * pitch + (d - pp * dpr);
        if (d < dim) real |= 1u << j;
    }
    auto fetch = [&](int tb) {               // global -> registers
        const int nt = min(TB, t1 - tb), tok = tb + min(ft, nt - 1);
        const size_t rb = (size_t)tok * a.src_ld + (size_t)hq * dim;
#pragma unroll
        for (int j = 0; j < 2 * DP; j++) {
            if (j < 2 * dpr) {
                const int d = gd[j];
                pq[j] = a.qsrc[rb + d]; pk[j] = a.ksrc[rb + d];
                if constexpr (GLA) pa[j] = a.gz[(size_t)tok * a.gz_ld + (size_t)h * dim + d];
            }
        }
        pv = a.vsrc[(size_t)(tb + min(tid >> 3, nt - 1)) * a.src_ld + (size_t)h * vdim + min(cb * NC + (tid & 7), vdim - 1)];      // threads below 128: (token, column)
        if constexpr (SSD) pg = a.dtz[(size_t)(tb + min(tid, nt - 1)) * a.dtz_ld + h];
    };
    const float ssd_rate = SSD ? -expf(a.a_log[h]) : 0.0f, ssd_bias = SSD ? a.dt_bias[h] : 0.0f;
    auto stash = [&](float* buf, int tb) {   // registers -> LDS
        const int nt = min(TB, t1 - tb);
        float* qs = buf; float* ks = qs + TB * dimp; float* as = ks + TB * dimp; float* vs = buf + (GLA ? 3 : 2) * TB * dimp; float* gs = vs + TB * NC;
#pragma unroll
        for (int j = 0; j < 2 * DP; j++)
            if (j < 2 * dpr) {
                const int idx = li[j];
                const bool ok = ft < nt && ((real >> j) & 1u);
                qs[idx] = ok ? pq[j] * a.q_scale : 0.0f; ks[idx] = ok ? pk[j] * a.k_scale : 0.0f;
                if constexpr (GLA) as[idx] = ok ? pa[j] : 0.0f;
            }
        if (tid < TB * NC) vs[tid] = ((tid >> 3) < nt && cb * NC + (tid & 7) < vdim) ? pv : 0.0f;
        if (SSD && tid < TB) {
            const float z = pg + ssd_bias;
            const float dt = fmaxf(z, 0.0f) + log1pf(expf(-fabsf(z)));      // softplus
            gs[2 * tid] = dt; gs[2 * tid + 1] = expf(ssd_rate * dt);
        }
    };
    fetch(t0); stash(lds, t0);
    __syncthreads();
    int b = 0;
    for (int tb = t0; tb < t1; tb += TB, b ^= 1) {
        const int nt = min(TB, t1 - tb);
        const bool more = tb + TB < t1;
        if (more) fetch(tb + TB);
        const float* buf = lds + b * per;
        const float* qs = buf; const float* ks = qs + TB * dimp; const float* as = ks + TB * dimp; const float* vs = buf + (GLA ? 3 : 2) * TB * dimp; const float* gs = vs + TB * NC;
        float outv[TB];
        if constexpr (PIPE) {
        // The walk, written as a pipeline: the lane's rows of q, k and the decays of token tt + 1 are read from LDS (16-byte reads when the lane's rows
        // fill DP) before token tt is worked on, and a token leaves only its lane's partial sum -- the exchanges among the 32 parts of a column are done
        // for all 16 tokens together afterwards, as 16 independent chains.  The state stays in registers; only S is carried from token to token.
        constexpr int G = 1;      // tokens read from LDS together, one group ahead of the group that is worked on
        float qq[2][G][DP], kk[2][G][DP], dd[2][G][DP], vv[2][G], g0[2][G], g1[2][G];      // two register sets, taken in turn (the loops are unrolled: every index is a constant)
        auto read = [&](int set, int t0g) {
            auto& qn = qq[set]; auto& kn = kk[set]; auto& dn = dd[set]; auto& vn = vv[set]; auto& g0n = g0[set]; auto& g1n = g1[set];
#pragma unroll
            for (int j = 0; j < G; j++) {
                const int tt = t0g + j;
                const float* qp = qs + tt * dimp + part * pitch; const float* kp = ks + tt * dimp + part * pitch; const float* ap = as + tt * dimp + part * pitch;
                if (dpr == DP) {
#pragma unroll
                    for (int r = 0; r < DP; r += 4) {
                        const float4 q4 = *reinterpret_cast<const float4*>(qp + r), k4 = *reinterpret_cast<const float4*>(kp + r);
                        qn[j][r] = q4.x; qn[j][r + 1] = q4.y; qn[j][r + 2] = q4.z; qn[j][r + 3] = q4.w; kn[j][r] = k4.x; kn[j][r + 1] = k4.y; kn[j][r + 2] = k4.z; kn[j][r + 3] = k4.w;
                        if constexpr (GLA) { const float4 a4 = *reinterpret_cast<const float4*>(ap + r); dn[j][r] = a4.x; dn[j][r + 1] = a4.y; dn[j][r + 2] = a4.z; dn[j][r + 3] = a4.w; }
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < DP; r++) { qn[j][r] = r < dpr ? qp[r] : 0.0f; kn[j][r] = r < dpr ? kp[r] : 0.0f; if constexpr (GLA) dn[j][r] = r < dpr ? ap[r] : 0.0f; }
                }
                vn[j] = vs[tt * NC + cl];
                g0n[j] = SSD ? gs[2 * tt] : 1.0f; g1n[j] = SSD ? gs[2 * tt + 1] : 1.0f;
            }
        };
        read(0, 0);
        auto walk = [&](auto full) {             // full: all 16 tokens of the batch exist -- no branch anywhere in the walk
#pragma unroll
        for (int tg = 0; tg < TB; tg += G) {
            const int cur = (tg / G) & 1;
            if (tg + G < TB) read(cur ^ 1, tg + G);
            auto& qv = qq[cur]; auto& kv = kk[cur]; auto& dv = dd[cur];
            float av[G], bvv[G];
#pragma unroll
            for (int j = 0; j < G; j++) { av[j] = g1[cur][j]; bvv[j] = SSD ? vv[cur][j] * g0[cur][j] : vv[cur][j]; }
#pragma unroll
            for (int j = 0; j < G; j++) {
                const int tt = tg + j;
                float po0 = 0.0f, po1 = 0.0f;
                if (decltype(full)::value || tt < nt) {
#pragma unroll
                    for (int r = 0; r < DP; r += 2) {
                        if constexpr (GLA) { S[r] = __builtin_fmaf(kv[j][r], bvv[j], dv[j][r] * S[r]); S[r + 1] = __builtin_fmaf(kv[j][r + 1], bvv[j], dv[j][r + 1] * S[r + 1]); }
                        else { S[r] = __builtin_fmaf(kv[j][r], bvv[j], av[j] * S[r]); S[r + 1] = __builtin_fmaf(kv[j][r + 1], bvv[j], av[j] * S[r + 1]); }
                        po0 = __builtin_fmaf(S[r], qv[j][r], po0); po1 = __builtin_fmaf(S[r + 1], qv[j][r + 1], po1);
                    }
                }
                outv[tt] = po0 + po1;
            }
        }
        };
        if (nt == TB) walk(std::true_type{}); else walk(std::false_type{});
#pragma unroll
        for (int tt = 0; tt < TB; tt++) {
            float po = outv[tt];
            po += SV_DPPF(po, KR_DPP_XOR1); po += SV_DPPF(po, KR_DPP_XOR2); po += SV_DPPF(po, KR_DPP_HALF_MIRROR); po += SV_DPPF(po, KR_DPP_MIRROR);
            outv[tt] = po;
        }
#pragma unroll
        for (int tt = 0; tt < TB; tt++) outv[tt] += __shfl_xor(outv[tt], 16);
        } else {
        // one token: the lane's rows of q, k and the decays come from LDS (16-byte reads when the lane's rows fill DP), the state stays in registers
        auto token = [&](int tt) -> float {
            const float* qp = qs + tt * dimp + part * pitch; const float* kp = ks + tt * dimp + part * pitch; const float* ap = as + tt * dimp + part * pitch;
            float qv[DP], kv[DP], dv[DP];
            if (dpr == DP) {
#pragma unroll
                for (int r = 0; r < DP; r += 4) {
                    const float4 q4 = *reinterpret_cast<const float4*>(qp + r), k4 = *reinterpret_cast<const float4*>(kp + r);
                    qv[r] = q4.x; qv[r + 1] = q4.y; qv[r + 2] = q4.z; qv[r + 3] = q4.w; kv[r] = k4.x; kv[r + 1] = k4.y; kv[r + 2] = k4.z; kv[r + 3] = k4.w;
                    if constexpr (GLA) { const float4 a4 = *reinterpret_cast<const float4*>(ap + r); dv[r] = a4.x; dv[r + 1] = a4.y; dv[r + 2] = a4.z; dv[r + 3] = a4.w; }
                }
            } else {
#pragma unroll
                for (int r = 0; r < DP; r++) { qv[r] = r < dpr ? qp[r] : 0.0f; kv[r] = r < dpr ? kp[r] : 0.0f; if constexpr (GLA) dv[r] = r < dpr ? ap[r] : 0.0f; }
            }
            float av = 1.0f, bvv = vs[tt * NC + cl];
            if constexpr (SSD) { bvv *= gs[2 * tt]; av = gs[2 * tt + 1]; }
            float po0 = 0.0f, po1 = 0.0f;
#pragma unroll
            for (int r = 0; r < DP; r += 2) {
                if constexpr (GLA) { S[r] = __builtin_fmaf(kv[r], bvv, dv[r] * S[r]); S[r + 1] = __builtin_fmaf(kv[r + 1], bvv, dv[r + 1] * S[r + 1]); }
                else { S[r] = __builtin_fmaf(kv[r], bvv, av * S[r]); S[r + 1] = __builtin_fmaf(kv[r + 1], bvv, av * S[r + 1]); }
                po0 = __builtin_fmaf(S[r], qv[r], po0); po1 = __builtin_fmaf(S[r + 1], qv[r + 1], po1);
            }
            float po = po0 + po1;
            po += SV_DPPF(po, KR_DPP_XOR1); po += SV_DPPF(po, KR_DPP_XOR2); po += SV_DPPF(po, KR_DPP_HALF_MIRROR); po += SV_DPPF(po, KR_DPP_MIRROR);
            return po + __shfl_xor(po, 16);
        };
        if (nt == TB) {
#pragma unroll
            for (int tt = 0; tt < TB; tt++) outv[tt] = token(tt);
        } else {
#pragma unroll
            for (int tt = 0; tt < TB; tt++) outv[tt] = tt < nt ? token(tt) : 0.0f;
        }
        }
        if (more) stash(lds + (b ^ 1) * per, tb + TB);
        // the outputs leave after the registers of the next batch have gone to LDS: the wait for those loads then has no younger store before it
        if (part == 0 && cv) {
            float* op = a.o + (size_t)tb * H * vdim + (size_t)h * vdim + col;
#pragma unroll
            for (int tt = 0; tt < TB; tt++) if (tt < nt) op[(size_t)tt * H * vdim] = outv[tt];
        }
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < DP; r++)
        if (r < dpr && part * dpr + r < dim && cv) Sg[r] = S[r];
}
// State-space mixer -> the block form of the recurrences: its recurrence is a retention whose decay changes from token to token,
// S_t = e^{l_t} S_(t-1) + (dt_t B_t) x_t^T with l_t = -e^{A_h} dt_t, read out by C_t.  One wave per (token, head) writes the head's own rows
// [q = C of its group | k = dt B of its group | v = x] where the block launches expect them and the token's log decay where sv_lin_prep_kernel would.
__global__ void __launch_bounds__(64) sv_ssd_expand_kernel(const KrSvLin a, float* __restrict__ zo, int ldz) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, H = a.heads, N = a.dim, dv = a.vdim, hq = h / a.qk_group;
    const float z = a.dtz[(size_t)t * a.dtz_ld + h] + a.dt_bias[h];
    const float dt = fmaxf(z, 0.0f) + log1pf(expf(-fabsf(z)));      // softplus
    const size_t r = (size_t)t * a.src_ld;
    float* o = zo + (size_t)t * ldz;
    for (int d = lane; d < N; d += 64) {
        o[(size_t)h * N + d] = a.qsrc[r + (size_t)hq * N + d];
        o[(size_t)H * N + (size_t)h * N + d] = a.ksrc[r + (size_t)hq * N + d] * dt;
    }
    for (int c = lane; c < dv; c += 64) o[(size_t)2 * H * N + (size_t)h * dv + c] = a.vsrc[r + (size_t)h * dv + c];
    if (lane == 0) a.tok[(size_t)t * H + h] = make_float4(-expf(a.a_log[h]) * dt, 0.0f, 0.0f, 0.0f);
}
// gla: the decays themselves from their logits, in place: a = sigmoid(z + b)^(1 / tau), formed through the logarithm
__global__ void sv_gla_decay_kernel(float* __restrict__ gz, const float* __restrict__ bias, size_t n, int cols, float inv_tau) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float z = gz[i] + bias[i % cols];
    gz[i] = expf((fminf(z, 0.0f) - log1pf(expf(-fabsf(z)))) * inv_tau);
}

// ---- chunked form for prompt portions (KrSvLin: tok, sbuf, nbuf)
// rotation and scales on q / k in place, and the log gates of every (token, head): tok.x = log decay a, tok.y = log input b
__global__ void __launch_bounds__(64) sv_lin_prep_kernel(const KrSvLin a) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, H = a.heads, dim = a.dim;
    float* q = a.z + (size_t)t * a.ld + (size_t)h * dim; float* k = q + (size_t)H * dim;
    const int half = a.rot_dims / 2;
    for (int i = lane; i < half; i += 64) {
        const float2 c = a.cs[(size_t)t * half + i];
        const float qu = q[i] * a.q_scale, qv = q[i + half] * a.q_scale, ku = k[i] * a.k_scale, kv = k[i + half] * a.k_scale;
        q[i] = qu * c.x - qv * c.y; q[i + half] = qv * c.x + qu * c.y;
        k[i] = ku * c.x - kv * c.y; k[i + half] = kv * c.x + ku * c.y;
    }
    for (int d = a.rot_dims + lane; d < dim; d += 64) { q[d] *= a.q_scale; k[d] *= a.k_scale; }
    if (lane == 0) {
        float la, lb;
        if (a.kind == 3) {
            const float* zg = a.z + (size_t)t * a.ld + (size_t)2 * H * dim + (size_t)2 * H * a.vdim;
            float zi = zg[h] + a.i_bias[h], zf = zg[H + h] + a.f_bias[h];
            if (a.gate_cap > 0.0f) { zi = a.gate_cap * tanhf(zi / a.gate_cap); zf = a.gate_cap * tanhf(zf / a.gate_cap); }
            lb = zi; la = fminf(zf, 0.0f) - log1pf(expf(-fabsf(zf)));
        } else { la = fmaxf(logf(a.decay[h]), -1.0e4f); lb = 0.0f; }
        a.tok[(size_t)t * H + h] = make_float4(la, lb, 0.0f, 0.0f);
    }
}
// The running sum F of the log decays (from each block's start) and the running maximum m, m_t = F_t + max(m_start, max_(s <= t) (b_s - F_s)), in three
// launches: (1) a wave per (block, head) scans F and the prefix maximum of b - F over its 64 lanes, and leaves the block's last values; (2) a thread per
// (entry, head) carries m from block to block, m_next = F_last + max(m, pm_last), and leaves the last m in the slot's state; (3) a wave per (block, head)
// forms what the other launches read per token: (F - m, b - F, exp(F + m_start - m), exp(-m)).  Retention (b = 0, no maximum) is done after (1).
template <bool ML>
__global__ void __launch_bounds__(64) sv_lin_mlocal_kernel(const KrSvLin a) {
    const int gc = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, H = a.heads;
    int e = 0;
    while (e + 1 < a.n_entries && a.ent_chunk0[e + 1] <= gc) e++;
    const int tb = a.ent_off[e] + 64 * (gc - a.ent_chunk0[e]), nt = min(64, a.ent_off[e + 1] - tb);
    const bool ok = lane < nt;
    const size_t ti = (size_t)(tb + lane) * H + h;
    const float4 ab = ok ? a.tok[ti] : make_float4(0.0f, -INFINITY, 0.0f, 0.0f);
    float F = ab.x;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) { const float up = __shfl_up(F, o); if (lane >= o) F += up; }
    if constexpr (!ML) { if (ok) a.tok[ti] = make_float4(F, -F, expf(F), 0.0f); }
    else {
        const float x = ok ? ab.y - F : -INFINITY;
        float pm = x;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { const float up = __shfl_up(pm, o); if (lane >= o) pm = fmaxf(pm, up); }
        if (ok) a.tok[ti] = make_float4(F, x, pm, 0.0f);
        if (lane == nt - 1) { float* cm = a.cmeta + ((size_t)gc * H + h) * 4; cm[0] = F; cm[1] = pm; }
    }
}
__global__ void __launch_bounds__(64) sv_lin_mchain_kernel(const KrSvLin a) {
    const int e = blockIdx.x, h = blockIdx.y * 64 + threadIdx.x, H = a.heads, ncb = (a.vdim + 15) / 16;
    if (h >= H) return;
    const int t0 = a.ent_off[e], nch = (a.ent_off[e + 1] - t0 + 63) / 64;
    float* nmh = a.nm + (size_t)a.ent_slot[e] * a.nm_stride + (size_t)h * ncb * (a.dim + 4);
    float m = a.pos[t0] != 0 ? nmh[a.dim] : 0.0f;
    float* cm = a.cmeta + ((size_t)a.ent_chunk0[e] * H + h) * 4; const size_t step = (size_t)H * 4;
    for (int c0 = 0; c0 < nch; c0 += 8) {                        // eight blocks' values are requested together: the chain itself is a few instructions a block
        float F[8], pm[8];
#pragma unroll
        for (int k = 0; k < 8; k++) { const size_t o = (size_t)min(c0 + k, nch - 1) * step; F[k] = cm[o]; pm[k] = cm[o + 1]; }
#pragma unroll
        for (int k = 0; k < 8; k++) if (c0 + k < nch) { cm[(size_t)(c0 + k) * step + 2] = m; m = F[k] + fmaxf(m, pm[k]); }
    }
    for (int cbk = 0; cbk < ncb; cbk++) nmh[(size_t)cbk * (a.dim + 4) + a.dim] = m;
}
__global__ void __launch_bounds__(64) sv_lin_mfinal_kernel(const KrSvLin a) {
    const int gc = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, H = a.heads;
    int e = 0;
    while (e + 1 < a.n_entries && a.ent_chunk0[e + 1] <= gc) e++;
    const int tb = a.ent_off[e] + 64 * (gc - a.ent_chunk0[e]), nt = min(64, a.ent_off[e + 1] - tb);
    if (lane >= nt) return;
    const size_t ti = (size_t)(tb + lane) * H + h;
    const float m0 = a.cmeta[((size_t)gc * H + h) * 4 + 2];
    const float4 v = a.tok[ti];
    const float m = v.x + fmaxf(m0, v.z);
    a.tok[ti] = make_float4(v.x - m, v.y, expf(v.x + m0 - m), expf(-m));
}
// The state at every block's start, in two launches.  (1) In parallel over the blocks, one wave per (block, head, 16 value columns, NDT tiles of 16 key
// rows): the block's own contribution U = sum_s exp(u_last + w_s) k_s v_s^T on the matrix instruction (row d = 16 tile + 4 (lane / 16) + i, column =
// lane % 16), written where the block's start state will stand; the normaliser's contribution sum_s exp(u_last + w_s) k_s likewise.
template <bool ML, int NDT>
__global__ void __launch_bounds__(64) sv_lin_cupd_kernel(const KrSvLin a) {
    const int gcb = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, r = lane & 15, kq = lane >> 4;
    const int H = a.heads, dim = a.dim, vdim = a.vdim, ncb = (vdim + 15) / 16;
    const int cb = blockIdx.z % ncb, dg = blockIdx.z / ncb;
    int e = 0;
    while (e + 1 < a.n_entries && a.ent_chunk0[e + 1] <= gcb) e++;
    const int tb = a.ent_off[e] + 64 * (gcb - a.ent_chunk0[e]), nt = min(64, a.ent_off[e + 1] - tb);
    const int col = cb * 16 + r; const bool cv = col < vdim;
    const float* zk = a.z + (size_t)H * dim + (size_t)h * dim; const float* zv = a.z + (size_t)2 * H * dim + (size_t)h * vdim;
    const float4 last = a.tok[(size_t)(tb + nt - 1) * H + h];
    float kk[16][NDT], vv[16], ww[16];
#pragma unroll
    for (int j = 0; j < 16; j++) {                                   // every operand of the block is requested before the first product
        const int s = 4 * j + kq; const size_t ts = (size_t)tb + min(s, nt - 1);
        ww[j] = s < nt ? a.tok[ts * H + h].y : -INFINITY;            // tokens past the portion's end weigh nothing
        vv[j] = cv ? zv[ts * a.ld + col] : 0.0f;
#pragma unroll
        for (int x = 0; x < NDT; x++) { const int da = (dg * NDT + x) * 16 + r; kk[j][x] = da < dim ? zk[ts * a.ld + da] : 0.0f; }
    }
    sv_f4 acc[NDT]; float nsum[NDT];
#pragma unroll
    for (int x = 0; x < NDT; x++) { acc[x] = sv_f4{0.0f, 0.0f, 0.0f, 0.0f}; nsum[x] = 0.0f; }
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const float wgt = expf(last.x + ww[j]);
#pragma unroll
        for (int x = 0; x < NDT; x++) {
            const float aval = kk[j][x] * wgt;
            acc[x] = __builtin_amdgcn_mfma_f32_16x16x4f32(aval, vv[j], acc[x], 0, 0, 0);
            nsum[x] += aval;
        }
    }
    const size_t gc = (size_t)gcb * H + h;
#pragma unroll
    for (int x = 0; x < NDT; x++) {
        const int dt = dg * NDT + x;
#pragma unroll
        for (int i = 0; i < 4; i++) { const int d = dt * 16 + 4 * kq + i; if (cv && d < dim) a.sbuf[(gc * dim + d) * vdim + col] = acc[x][i]; }
        if constexpr (ML) {
            float v = nsum[x]; v += __shfl_xor(v, 16); v += __shfl_xor(v, 32);
            const int da = dt * 16 + r;
            if (cb == 0 && kq == 0 && da < dim) a.nbuf[gc * dim + da] = v;
        }
    }
}
// (2) Serial over the blocks of an entry, but element by element: a thread owns one element of S (or, in the last workgroups of a head, of the
// normaliser), walks the entry's blocks, leaves the state at the block's start where the block's contribution stood, and takes S <- g_last S + U.
// The contributions do not depend on the state, so their loads run ahead of the chain.
template <bool ML>
__global__ void __launch_bounds__(256) sv_lin_cscan_kernel(const KrSvLin a) {
    const int e = blockIdx.x, h = blockIdx.y, H = a.heads, dim = a.dim, vdim = a.vdim, ncb = (vdim + 15) / 16;
    const int t0 = a.ent_off[e], t1 = a.ent_off[e + 1], sl = a.ent_slot[e], c0 = a.ent_chunk0[e], nch = (t1 - t0 + 63) / 64;
    const bool fresh = a.pos[t0] == 0;
    const int idx = blockIdx.z * 256 + threadIdx.x;
    const int nS = dim * vdim;
    if (idx < nS) {
        const int d = idx / vdim, col = idx - d * vdim;
        float* Sg = a.state + (size_t)sl * a.state_stride + ((size_t)h * vdim + col) * dim + d;
        float S = fresh ? 0.0f : *Sg;
        float* p = a.sbuf + ((size_t)c0 * H + h) * nS + idx; const size_t step = (size_t)H * nS;
        int c = 0;
        for (; c + 4 <= nch; c += 4) {
            float u[4], g[4];
#pragma unroll
            for (int k = 0; k < 4; k++) { u[k] = p[(size_t)(c + k) * step]; g[k] = a.tok[(size_t)(min(t0 + 64 * (c + k + 1), t1) - 1) * H + h].z; }
#pragma unroll
            for (int k = 0; k < 4; k++) { p[(size_t)(c + k) * step] = S; S = __builtin_fmaf(g[k], S, u[k]); }
        }
        for (; c < nch; c++) {
            const float u = p[(size_t)c * step], g = a.tok[(size_t)(min(t0 + 64 * (c + 1), t1) - 1) * H + h].z;
            p[(size_t)c * step] = S; S = __builtin_fmaf(g, S, u);
        }
        *Sg = S;
    } else if (ML && idx - nS < dim) {
        const int d = idx - nS;
        float* nm = a.nm + (size_t)sl * a.nm_stride + (size_t)h * ncb * (dim + 4);
        float n = fresh ? 0.0f : nm[d];
        float* p = a.nbuf + ((size_t)c0 * H + h) * dim + d; const size_t step = (size_t)H * dim;
        for (int c = 0; c < nch; c++) {
            const float u = p[(size_t)c * step], g = a.tok[(size_t)(min(t0 + 64 * (c + 1), t1) - 1) * H + h].z;
            p[(size_t)c * step] = n; n = __builtin_fmaf(g, n, u);
        }
        for (int cbk = 0; cbk < ncb; cbk++) nm[(size_t)cbk * (dim + 4) + d] = n;      // every block of value columns keeps its own copy
    }
}
// parallel over blocks: a workgroup per (block, head), wave w owns the 16 tokens [16 w, 16 w + 16) of the block.  As in the matrix-instruction attention both
// products are formed transposed: S^T[s][t] = K Q^T (queries of the wave's tokens stay in registers: lane (t = lane % 16, quarter = lane / 16) keeps
// the quarter-th part of q_t), O^T[c][t] += V^T P^T with the weights where the first product left them; the state's share S_start^T q_t goes into the
// same accumulators first.  DQ >= ceil(dim / 4), DB >= ceil(vdim / 16).
template <bool ML, int DB>
__global__ void __launch_bounds__(256) sv_lin_cout_kernel(const KrSvLin a) {
    extern __shared__ __attribute__((aligned(16))) float sl[];      // [32][lds] rows of the block's start state | [4 waves][dq][64] the waves' queries
    const int gc = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, kq = lane >> 4;
    const int H = a.heads, dim = a.dim, vdim = a.vdim, dq = 4 * ((dim + 15) / 16), nct = (vdim + 15) / 16;
    const int lds = ((vdim + 31) / 32) * 32 + 16;                   // rows 16 banks apart: the lanes of two neighbouring rows fall into distinct banks
    float* qs = sl + 32 * lds + (size_t)wave * dq * 64;             // this wave's queries, one word per (step, lane): a register file that loops can index
    int e = 0;
    while (e + 1 < a.n_entries && a.ent_chunk0[e + 1] <= gc) e++;
    const int tb = a.ent_off[e] + 64 * (gc - a.ent_chunk0[e]), nt = min(64, a.ent_off[e + 1] - tb);
    const bool active = wave * 16 < nt;                             // a wave without tokens still helps to stage the state
    const int trow = wave * 16 + r; const bool tv = trow < nt;
    const size_t tg = (size_t)tb + min(trow, nt - 1);
    const float4 me = a.tok[tg * H + h];
    const float* zq = a.z + (size_t)h * dim; const float* zk = zq + (size_t)H * dim; const float* zv = a.z + (size_t)2 * H * dim + (size_t)h * vdim;
    // the reduction index of a matrix instruction is spread over the four 16-lane groups: in step i lane group kq takes the key coordinate
    // d = 16 (i / 4) + 4 kq + i % 4, so that four steps of a lane are 16 contiguous bytes of a key row
    auto dof = [&](int i) { return 16 * (i >> 2) + 4 * kq + (i & 3); };
    const bool kvec = (a.ld & 3) == 0 && (dim & 15) == 0;          // key rows start 16-byte aligned and hold whole pieces
    for (int i = 0; i < dq; i++) { const int d = dof(i); qs[i * 64 + lane] = (active && d < dim) ? zq[tg * a.ld + d] : 0.0f; }
    sv_f4 acc[DB];
#pragma unroll
    for (int c = 0; c < DB; c++) acc[c] = sv_f4{0.0f, 0.0f, 0.0f, 0.0f};
    const float* Sc = a.sbuf + ((size_t)gc * H + h) * dim * vdim;
    const float* nc = a.nbuf + ((size_t)gc * H + h) * dim;
    float den = 0.0f;
    for (int p0 = 0; p0 < dim; p0 += 32) {                          // passes over 32 rows of the state
        const int rows = min(32, dim - p0);
        __syncthreads();
        if ((vdim & 3) == 0) {                                      // 16-byte pieces: sbuf rows and the LDS rows are 16-byte aligned when vdim is a multiple of four
            const int v4 = vdim >> 2;
            for (int idx = tid; idx < rows * v4; idx += 256) {
                const int rr = idx / v4, c4 = idx - rr * v4;
                *reinterpret_cast<float4*>(sl + rr * lds + 4 * c4) = *reinterpret_cast<const float4*>(Sc + (size_t)(p0 + rr) * vdim + 4 * c4);
            }
        } else {
            for (int idx = tid; idx < rows * vdim; idx += 256) { const int rr = idx / vdim, cc = idx - rr * vdim; sl[rr * lds + cc] = Sc[(size_t)(p0 + rr) * vdim + cc]; }
        }
        __syncthreads();
        if (active) {
#pragma unroll 2
            for (int i = 0; i < 8; i++) {
                const int lr = dof(i);                            // row inside the pass (a pass is eight steps = 32 rows)
                const float qi = lr < rows ? qs[(p0 / 4 + i) * 64 + lane] : 0.0f;      // a row past dim meets a zero
                const float* srow = sl + min(lr, rows - 1) * lds + r;
#pragma unroll
                for (int c = 0; c < DB; c++) acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(c * 16 + r < vdim ? srow[c * 16] : 0.0f, qi, acc[c], 0, 0, 0);
                if constexpr (ML) den = __builtin_fmaf(qi, nc[min(p0 + lr, dim - 1)], den);
            }
        }
    }
    if (!active) return;
    if constexpr (ML) { den += __shfl_xor(den, 16); den += __shfl_xor(den, 32); den *= me.z; }
#pragma unroll
    for (int c = 0; c < DB; c++) acc[c] *= me.z;
#pragma nounroll
    for (int stile = 0; stile <= wave; stile++) {
        const float* krow = zk + ((size_t)tb + min(stile * 16 + r, nt - 1)) * a.ld;
        sv_f4 st = sv_f4{0.0f, 0.0f, 0.0f, 0.0f};
        for (int i0 = 0; i0 < dq; i0 += 16) {                    // sixteen key coordinates and queries requested at a time, then their products
            float kf[16], qf[16];
#pragma unroll
            for (int i = 0; i < 16; i++) qf[i] = i0 + i < dq ? qs[(i0 + i) * 64 + lane] : 0.0f;
            if (kvec) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float4 k4 = i0 + 4 * j < dq ? *reinterpret_cast<const float4*>(krow + 16 * (i0 / 4 + j) + 4 * kq) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                    kf[4 * j] = k4.x; kf[4 * j + 1] = k4.y; kf[4 * j + 2] = k4.z; kf[4 * j + 3] = k4.w;
                }
            } else {
#pragma unroll
                for (int i = 0; i < 16; i++) kf[i] = krow[min(dof(i0 + i), dim - 1)];
            }
#pragma unroll
            for (int i = 0; i < 16; i++) st = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[i], qf[i], st, 0, 0, 0);
        }
        float ps = 0.0f;
        size_t srow[4];
#pragma unroll
        for (int i = 0; i < 4; i++) srow[i] = (size_t)tb + min(stile * 16 + 4 * kq + i, nt - 1);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int s = stile * 16 + 4 * kq + i;
            const bool ok = tv && s <= trow;
            const float p = ok ? st[i] * expf(me.x + a.tok[srow[i] * H + h].y) : 0.0f;
            st[i] = p; ps += p;
        }
        if constexpr (ML) { ps += __shfl_xor(ps, 16); ps += __shfl_xor(ps, 32); den += ps; }
        float vf[4][DB];                                          // the value rows of the tile's keys
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int c = 0; c < DB; c++) { const int cc = c * 16 + r; vf[i][c] = cc < vdim ? zv[srow[i] * a.ld + cc] : 0.0f; }
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int c = 0; c < DB; c++) acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[i][c], st[i], acc[c], 0, 0, 0);
    }
    const float inv = ML ? 1.0f / (fmaxf(fabsf(den), me.w) + 1e-6f) : 1.0f;
    if (!tv) return;
    float* o = a.o + tg * H * vdim + (size_t)h * vdim;
#pragma unroll
    for (int c = 0; c < DB; c++) {
        const int c0 = c * 16 + 4 * kq;
        if ((vdim & 3) == 0) { if (c0 < vdim) *reinterpret_cast<float4*>(o + c0) = make_float4(acc[c][0] * inv, acc[c][1] * inv, acc[c][2] * inv, acc[c][3] * inv); }
        else {
#pragma unroll
            for (int i = 0; i < 4; i++) if (c0 + i < vdim) o[c0 + i] = acc[c][i] * inv;
        }
    }
}

// one wave per (token, head): o / rms(o) (* weight) * act(g) -> the output projection's input
template <typename T>
__global__ void __launch_bounds__(64) sv_lin_out_kernel(const KrSvLin a, T* __restrict__ out) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, vdim = a.vdim, H = a.heads;
    const float* o = a.o + ((size_t)t * H + h) * vdim;
    const float* g = a.z + (size_t)t * a.ld + (size_t)2 * H * a.dim + (size_t)H * vdim + (size_t)h * vdim;
    float ss = 0.0f;
    for (int d = lane; d < vdim; d += 64) ss = __builtin_fmaf(o[d], o[d], ss);
    const float inv = 1.0f / sqrtf(sv_wave_sum(ss) / (float)vdim + a.eps);
    for (int d = lane; d < vdim; d += 64) {
        const float gz = g[d], sg = 1.0f / (1.0f + expf(-gz));
        float v = o[d] * inv;
        if (a.norm_w) v *= a.norm_w[a.norm_shared ? (size_t)d : (size_t)h * vdim + d];
        sv_st(out + ((size_t)t * H + h) * vdim + d, v * (a.kind == 3 ? sg : gz * sg));
    }
}

// the selective state-space mixer after its scan (KrSvSsdOut): one workgroup per token, the gated row in LDS
template <typename T>
__global__ void __launch_bounds__(256) sv_ssd_out_kernel(const KrSvSsdOut a, T* __restrict__ out) {
    extern __shared__ float yr[];            // [inner] | [2 * groups]
    const size_t t = blockIdx.x;
    const int inner = a.heads * a.vdim;
    float* gst = yr + inner;
    for (int c = threadIdx.x; c < inner; c += 256) {
        const float xv = a.x[t * a.ld_x + c], zv = a.z[t * a.ld_z + c];
        yr[c] = __builtin_fmaf(a.D[c / a.vdim], xv, a.o[t * inner + c]) * (zv / (1.0f + expf(-zv)));
    }
    __syncthreads();
    sv_group_stats<KR_SV_NORM_RMS, 4>(yr, inner, a.groups, a.eps, gst);
    __syncthreads();
    const int gw = inner / a.groups;
    for (int c = threadIdx.x; c < inner; c += 256) sv_st(out + t * a.out_ld + c, yr[c] * gst[2 * (c / gw) + 1] * a.w[c] * a.scale);
}

__global__ void __launch_bounds__(1024) sv_argmax_kernel(const float* __restrict__ logits, int vocab, int* __restrict__ out) {
    __shared__ float bv[16]; __shared__ int bi[16];
    const float* row = logits + (size_t)blockIdx.x * vocab;
    float v = -INFINITY; int idx = 0x7fffffff;
#pragma unroll 8
    for (int c = threadIdx.x; c < vocab; c += 1024) { const float x = row[c]; if (x > v || (x == v && c < idx)) { v = x; idx = c; } }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o); const int oi = __shfl_xor(idx, o);
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
    if ((threadIdx.x & 63) == 0) { bv[threadIdx.x >> 6] = v; bi[threadIdx.x >> 6] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; w++) if (bv[w] > v || (bv[w] == v && bi[w] < idx)) { v = bv[w]; idx = bi[w]; }
        out[blockIdx.x] = idx == 0x7fffffff ? 0 : idx;
    }
}
template <typename T>
__global__ void sv_fill_uniform_kernel(T* __restrict__ p, size_t n, uint64_t seed, float amp) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint64_t z = seed + 0x9E3779B97F4A7C15ull * (i + 1);      // splitmix64 of the element index
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull; z = (z ^ (z >> 27)) * 0x94D049BB133111EBull; z ^= z >> 31;
    const float u = (float)(z >> 40) * (1.0f / 16777216.0f);  // [0, 1)
    sv_st(p + i, (2.0f * u - 1.0f) * amp);
}
}  // namespace

void kr_sv_fill_uniform(void* p, bool f32, size_t n, uint64_t seed, float amp, hipStream_t st) {
    if (n == 0) return;
    const dim3 grid((unsigned)((n + 255) / 256));
    if (f32) hipLaunchKernelGGL(sv_fill_uniform_kernel<float>, grid, dim3(256), 0, st, (float*)p, n, seed, amp);
    else hipLaunchKernelGGL(sv_fill_uniform_kernel<uint16_t>, grid, dim3(256), 0, st, (uint16_t*)p, n, seed, amp);
}

void kr_sv_embed(const void* table, bool f32, const int* tokens, float* x, void* h_out, int T, int width, float scale, const void* table2, const int* rows2, hipStream_t st) {
    if (T <= 0) return;
    if (f32) hipLaunchKernelGGL(sv_embed_kernel<float>, dim3(T), dim3(256), 0, st, (const float*)table, tokens, x, (float*)h_out, width, scale, (const float*)table2, rows2);
    else hipLaunchKernelGGL(sv_embed_kernel<uint16_t>, dim3(T), dim3(256), 0, st, (const uint16_t*)table, tokens, x, (uint16_t*)h_out, width, scale, (const uint16_t*)table2, rows2);
}

void kr_sv_stream_norm(float* x, const float* add, const float* w, const float* b, bool in_place, void* out, bool out_f32, int T, int width, float eps, int kind, int groups,
                       hipStream_t st) {
    if (T <= 0 || (!add && !w)) return;
    const size_t lds = (size_t)(width + 2 * (groups > 1 ? groups : 0)) * sizeof(float);
#define SV_SN(T_, K_) hipLaunchKernelGGL((sv_stream_norm_kernel<T_, K_>), dim3(T), dim3(256), lds, st, x, add, w, b, (int)in_place, (T_*)out, width, eps, groups)
    if (kind == KR_SV_NORM_LAYER) { if (out_f32) SV_SN(float, KR_SV_NORM_LAYER); else SV_SN(uint16_t, KR_SV_NORM_LAYER); }
    else { if (out_f32) SV_SN(float, KR_SV_NORM_RMS); else SV_SN(uint16_t, KR_SV_NORM_RMS); }
#undef SV_SN
}

void kr_sv_chan_conv(const KrSvChanConv& c, hipStream_t st) {
    if (c.T <= 0 || c.C <= 0) return;
    hipLaunchKernelGGL(sv_chan_conv_kernel, dim3(c.T, (c.C + 255) / 256), dim3(256), 0, st, c);
}
void kr_sv_chan_conv_save(const KrSvChanConv& c, hipStream_t st) {
    if (c.T <= 0 || c.C <= 0 || c.taps < 2 || c.n_entries <= 0) return;
    hipLaunchKernelGGL(sv_chan_conv_save_kernel, dim3(c.n_entries, c.taps - 1, (c.C + 255) / 256), dim3(256), 0, st, c);
}
void kr_sv_scale(float* p, size_t n, float scale, hipStream_t st) {
    if (n == 0) return;
    hipLaunchKernelGGL(sv_scale_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, p, n, scale);
}
void kr_sv_ssd_out(const KrSvSsdOut& a, bool f32, hipStream_t st) {
    if (a.T <= 0) return;
    const size_t lds = (size_t)(a.heads * a.vdim + 2 * a.groups) * sizeof(float);
    if (f32) hipLaunchKernelGGL(sv_ssd_out_kernel<float>, dim3(a.T), dim3(256), lds, st, a, (float*)a.out);
    else hipLaunchKernelGGL(sv_ssd_out_kernel<uint16_t>, dim3(a.T), dim3(256), lds, st, a, (uint16_t*)a.out);
}

void kr_sv_norm(const float* x, const int* rows, const float* w, const float* b, void* out, bool out_f32, int R, int width, float eps, int kind, int groups, float* out32,
                hipStream_t st) {
    if (R <= 0) return;
    const size_t lds = groups > 1 ? (size_t)2 * groups * sizeof(float) : 0;
#define SV_NORM(T_, K_) hipLaunchKernelGGL((sv_norm_kernel<T_, K_>), dim3(R), dim3(256), lds, st, x, rows, w, b, (T_*)out, width, eps, groups, out32)
    if (kind == KR_SV_NORM_LAYER) { if (out_f32) SV_NORM(float, KR_SV_NORM_LAYER); else SV_NORM(uint16_t, KR_SV_NORM_LAYER); }
    else { if (out_f32) SV_NORM(float, KR_SV_NORM_RMS); else SV_NORM(uint16_t, KR_SV_NORM_RMS); }
#undef SV_NORM
}

void kr_sv_rope_table(const int* pos, const double* inv_freq, float2* cs, int T, int half, float mult, hipStream_t st) {
    const int n = T * half;
    if (n <= 0) return;
    hipLaunchKernelGGL(sv_rope_table_kernel, dim3((n + 255) / 256), dim3(256), 0, st, pos, inv_freq, cs, T, half, mult);
}

void kr_sv_qk_rms(const KrSvAttn& a, hipStream_t st) {
    if (a.T <= 0) return;
    hipLaunchKernelGGL(sv_qk_rms_kernel, dim3(a.T, 2), dim3(256), 0, st, a);
}

void kr_sv_canon(const KrSvCanon& c, bool f32, hipStream_t st) {
    if (c.T <= 0) return;
    const dim3 grid(c.T, (c.width + 255) / 256);
    if (f32) hipLaunchKernelGGL(sv_canon_kernel<float>, grid, dim3(256), 0, st, c, (float*)c.out);
    else hipLaunchKernelGGL(sv_canon_kernel<uint16_t>, grid, dim3(256), 0, st, c, (uint16_t*)c.out);
}

void kr_sv_qk_prep(const KrSvAttn& a, bool f32, hipStream_t st) {
    if (a.T <= 0) return;
    const dim3 grid(a.T, a.heads + (a.own_kv ? (a.v_from_k ? 1 : 2) * a.kv_heads : 0));
    const size_t lds = (size_t)a.dim * sizeof(float);
    if (f32) hipLaunchKernelGGL(sv_qk_prep_kernel<float>, grid, dim3(64), lds, st, a);
    else hipLaunchKernelGGL(sv_qk_prep_kernel<uint16_t>, grid, dim3(64), lds, st, a);
}

// the register tilings of the matrix-instruction attention: (dim / 4, vdim / 16)
static bool sv_mfma_tiling(int dq, int db) {
    static const int tab[][2] = {{16, 4}, {32, 8}, {16, 8}, {32, 4}, {8, 2}, {8, 4}, {16, 2}, {64, 16}, {64, 8}, {32, 16}, {8, 16}, {8, 1}, {16, 1},
                                 // latent cache rows: [latent | rotated part] as the key, the latent as the value (512 + 64, 256 + 64, 128 + 64 and the like)
                                 {144, 32}, {80, 16}, {48, 8}};
    for (const auto& t : tab) if (t[0] == dq && t[1] == db) return true;
    return false;
}
static bool sv_mfma_fits(int heads, int kv_heads, int dim, int vdim, int ldk, int ldv, bool f32) {
    const int VEC = f32 ? 4 : 8, R = heads / kv_heads;
    if (!((R <= 16 && 16 % R == 0) || R % 16 == 0)) return false;
    if (dim % (4 * VEC) != 0 || vdim % 16 != 0 || ldk % VEC != 0 || ldv % VEC != 0) return false;
    return sv_mfma_tiling(dim / 4, vdim / 16);
}
// keys a wave takes at a time in a split launch: long rows on the matrix path go 16 at a time (a wave's loads of one 64-key block are ~40 dependent
// batches at one wave per SIMD: a decode step is over sooner with four times the waves), everything else 64
static int sv_split_key_block(int heads, int kv_heads, int dim, int vdim, int ldk, int ldv, bool f32) {
    return (dim >= 192 && sv_mfma_fits(heads, kv_heads, dim, vdim, ldk, ldv, f32)) ? 16 : 64;
}

int kr_sv_attention_splits(int T, int heads, int kv_heads, int dim, int vdim, int ldk, int ldv, bool f32, int max_visible) {
    const int R = heads / kv_heads;
    const int vc = vdim <= 64 ? 1 : vdim <= 128 ? 2 : vdim <= 256 ? 4 : 8;
    const int rmax = vc <= 2 ? 16 : vc == 4 ? 8 : 4;
    int rm = 2;
    while (rm < R && rm < rmax) rm *= 2;
    const long blocks = (long)T * kv_heads * ((R + rm - 1) / rm);
    const int kblk = sv_split_key_block(heads, kv_heads, dim, vdim, ldk, ldv, f32);
    const int nch = (max_visible + kblk - 1) / kblk;
    long ns = 1024 / (blocks > 0 ? blocks : 1);              // about four workgroups per compute unit
    if (ns > (nch + 3) / 4) ns = (nch + 3) / 4;              // a workgroup keeps at least one block of keys per wave
    return ns < 1 ? 1 : (int)ns;
}

// the matrix-instruction form takes prompt-sized steps whose head sizes fit its register tiling
template <typename T>
static bool sv_attn_mfma_launch(const KrSvAttn& a, hipStream_t st) {
    if (!sv_mfma_fits(a.heads, a.kv_heads, a.dim, a.vdim, a.ldk, a.ldv, sizeof(T) == 4)) return false;
    const int R = a.heads / a.kv_heads;
    const int Rb = R < 16 ? R : 16;
    KrSvAttn b = a;
    b.tq = a.nsplit > 1 ? 1 : 16 / Rb;      // a split launch is a decode-shaped step: its tokens belong to different requests
    const dim3 grid((a.T + b.tq - 1) / b.tq, a.kv_heads, (R <= 16 ? 1 : R / 16) * a.nsplit);
    const size_t lds = (size_t)(4 * 16 * 2 + 16 * 2 + 16 * (a.vdim + 65)) * sizeof(float);
#define SV_MF(DQ_, DB_) do { hipLaunchKernelGGL((sv_attn_mfma_kernel<T, DQ_, DB_>), grid, dim3(256), lds, st, b); return true; } while (0)
#define SV_MF1(DQ_, DB_) do { if (a.nsplit > 1) hipLaunchKernelGGL((sv_attn_mfma_kernel<T, DQ_, DB_, 1>), grid, dim3(256), lds, st, b); \
                              else hipLaunchKernelGGL((sv_attn_mfma_kernel<T, DQ_, DB_>), grid, dim3(256), lds, st, b); return true; } while (0)
    const int dq = a.dim / 4, db = a.vdim / 16;
    if (dq == 16 && db == 4) SV_MF(16, 4);
    if (dq == 32 && db == 8) SV_MF(32, 8);
    if (dq == 16 && db == 8) SV_MF(16, 8);
    if (dq == 32 && db == 4) SV_MF(32, 4);
    if (dq == 8 && db == 2) SV_MF(8, 2);
    if (dq == 8 && db == 4) SV_MF(8, 4);
    if (dq == 16 && db == 2) SV_MF(16, 2);
    if (dq == 64 && db == 16) SV_MF(64, 16);
    if (dq == 64 && db == 8) SV_MF(64, 8);
    if (dq == 32 && db == 16) SV_MF(32, 16);
    if (dq == 8 && db == 16) SV_MF(8, 16);
    if (dq == 8 && db == 1) SV_MF(8, 1);
    if (dq == 16 && db == 1) SV_MF(16, 1);
    if (dq == 144 && db == 32) SV_MF1(144, 32);     // split launches of the long rows: 16 keys per wave at a time (sv_split_key_block)
    if (dq == 80 && db == 16) SV_MF1(80, 16);
    if (dq == 48 && db == 8) SV_MF1(48, 8);
#undef SV_MF
#undef SV_MF1
    return false;
}

void kr_sv_attention(const KrSvAttn& a, bool f32, hipStream_t st) {
    if (a.T <= 0) return;
    if (f32 ? sv_attn_mfma_launch<float>(a, st) : sv_attn_mfma_launch<uint16_t>(a, st)) {
        if (a.nsplit > 1) {
            if (f32) hipLaunchKernelGGL(sv_attn_merge_kernel<float>, dim3(a.T, a.heads), dim3(256), (size_t)(a.nsplit + 1) * sizeof(float), st, a);
            else hipLaunchKernelGGL(sv_attn_merge_kernel<uint16_t>, dim3(a.T, a.heads), dim3(256), (size_t)(a.nsplit + 1) * sizeof(float), st, a);
        }
        return;
    }
    const int R = a.heads / a.kv_heads;
    const int vc = a.vdim <= 64 ? 1 : a.vdim <= 128 ? 2 : a.vdim <= 256 ? 4 : 8;
    const int rmax = vc <= 2 ? 16 : vc == 4 ? 8 : 4;       // RM * VC accumulators per lane stay within 32
    int rm = 2;
    while (rm < R && rm < rmax) rm *= 2;
    const dim3 grid(a.T, a.kv_heads, ((R + rm - 1) / rm) * a.nsplit);
    const size_t lds = ((size_t)rm * a.dim + 4 * 64 * rm + 8 * rm + (size_t)rm * a.vdim) * sizeof(float);
#define SV_ATT(T_, RM_, VC_) hipLaunchKernelGGL((sv_attn_group_kernel<T_, RM_, VC_>), grid, dim3(256), lds, st, a)
#define SV_ATT_R(T_, VC_) do { if (rm == 2) SV_ATT(T_, 2, VC_); else if (rm == 4) SV_ATT(T_, 4, VC_); else if (rm == 8) SV_ATT(T_, 8, VC_); else SV_ATT(T_, 16, VC_); } while (0)
#define SV_ATT_T(T_) do { if (vc == 1) SV_ATT_R(T_, 1); else if (vc == 2) SV_ATT_R(T_, 2); else if (vc == 4) { if (rm == 2) SV_ATT(T_, 2, 4); else if (rm == 4) SV_ATT(T_, 4, 4); else SV_ATT(T_, 8, 4); } \
                          else { if (rm == 2) SV_ATT(T_, 2, 8); else SV_ATT(T_, 4, 8); } } while (0)
    if (f32) SV_ATT_T(float); else SV_ATT_T(uint16_t);
    if (a.nsplit > 1) {
        if (f32) hipLaunchKernelGGL(sv_attn_merge_kernel<float>, dim3(a.T, a.heads), dim3(256), (size_t)(a.nsplit + 1) * sizeof(float), st, a);
        else hipLaunchKernelGGL(sv_attn_merge_kernel<uint16_t>, dim3(a.T, a.heads), dim3(256), (size_t)(a.nsplit + 1) * sizeof(float), st, a);
    }
#undef SV_ATT_T
#undef SV_ATT_R
#undef SV_ATT
}

void kr_sv_router_select(const float* z, int ld, int parts, const float* bias, int bias_mode, int score_kind, int group_kind, int T, int E, int top, int groups, int keep,
                         int renorm, int* ids, float* wts, hipStream_t st) {
    if (T <= 0) return;
    const size_t lds = (size_t)(2 * E + 2 * groups) * sizeof(float);
    hipLaunchKernelGGL(sv_router_select_kernel, dim3(T), dim3(64), lds, st, z, ld, parts, bias, bias_mode, score_kind, group_kind, E, top, groups, keep, renorm, ids, wts);
}

void kr_sv_moe_sort(const int* ids, int T, int top, int E, int* counts, int* seg, int* cursor, int* src_row, int* row_group, int* pair_pos, hipStream_t st) {
    const int n = T * top;
    if (n <= 0) return;
    if (n <= 1024 && E <= 4096) {
        hipLaunchKernelGGL(sv_moe_sort_small_kernel, dim3(1), dim3(256), (size_t)2 * E * sizeof(int), st, ids, n, top, E, seg, src_row, row_group, pair_pos);
        return;
    }
    hipLaunchKernelGGL(sv_fill_int_kernel, dim3((E + 255) / 256), dim3(256), 0, st, counts, E, 0);
    hipLaunchKernelGGL(sv_moe_count_kernel, dim3((n + 255) / 256), dim3(256), 0, st, ids, n, counts);
    hipLaunchKernelGGL(sv_moe_scan_kernel, dim3(1), dim3(64), 0, st, counts, E, seg, cursor);
    hipLaunchKernelGGL(sv_moe_fill_kernel, dim3((n + 255) / 256), dim3(256), 0, st, ids, n, top, seg, cursor, src_row, row_group, pair_pos);
}

void kr_sv_act(const float* gu, int ld, void* y, bool f32, int M, int F, int kind, float limit, float alpha, hipStream_t st) {
    const size_t n = (size_t)M * F;
    if (n == 0) return;
    const dim3 grid((unsigned)((n + 255) / 256));
    if (f32) hipLaunchKernelGGL(sv_act_kernel<float>, grid, dim3(256), 0, st, gu, ld, (float*)y, M, F, kind, limit, alpha);
    else hipLaunchKernelGGL(sv_act_kernel<uint16_t>, grid, dim3(256), 0, st, gu, ld, (uint16_t*)y, M, F, kind, limit, alpha);
}

void kr_sv_residual_norm(const KrSvResidual& r, bool out_f32, hipStream_t st) {
    if (r.T <= 0) return;
    const size_t lds = (size_t)(r.width + 2 * (r.groups > 1 ? r.groups : 0)) * sizeof(float);
#define SV_RN(T_, K_) do { if (r.T <= 64) hipLaunchKernelGGL((sv_residual_norm_kernel<T_, K_, 1024>), dim3(r.T), dim3(1024), lds, st, r, (T_*)r.h_out); \
                        else hipLaunchKernelGGL((sv_residual_norm_kernel<T_, K_, 256>), dim3(r.T), dim3(256), lds, st, r, (T_*)r.h_out); } while (0)
    if (r.kind == KR_SV_NORM_LAYER) { if (out_f32) SV_RN(float, KR_SV_NORM_LAYER); else SV_RN(uint16_t, KR_SV_NORM_LAYER); }
    else { if (out_f32) SV_RN(float, KR_SV_NORM_RMS); else SV_RN(uint16_t, KR_SV_NORM_RMS); }
#undef SV_RN
}

void kr_sv_latent_prep(const KrSvLatent& a, bool f32, hipStream_t st) {
    if (a.T <= 0) return;
    if (f32) hipLaunchKernelGGL(sv_latent_prep_kernel<float>, dim3(a.T, 2), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(sv_latent_prep_kernel<uint16_t>, dim3(a.T, 2), dim3(256), 0, st, a);
}
void kr_sv_latent_q(const KrSvLatent& a, const float* q2, void* qn, float* qe, bool f32, hipStream_t st) {
    if (a.T <= 0) return;
    if (f32) hipLaunchKernelGGL(sv_latent_q_kernel<float>, dim3(a.T, a.heads), dim3(64), 0, st, a, q2, (float*)qn, qe);
    else hipLaunchKernelGGL(sv_latent_q_kernel<uint16_t>, dim3(a.T, a.heads), dim3(64), 0, st, a, q2, (uint16_t*)qn, qe);
}
void kr_sv_head_rows(int T, int heads, int* seg, int* rows, int* group, hipStream_t st) {
    const int n = T * heads > heads + 1 ? T * heads : heads + 1;
    if (T <= 0) return;
    hipLaunchKernelGGL(sv_head_rows_kernel, dim3((n + 255) / 256), dim3(256), 0, st, T, heads, seg, rows, group);
}

void kr_sv_lin_scan(const KrSvLin& a, hipStream_t st) {
    if (a.T <= 0 || a.n_entries <= 0) return;
    const int dpr = (a.dim + 3) / 4;
    const dim3 grid(a.n_entries, a.heads, (a.vdim + 15) / 16);
    const size_t lds = (size_t)((a.kind == 4 ? 3 : 2) * 8 * 4 * dpr + 8 * 16 + 8 * 2) * sizeof(float);
#define SV_LIN(K_, DP_) hipLaunchKernelGGL((sv_lin_scan_kernel<K_, DP_>), grid, dim3(64), lds, st, a)
#define SV_LIN_D(K_) do { if (dpr <= 8) SV_LIN(K_, 8); else if (dpr <= 16) SV_LIN(K_, 16); else if (dpr <= 32) SV_LIN(K_, 32); else if (dpr <= 64) SV_LIN(K_, 64); else SV_LIN(K_, 128); } while (0)
    if (a.kind == 3) SV_LIN_D(3); else if (a.kind == 4) SV_LIN_D(4); else if (a.kind == 5) SV_LIN_D(5); else SV_LIN_D(2);
#undef SV_LIN_D
#undef SV_LIN
}
// the workgroup form for prompt portions of kinds 4 and 5; false: the shape does not fit its LDS buffers (the caller takes kr_sv_lin_scan)
static size_t sv_scanw_lds(int kind, int dim) {
    const int dpr = (dim + 31) / 32, dimp = 32 * ((dpr % 8 == 0) ? dpr + 4 : dpr);
    return (size_t)2 * ((kind == 4 ? 3 : 2) * 16 * dimp + 16 * 8 + 16 * 2) * sizeof(float);
}
bool kr_sv_lin_scan_wide_fits(int kind, int dim) { return (kind == 4 || kind == 5) && dim <= 512 && sv_scanw_lds(kind, dim) <= 150 * 1024; }
void kr_sv_lin_scan_wide(const KrSvLin& a, hipStream_t st) {
    if (a.T <= 0 || a.n_entries <= 0) return;
    const int dpr = (a.dim + 31) / 32;
    const dim3 grid(a.n_entries, a.heads, (a.vdim + 7) / 8);
    const size_t lds = sv_scanw_lds(a.kind, a.dim);
    if (a.kind == 4) {
        const size_t n = (size_t)a.T * a.heads * a.dim;
        hipLaunchKernelGGL(sv_gla_decay_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, const_cast<float*>(a.gz), a.gz_bias, n, a.heads * a.dim, a.inv_tau);
    }
    // one workgroup per compute unit or fewer: the pipelined walk; more: the plain one (256 compute units, up to three workgroups on each)
    const bool pipe = (size_t)grid.x * grid.y * grid.z <= 384;
#define SV_LW(K_, DP_, P_) do { if (lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)sv_lin_scanw_kernel<K_, DP_, P_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
                                hipLaunchKernelGGL((sv_lin_scanw_kernel<K_, DP_, P_>), grid, dim3(256), lds, st, a); } while (0)
#define SV_LW_P(K_, DP_) do { if (pipe) SV_LW(K_, DP_, true); else SV_LW(K_, DP_, false); } while (0)
#define SV_LW_D(K_) do { if (dpr <= 4) SV_LW_P(K_, 4); else if (dpr <= 8) SV_LW_P(K_, 8); else SV_LW_P(K_, 16); } while (0)
    if (a.kind == 4) SV_LW_D(4); else SV_LW_D(5);
#undef SV_LW_D
#undef SV_LW_P
#undef SV_LW
}
bool kr_sv_lin_chunked_fits(int dim, int vdim) { return dim <= 128 && vdim <= 128; }
void kr_sv_ssd_expand(const KrSvLin& a, float* z_out, int ldz, hipStream_t st) {
    if (a.T <= 0) return;
    hipLaunchKernelGGL(sv_ssd_expand_kernel, dim3(a.T, a.heads), dim3(64), 0, st, a, z_out, ldz);
}
void kr_sv_lin_chunked(const KrSvLin& a, hipStream_t st) {
    if (a.T <= 0 || a.n_entries <= 0 || a.n_chunks <= 0) return;
    const bool ml = a.kind == 3;
    const int ncb = (a.vdim + 15) / 16, ndt = (a.dim + 15) / 16, ndg = (ndt + 1) / 2;
    if (!a.prepped) hipLaunchKernelGGL(sv_lin_prep_kernel, dim3(a.T, a.heads), dim3(64), 0, st, a);
    if (ml) {
        hipLaunchKernelGGL(sv_lin_mlocal_kernel<true>, dim3(a.n_chunks, a.heads), dim3(64), 0, st, a);
        hipLaunchKernelGGL(sv_lin_mchain_kernel, dim3(a.n_entries, (a.heads + 63) / 64), dim3(64), 0, st, a);
        hipLaunchKernelGGL(sv_lin_mfinal_kernel, dim3(a.n_chunks, a.heads), dim3(64), 0, st, a);
    } else hipLaunchKernelGGL(sv_lin_mlocal_kernel<false>, dim3(a.n_chunks, a.heads), dim3(64), 0, st, a);
    const dim3 gu(a.n_chunks, a.heads, ncb * ndg);
    if (ml) hipLaunchKernelGGL((sv_lin_cupd_kernel<true, 2>), gu, dim3(64), 0, st, a);
    else hipLaunchKernelGGL((sv_lin_cupd_kernel<false, 2>), gu, dim3(64), 0, st, a);
    const dim3 gs(a.n_entries, a.heads, (a.dim * a.vdim + (ml ? a.dim : 0) + 255) / 256);
    if (ml) hipLaunchKernelGGL(sv_lin_cscan_kernel<true>, gs, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(sv_lin_cscan_kernel<false>, gs, dim3(256), 0, st, a);
    const dim3 go(a.n_chunks, a.heads);
    const bool small = a.dim <= 64 && a.vdim <= 64;
    const size_t lds = ((size_t)32 * (((a.vdim + 31) / 32) * 32 + 16) + (size_t)4 * (4 * ((a.dim + 15) / 16)) * 64) * sizeof(float);
#define SV_CO(ML_) do { if (small) hipLaunchKernelGGL((sv_lin_cout_kernel<ML_, 4>), go, dim3(256), lds, st, a); \
                        else hipLaunchKernelGGL((sv_lin_cout_kernel<ML_, 8>), go, dim3(256), lds, st, a); } while (0)
    if (ml) SV_CO(true); else SV_CO(false);
#undef SV_CO
}
void kr_sv_lin_out(const KrSvLin& a, bool f32, hipStream_t st) {
    if (a.T <= 0) return;
    if (f32) hipLaunchKernelGGL(sv_lin_out_kernel<float>, dim3(a.T, a.heads), dim3(64), 0, st, a, (float*)a.out);
    else hipLaunchKernelGGL(sv_lin_out_kernel<uint16_t>, dim3(a.T, a.heads), dim3(64), 0, st, a, (uint16_t*)a.out);
}

void kr_sv_argmax(const float* logits, int R, int vocab, int* out, hipStream_t st) {
    if (R <= 0) return;
    hipLaunchKernelGGL(sv_argmax_kernel, dim3(R), dim3(1024), 0, st, logits, vocab, out);
}

#ifdef KR_SV_STAMPS
extern "C" int kr_sv_read_stamps(long long* out16) { return hipMemcpyFromSymbol(out16, HIP_SYMBOL(sv_stamps), sizeof(long long) * 16) != hipSuccess; }
#endif
