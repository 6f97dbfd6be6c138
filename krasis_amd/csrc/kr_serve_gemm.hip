// kr_serve_gemm.hip -- C[M, N] (f32) = A[M, K] x W[N, K]^T for the batched serving step, single matrix or grouped (one matrix per expert, the rows
// of a group contiguous, optional row gather for A).  Three forms:
//   * small M (decode steps): one WAVE per output column, the K range over its lanes in 16-byte reads, up to 8 rows of A against one pass over
//     the weight row -- bound by the weight stream;
//   * bf16, larger M: workgroup tile 128 x 128 x 64 staged through LDS, four waves of 64 x 64 on v_mfma_f32_32x32x16_bf16, f32 accumulators, the next
//     tile's global loads in flight during the MFMAs;
//   * f32, larger M: 64 x 64 x 16 tile, 4 x 4 outputs per thread, plain fused multiply-adds (no reduced-precision matrix mode).
// Every shape is accepted: edges are guarded, and rows whose byte length is not a multiple of 16 take element loads.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kr_device.h"
#include "kr_serve_ops.h"

namespace {
typedef float gv16f __attribute__((ext_vector_type(16)));
typedef __bf16 gb8 __attribute__((ext_vector_type(8)));
typedef uint32_t gu4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float gm_ld(const float* p) { return *p; }
__device__ __forceinline__ float gm_ld(const uint16_t* p) { return kr_bf16_to_f32(*p); }
// one element of C: f32, or the storage type when the output feeds another GEMM as it is (BF = a bf16 store)
template <bool BF>
__device__ __forceinline__ void gm_store(const KrSvGemm& g, int m, int n, float v) {
    const size_t i = (size_t)(g.c_rows ? g.c_rows[m] : m) * g.ldc + n;
    if (BF && g.c_storage) ((uint16_t*)g.C)[i] = kr_f32_to_bf16(v);
    else g.C[i] = v;
}

// row tile `tile` of a grouped problem: walks the segment table; returns false past the last tile
__device__ __forceinline__ bool gm_find_tile(const int* seg, int n_groups, int tile, int BM, int& group, int& m0, int& mend) {
    int acc = 0;
    for (int g = 0; g < n_groups; g++) {
        const int lo = seg[g], hi = seg[g + 1];
        const int nt = (hi - lo + BM - 1) / BM;
        if (tile < acc + nt) { group = g; m0 = lo + (tile - acc) * BM; mend = hi; return true; }
        acc += nt;
    }
    return false;
}

// ---------------------------------------------------------------------------------------------------------------- small M
__device__ __forceinline__ float gm_act(float g, float u, int kind, float limit, float alpha) {
    if (kind == KR_SV_ACT_RELU2) { g = fmaxf(g, 0.0f); return g * g; }
    if (kind == KR_SV_ACT_GELU_TANH) return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
    if (kind == KR_SV_ACT_CLAMPED_SWIGLU) { g = fminf(g, limit); u = fminf(fmaxf(u, -limit), limit); return g / (1.0f + expf(-alpha * g)) * (u + 1.0f); }
    return g / (1.0f + expf(-g)) * u;
}
template <typename T> __device__ __forceinline__ float gm_round(float v) { return v; }
template <> __device__ __forceinline__ float gm_round<uint16_t>(float v) { return kr_bf16_to_f32(kr_f32_to_bf16(v)); }

// ACT: the A operand is the gated activation of g.act_gu, formed as it is needed.  A wave owns CN consecutive output columns: their weight rows are
// requested together (CN 16-byte reads in flight per k step), the input rows are read once for all of them.
template <typename T, int MB, int CN, bool ACT>
__global__ void __launch_bounds__(256) sv_gemv_kernel(const KrSvGemm g, int mbase) {
    constexpr int VEC = 16 / sizeof(T);
    const int lane = threadIdx.x & 63, n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * CN;
    if (n0 >= g.N) return;
    int m0 = mbase, mcnt;
    const T* W = (const T*)g.W;
    if (g.row_group) { m0 = blockIdx.y; mcnt = 1; W += (size_t)g.row_group[m0] * g.w_stride; }
    else mcnt = min(MB, g.M - m0);
    const T* wr[CN];
#pragma unroll
    for (int c = 0; c < CN; c++) wr[c] = W + (size_t)min(n0 + c, g.N - 1) * g.K;       // columns past N repeat the last one and are not stored
    const T* ar[MB]; const float* gr[MB];
#pragma unroll
    for (int m = 0; m < MB; m++) {
        const int r = min(m0 + m, g.M - 1);
        const int src = g.a_rows ? g.a_rows[r] : r;
        ar[m] = ACT ? nullptr : (const T*)g.A + (size_t)src * g.lda;
        gr[m] = ACT ? g.act_gu + (size_t)src * g.act_ld : nullptr;
    }
    const int uoff = g.act_kind == KR_SV_ACT_RELU2 ? 0 : g.K;     // an un-gated activation has no up columns: the second read repeats the first
    float acc[MB][CN];
#pragma unroll
    for (int m = 0; m < MB; m++)
#pragma unroll
        for (int c = 0; c < CN; c++) acc[m][c] = 0.0f;
    const bool vec = ACT ? (g.K % VEC == 0) && (g.act_ld % 4 == 0) && (g.K % 4 == 0) && ((uintptr_t)g.act_gu % 16 == 0) && ((uintptr_t)g.W % 16 == 0) && (g.w_stride % VEC == 0)
                         : (g.K % VEC == 0) && (g.lda % VEC == 0) && (((uintptr_t)g.A | (uintptr_t)g.W) % 16 == 0) && (g.w_stride % VEC == 0);
    if (vec) {
        for (int k = lane * VEC; k < g.K; k += 64 * VEC) {
            gu4 wv[CN];
#pragma unroll
            for (int c = 0; c < CN; c++) wv[c] = *reinterpret_cast<const gu4*>(wr[c] + k);
#pragma unroll
            for (int m = 0; m < MB; m++) {
                if (m < mcnt) {
                    float af[VEC];
                    if constexpr (ACT) {
#pragma unroll
                        for (int q = 0; q < VEC / 4; q++) {
                            const float4 gg = *reinterpret_cast<const float4*>(gr[m] + k + 4 * q), uu = *reinterpret_cast<const float4*>(gr[m] + uoff + k + 4 * q);
                            af[4 * q] = gm_round<T>(gm_act(gg.x, uu.x, g.act_kind, g.act_limit, g.act_alpha)); af[4 * q + 1] = gm_round<T>(gm_act(gg.y, uu.y, g.act_kind, g.act_limit, g.act_alpha));
                            af[4 * q + 2] = gm_round<T>(gm_act(gg.z, uu.z, g.act_kind, g.act_limit, g.act_alpha)); af[4 * q + 3] = gm_round<T>(gm_act(gg.w, uu.w, g.act_kind, g.act_limit, g.act_alpha));
                        }
                    } else {
                        const gu4 av = *reinterpret_cast<const gu4*>(ar[m] + k);
                        if constexpr (sizeof(T) == 2) {
#pragma unroll
                            for (int i = 0; i < 4; i++) { af[2 * i] = __uint_as_float(av[i] << 16); af[2 * i + 1] = __uint_as_float(av[i] & 0xFFFF0000u); }
                        } else {
#pragma unroll
                            for (int i = 0; i < 4; i++) af[i] = __uint_as_float(av[i]);
                        }
                    }
#pragma unroll
                    for (int c = 0; c < CN; c++) {
                        if constexpr (sizeof(T) == 2) {
#pragma unroll
                            for (int i = 0; i < 4; i++) {
                                acc[m][c] = __builtin_fmaf(af[2 * i], __uint_as_float(wv[c][i] << 16), acc[m][c]);
                                acc[m][c] = __builtin_fmaf(af[2 * i + 1], __uint_as_float(wv[c][i] & 0xFFFF0000u), acc[m][c]);
                            }
                        } else {
#pragma unroll
                            for (int i = 0; i < 4; i++) acc[m][c] = __builtin_fmaf(af[i], __uint_as_float(wv[c][i]), acc[m][c]);
                        }
                    }
                }
            }
        }
    } else {
        for (int k = lane; k < g.K; k += 64) {
            float w[CN];
#pragma unroll
            for (int c = 0; c < CN; c++) w[c] = gm_ld(wr[c] + k);
#pragma unroll
            for (int m = 0; m < MB; m++) {
                if (m < mcnt) {
                    float av;
                    if constexpr (ACT) av = gm_round<T>(gm_act(gr[m][k], gr[m][uoff + k], g.act_kind, g.act_limit, g.act_alpha));
                    else av = gm_ld(ar[m] + k);
#pragma unroll
                    for (int c = 0; c < CN; c++) acc[m][c] = __builtin_fmaf(av, w[c], acc[m][c]);
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MB; m++)
#pragma unroll
        for (int c = 0; c < CN; c++) {
            float v = acc[m][c];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
            if (lane == 0 && m < mcnt && n0 + c < g.N) gm_store<sizeof(T) == 2>(g, m0 + m, n0 + c, v);
        }
}

// ---------------------------------------------------------------------------------------------------------------- f32 tiles
__global__ void __launch_bounds__(256) sv_gemm_f32_kernel(const KrSvGemm g) {
    constexpr int BM = 64, BN = 64, BK = 16;
    __shared__ float As[BK][BM + 4], Bs[BK][BN + 4];
    int group = 0, m0 = blockIdx.y * BM, mend = g.M;
    if (g.seg && !gm_find_tile(g.seg, g.n_groups, blockIdx.y, BM, group, m0, mend)) return;
    const int n0 = blockIdx.x * BN;
    const float* A = (const float*)g.A;
    const float* W = (const float*)g.W + (size_t)group * g.w_stride;
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    // loader: thread -> (row = tid / 4, four k = (tid % 4) * 4 ..)
    const int lr = tid >> 2, lk = (tid & 3) * 4;
    const int am = m0 + lr;
    const float* arow = am < mend ? A + (size_t)(g.a_rows ? g.a_rows[am] : am) * g.lda : nullptr;
    const float* wrow = n0 + lr < g.N ? W + (size_t)(n0 + lr) * g.K : nullptr;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = 0.0f;
    for (int k0 = 0; k0 < g.K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int k = k0 + lk + i;
            As[lk + i][lr] = (arow && k < g.K) ? arow[k] : 0.0f;
            Bs[lk + i][lr] = (wrow && k < g.K) ? wrow[k] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; k++) {
            const float4 a = *reinterpret_cast<const float4*>(&As[k][ty * 4]);
            const float4 b = *reinterpret_cast<const float4*>(&Bs[k][tx * 4]);
            const float av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int m = m0 + ty * 4 + i;
        if (m >= mend) continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int n = n0 + tx * 4 + j;
            if (n < g.N) gm_store<false>(g, m, n, acc[i][j]);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------- bf16 tiles on the matrix cores
#define GM_BK 64             // k depth of an LDS tile
#define GM_KCH (GM_BK / 8)    // 16-byte chunks per tile row
#define GM_LD (GM_BK + 8)    // LDS row: GM_BK bf16 + 8 pad (an odd number of 16-byte units: fragment reads of consecutive rows fall into distinct bank groups)
template <int BM>            // 128 or 64 rows per workgroup; waves 2 x 2, each (BM / 2) x 64
__global__ void __launch_bounds__(256) sv_gemm_bf16_kernel(const KrSvGemm g) {
    constexpr int BN = 128, BK = GM_BK, MBW = BM / 64;   // 32-row blocks per wave
    constexpr int ACH = BM * GM_KCH / 256, BCH = BN * GM_KCH / 256;      // 16-byte chunks of the A / B tile per thread
    __shared__ __attribute__((aligned(16))) uint16_t As[BM * GM_LD];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[BN * GM_LD];
    int group = 0, m0 = blockIdx.y * BM, mend = g.M;
    if (g.seg && !gm_find_tile(g.seg, g.n_groups, blockIdx.y, BM, group, m0, mend)) return;
    const int n0 = blockIdx.x * BN;
    const uint16_t* A = (const uint16_t*)g.A;
    const uint16_t* W = (const uint16_t*)g.W + (size_t)group * g.w_stride;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, h = lane >> 5;
    const int wr = wave >> 1, wc = wave & 1;
    const bool vec = (g.K % 8 == 0) && (g.lda % 8 == 0) && (((uintptr_t)g.A | (uintptr_t)g.W) % 16 == 0) && (g.w_stride % 8 == 0);
    const uint16_t* ap[ACH]; const uint16_t* bp[BCH];
    int akc[ACH], bkc[BCH];
#pragma unroll
    for (int i = 0; i < ACH; i++) {
        const int c = tid + i * 256, row = c / GM_KCH;
        akc[i] = (c % GM_KCH) * 8;
        const int m = m0 + row;
        ap[i] = m < mend ? A + (size_t)(g.a_rows ? g.a_rows[m] : m) * g.lda : nullptr;
    }
#pragma unroll
    for (int i = 0; i < BCH; i++) {
        const int c = tid + i * 256, row = c / GM_KCH;
        bkc[i] = (c % GM_KCH) * 8;
        bp[i] = n0 + row < g.N ? W + (size_t)(n0 + row) * g.K : nullptr;
    }
    auto load16 = [&](const uint16_t* p, int k) -> gu4 {
        gu4 v = {0u, 0u, 0u, 0u};
        if (!p) return v;
        if (vec) { if (k < g.K) v = *reinterpret_cast<const gu4*>(p + k); return v; }
#pragma unroll
        for (int i = 0; i < 8; i++) if (k + i < g.K) v[i >> 1] |= (uint32_t)p[k + i] << (16 * (i & 1));
        return v;
    };
    gv16f acc[MBW][2];
#pragma unroll
    for (int a = 0; a < MBW; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[a][b][i] = 0.0f;
    gu4 ra[ACH], rb[BCH];
#pragma unroll
    for (int i = 0; i < ACH; i++) ra[i] = load16(ap[i], akc[i]);
#pragma unroll
    for (int i = 0; i < BCH; i++) rb[i] = load16(bp[i], bkc[i]);
    for (int k0 = 0; k0 < g.K; k0 += BK) {
        __syncthreads();                                 // the previous tile's fragment reads are done
#pragma unroll
        for (int i = 0; i < ACH; i++) { const int c = tid + i * 256; *reinterpret_cast<gu4*>(&As[(c / GM_KCH) * GM_LD + akc[i]]) = ra[i]; }
#pragma unroll
        for (int i = 0; i < BCH; i++) { const int c = tid + i * 256; *reinterpret_cast<gu4*>(&Bs[(c / GM_KCH) * GM_LD + bkc[i]]) = rb[i]; }
        __syncthreads();
        if (k0 + BK < g.K) {
#pragma unroll
            for (int i = 0; i < ACH; i++) ra[i] = load16(ap[i], k0 + BK + akc[i]);
#pragma unroll
            for (int i = 0; i < BCH; i++) rb[i] = load16(bp[i], k0 + BK + bkc[i]);
        }
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            gb8 af[MBW], bf[2];
#pragma unroll
            for (int a = 0; a < MBW; a++) af[a] = __builtin_bit_cast(gb8, *reinterpret_cast<const gu4*>(&As[(wr * (BM / 2) + a * 32 + r) * GM_LD + ks * 16 + h * 8]));
#pragma unroll
            for (int b = 0; b < 2; b++) bf[b] = __builtin_bit_cast(gb8, *reinterpret_cast<const gu4*>(&Bs[(wc * 64 + b * 32 + r) * GM_LD + ks * 16 + h * 8]));
#pragma unroll
            for (int a = 0; a < MBW; a++)
#pragma unroll
                for (int b = 0; b < 2; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bf[b], acc[a][b], 0, 0, 0);
        }
    }
#pragma unroll
    for (int a = 0; a < MBW; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const int n = n0 + wc * 64 + b * 32 + r;
            if (n >= g.N) continue;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int m = m0 + wr * (BM / 2) + a * 32 + (i & 3) + 8 * (i >> 2) + 4 * h;
                if (m < mend) gm_store<true>(g, m, n, acc[a][b][i]);
            }
        }
}
}  // namespace

bool kr_sv_gemm_small(const KrSvGemm& g) {
    // decode-sized problems: a pass over the weights per 8 rows; grouped problems take one row per workgroup row (each row has its own expert)
    return g.seg ? (g.M <= (g.rowwise_upto > 64 ? g.rowwise_upto : 64) && g.row_group) : g.M <= 16;
}

void kr_sv_gemm(const KrSvGemm& g, bool f32, hipStream_t st) {
    if (g.M <= 0 || g.N <= 0) return;
    const bool grouped = g.seg != nullptr;
    if (kr_sv_gemm_small(g)) {
#define GM_V(T_, MB_, CN_, GRID_, ARG_, MBASE_) do { if (g.act_gu) hipLaunchKernelGGL((sv_gemv_kernel<T_, MB_, CN_, true>), GRID_, dim3(256), 0, st, ARG_, MBASE_); \
                                                      else hipLaunchKernelGGL((sv_gemv_kernel<T_, MB_, CN_, false>), GRID_, dim3(256), 0, st, ARG_, MBASE_); } while (0)
        // columns per wave: 4 while that still leaves a few waves for every SIMD of the chip, else 1
        if (grouped) {
            const bool wide = (long)g.N * g.M >= 8192;
            const dim3 grid((g.N + (wide ? 15 : 3)) / (wide ? 16 : 4), g.M);
            if (wide) { if (f32) GM_V(float, 1, 4, grid, g, 0); else GM_V(uint16_t, 1, 4, grid, g, 0); }
            else { if (f32) GM_V(float, 1, 1, grid, g, 0); else GM_V(uint16_t, 1, 1, grid, g, 0); }
        } else {
            KrSvGemm p = g; p.row_group = nullptr;
            const bool wide = g.N >= 8192;
            const dim3 grid((g.N + (wide ? 15 : 3)) / (wide ? 16 : 4));
            for (int mb = 0; mb < g.M; mb += 8) {
                if (wide) { if (f32) GM_V(float, 8, 4, grid, p, mb); else GM_V(uint16_t, 8, 4, grid, p, mb); }
                else { if (f32) GM_V(float, 8, 1, grid, p, mb); else GM_V(uint16_t, 8, 1, grid, p, mb); }
            }
        }
#undef GM_V
        return;
    }
    if (f32) {
        const int tiles = grouped ? (g.M + 63) / 64 + g.n_groups : (g.M + 63) / 64;
        hipLaunchKernelGGL(sv_gemm_f32_kernel, dim3((g.N + 63) / 64, tiles), dim3(256), 0, st, g);
        return;
    }
    // grouped problems have few rows per expert: the 64-row tile wastes less of the matrix cores.  (A 256-row tile -- wave tiles of 128 x 64, six fragment
    // reads per eight MFMAs -- was measured and did not pay: two workgroups per compute unit instead of three.)
    const bool small = grouped ? (g.M / (g.n_groups > 0 ? g.n_groups : 1) < 96) : g.M <= 64;
    if (small) {
        const int tiles = grouped ? (g.M + 63) / 64 + g.n_groups : (g.M + 63) / 64;
        hipLaunchKernelGGL(sv_gemm_bf16_kernel<64>, dim3((g.N + 127) / 128, tiles), dim3(256), 0, st, g);
    } else {
        const int tiles = grouped ? (g.M + 127) / 128 + g.n_groups : (g.M + 127) / 128;
        hipLaunchKernelGGL(sv_gemm_bf16_kernel<128>, dim3((g.N + 127) / 128, tiles), dim3(256), 0, st, g);
    }
}
