// Kernels of libi64hip_dense.so for decoder models with bf16 weights and a 32-bit residual stream (include/i64h_dense.h):
//   linear_tile_kernel   : C = epilogue(A W^T), 64 x 64 tiles, four waves of 32 x 32, on v_mfma_f32_16x16x32_bf16 (A rounded to
//                          bf16 while staged) or v_mfma_f32_16x16x4_f32 (W widened while staged: true 32-bit); batched over
//                          blockIdx.z (per-head weights on column blocks of wider matrices); epilogues: gelu_tanh(gate) * up
//                          on two accumulators, * sigmoid(E), logit soft cap
//   linear_tile128_kernel: bf16 form, 128 x 128 tiles (waves of 64 x 64); behind a knob, measured slower at the sizes tried
//   linear_skinny_kernel : the same product for at most I64H_SKINNY_ROWS rows (decode steps): the rows sit in LDS as bf16, every
//                          wave streams four weight rows at a time with 16-byte loads and reduces over its lanes
//   linear_rows64_kernel : at most 64 rows: 16 output columns per workgroup, the k steps dealt to its four waves, every operand read
//                          from memory as a matrix-core fragment, partial tiles summed through LDS
//   embed_scaled_kernel  : bf16 table row * scale -> fp32
//   gated_postnorm_kernel: alpha * x + sigmoid(gate) * y -> RMS norm in groups -> (optional) weighted sum over the outputs of
//                          all earlier layers; one workgroup per row, the row held in LDS between the passes
//   sample_rows_kernel   : greedy / temperature / top-k / top-p draw of one token per row
#include "i64h_common.h"
#include "i64h_dense.h"
#include <type_traits>

typedef float dn_v4f __attribute__((ext_vector_type(4)));
typedef __bf16 dn_v8bf __attribute__((ext_vector_type(8)));

__device__ __forceinline__ uint32_t dn_bf16_rne(float f) {  // round to nearest even, NaN stays NaN: the hardware conversion of this chip
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ float dn_bf16_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ float dn_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float dn_gelu_tanh(float z) {
    const float inner = 0.7978845608028654f * (z + 0.044715f * z * z * z);
    return 0.5f * z * (1.0f + tanhf(inner));
}

__device__ __forceinline__ float dn_gelu_erf(float z) { return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f)); }

__device__ __forceinline__ float dn_xielu(float z, float a, float b) {
    return z > 0.0f ? a * z * z + 0.5f * z : b * (expm1f(z) - z) + 0.5f * z;
}
constexpr bool dn_dual(int epi) { return epi == I64H_EPI_GELU_MUL || epi == I64H_EPI_SILU_MUL; }  // two accumulators: gate rows and up rows

template <int EPI>
__device__ __forceinline__ float dn_epilogue(const i64h_linear& p, float acc, float acc2, int64_t b, int64_t r, int c) {
    if (EPI == I64H_EPI_GELU_MUL) return dn_gelu_tanh(acc) * acc2;
    if (EPI == I64H_EPI_SILU_MUL) return acc * dn_sigmoid(acc) * acc2;
    if (p.bias) acc += p.bias[b * p.bias_batch + c];
    if (EPI == I64H_EPI_XIELU) return dn_xielu(acc, p.act_a, p.act_b);
    if (EPI == I64H_EPI_RELU_SQ) return acc > 0.0f ? acc * acc : 0.0f;
    if (EPI == I64H_EPI_GELU_ERF) return dn_gelu_erf(acc);
    if (EPI == I64H_EPI_SCALE) return acc * p.scale;
    if (EPI == I64H_EPI_MUL_SIGMOID) return acc * dn_sigmoid(p.E[b * p.e_batch + r * p.lde + c]);
    if (EPI == I64H_EPI_SOFTCAP) return p.softcap * tanhf(acc / p.softcap);
    return acc;
}

// ---------------------------------------------------------------------------------------------------------------------------
template <bool EXACT, int EPI>
__global__ __launch_bounds__(256) void linear_tile_kernel(const i64h_linear p, const int vecA, const int vecW) {
    constexpr bool DUAL = dn_dual(EPI);
    constexpr int LD = EXACT ? 33 : 40;  // 33 words: conflict-free column reads; 40 halves = 80 bytes: 16-byte aligned fragments
    using T = typename std::conditional<EXACT, float, uint16_t>::type;
    __shared__ __attribute__((aligned(16))) T sA[2][64][LD];
    __shared__ __attribute__((aligned(16))) T sB[2][64][LD];
    __shared__ __attribute__((aligned(16))) T sB2[DUAL ? 2 : 1][DUAL ? 64 : 1][LD];
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int wm = wid >> 1, wn = wid & 1;
    const int64_t b = blockIdx.z;
    int64_t m0 = (int64_t)blockIdx.y * 64;
    const int n0 = blockIdx.x * 64;
    int64_t rows = p.M;
    if (p.group_off) {   // this batch's share of the rows; m0 becomes the tile's first row among all rows
        const int64_t g0 = p.group_off[b];
        rows = min(rows, (int64_t)p.group_off[b + 1] - g0);
        if (m0 >= rows) return;
        rows += g0;
        m0 += g0;
    }
    const int M = (int)min((int64_t)64, rows - m0);  // rows of this tile
    const int N = p.N, K = p.K;
    const int lr = tid >> 2, lc = (tid & 3) * 8;
    const bool aok = lr < M, bok = n0 + lr < N;
    const int64_t arow = aok ? (p.a_rows ? (int64_t)p.a_rows[m0 + lr] : m0 + lr) : 0;
    const float* pa = p.A + b * p.a_batch + arow * p.lda;
    const uint16_t* pw = (const uint16_t*)p.W + b * p.w_batch + (int64_t)(bok ? n0 + lr : 0) * K;
    const uint16_t* pw2 = pw + (int64_t)N * K;
    float ra[8];
    uint16_t rb[8], rb2[8];
    auto gload = [&](int k0) {
        const int k = k0 + lc;
        if (aok && vecA && k + 8 <= K) {
            const float4 u = *(const float4*)(pa + k), v = *(const float4*)(pa + k + 4);
            ra[0] = u.x; ra[1] = u.y; ra[2] = u.z; ra[3] = u.w; ra[4] = v.x; ra[5] = v.y; ra[6] = v.z; ra[7] = v.w;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) ra[i] = (aok && k + i < K) ? pa[k + i] : 0.0f;
        }
        if (bok && vecW && k + 8 <= K) {
            *(uint4*)rb = *(const uint4*)(pw + k);
            if (DUAL) *(uint4*)rb2 = *(const uint4*)(pw2 + k);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                rb[i] = (bok && k + i < K) ? pw[k + i] : (uint16_t)0;
                if (DUAL) rb2[i] = (bok && k + i < K) ? pw2[k + i] : (uint16_t)0;
            }
        }
    };
    auto lstore = [&](int buf) {
        if (EXACT) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                sA[buf][lr][lc + i] = (T)ra[i];
                sB[buf][lr][lc + i] = (T)dn_bf16_to_f32(rb[i]);
                if (DUAL) sB2[buf][lr][lc + i] = (T)dn_bf16_to_f32(rb2[i]);
            }
        } else {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = dn_bf16_rne(ra[2 * i]) | (dn_bf16_rne(ra[2 * i + 1]) << 16);
            *(uint4*)&sA[buf][lr][lc] = make_uint4(w[0], w[1], w[2], w[3]);
            *(uint4*)&sB[buf][lr][lc] = *(const uint4*)rb;
            if (DUAL) *(uint4*)&sB2[buf][lr][lc] = *(const uint4*)rb2;
        }
    };
    dn_v4f acc[2][2], acc2[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            acc[i][j] = dn_v4f{0, 0, 0, 0};
            acc2[i][j] = dn_v4f{0, 0, 0, 0};
        }
    const int fr = lane & 15, fk = lane >> 4;
    gload(0);
    lstore(0);
    __syncthreads();
    const int KT = (K + 31) / 32;
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) gload((kt + 1) * 32);  // the next tile is in flight behind the matrix instructions of this one
        if (EXACT) {
#pragma unroll
            for (int kk = 0; kk < 32; kk += 4) {
                float a[2], bb[2], b2[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) a[i] = (float)sA[cur][wm * 32 + i * 16 + fr][kk + fk];
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    bb[j] = (float)sB[cur][wn * 32 + j * 16 + fr][kk + fk];
                    if (DUAL) b2[j] = (float)sB2[cur][wn * 32 + j * 16 + fr][kk + fk];
                }
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], bb[j], acc[i][j], 0, 0, 0);
                        if (DUAL) acc2[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b2[j], acc2[i][j], 0, 0, 0);
                    }
            }
        } else {
            dn_v8bf a[2], bb[2], b2[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = *(const dn_v8bf*)&sA[cur][wm * 32 + i * 16 + fr][fk * 8];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                bb[j] = *(const dn_v8bf*)&sB[cur][wn * 32 + j * 16 + fr][fk * 8];
                if (DUAL) b2[j] = *(const dn_v8bf*)&sB2[cur][wn * 32 + j * 16 + fr][fk * 8];
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], bb[j], acc[i][j], 0, 0, 0);
                    if (DUAL) acc2[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b2[j], acc2[i][j], 0, 0, 0);
                }
        }
        if (kt + 1 < KT) lstore(cur ^ 1);
        __syncthreads();
    }
    float* C = p.C + b * p.c_batch;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int reg = 0; reg < 4; ++reg) {
            const int rl = wm * 32 + i * 16 + fk * 4 + reg;
            if (rl >= M) continue;
            const int64_t r = m0 + rl;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int c = n0 + wn * 32 + j * 16 + fr;
                if (c < N) C[r * p.ldc + c] = dn_epilogue<EPI>(p, acc[i][j][reg], acc2[i][j][reg], b, r, c);
            }
        }
}


// ---------------------------------------------------------------------------------------------------------------------------
// The bf16 form for launches with many tiles: 128 x 128 per workgroup, four waves of 64 x 64 (16 matrix instructions per wave and
// 32-wide k step against 8 fragment reads - four times the 64 x 64 kernel's ratio), the same staging scheme.
template <int EPI>
__global__ __launch_bounds__(256) void linear_tile128_kernel(const i64h_linear p, const int vecA, const int vecW) {
    constexpr bool DUAL = dn_dual(EPI);
    constexpr int LD = 40;
    __shared__ __attribute__((aligned(16))) uint16_t sA[2][128][LD];
    __shared__ __attribute__((aligned(16))) uint16_t sB[2][128][LD];
    __shared__ __attribute__((aligned(16))) uint16_t sB2[DUAL ? 2 : 1][DUAL ? 128 : 1][LD];
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int wm = wid >> 1, wn = wid & 1;
    const int64_t b = blockIdx.z;
    const int64_t m0 = (int64_t)blockIdx.y * 128;
    const int n0 = blockIdx.x * 128;
    const int M = (int)min((int64_t)128, p.M - m0);
    const int N = p.N, K = p.K;
    const int lr = tid >> 2, lc = (tid & 3) * 8;
    bool aok[2], bok[2];
    const float* pa[2];
    const uint16_t* pw[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int rr = lr + 64 * h;
        aok[h] = rr < M;
        bok[h] = n0 + rr < N;
        const int64_t arow = aok[h] ? (p.a_rows ? (int64_t)p.a_rows[m0 + rr] : m0 + rr) : 0;
        pa[h] = p.A + b * p.a_batch + arow * p.lda;
        pw[h] = (const uint16_t*)p.W + b * p.w_batch + (int64_t)(bok[h] ? n0 + rr : 0) * K;
    }
    const int64_t w2 = (int64_t)N * K;
    float ra[2][8];
    uint16_t rb[2][8], rb2[2][8];
    auto gload = [&](int k0) {
        const int k = k0 + lc;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (aok[h] && vecA && k + 8 <= K) {
                const float4 u = *(const float4*)(pa[h] + k), v = *(const float4*)(pa[h] + k + 4);
                ra[h][0] = u.x; ra[h][1] = u.y; ra[h][2] = u.z; ra[h][3] = u.w; ra[h][4] = v.x; ra[h][5] = v.y; ra[h][6] = v.z; ra[h][7] = v.w;
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) ra[h][i] = (aok[h] && k + i < K) ? pa[h][k + i] : 0.0f;
            }
            if (bok[h] && vecW && k + 8 <= K) {
                *(uint4*)rb[h] = *(const uint4*)(pw[h] + k);
                if (DUAL) *(uint4*)rb2[h] = *(const uint4*)(pw[h] + w2 + k);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    rb[h][i] = (bok[h] && k + i < K) ? pw[h][k + i] : (uint16_t)0;
                    if (DUAL) rb2[h][i] = (bok[h] && k + i < K) ? pw[h][w2 + k + i] : (uint16_t)0;
                }
            }
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = dn_bf16_rne(ra[h][2 * i]) | (dn_bf16_rne(ra[h][2 * i + 1]) << 16);
            *(uint4*)&sA[buf][lr + 64 * h][lc] = make_uint4(w[0], w[1], w[2], w[3]);
            *(uint4*)&sB[buf][lr + 64 * h][lc] = *(const uint4*)rb[h];
            if (DUAL) *(uint4*)&sB2[buf][lr + 64 * h][lc] = *(const uint4*)rb2[h];
        }
    };
    dn_v4f acc[4][4], acc2[DUAL ? 4 : 1][DUAL ? 4 : 1];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[i][j] = dn_v4f{0, 0, 0, 0};
            if (DUAL) acc2[DUAL ? i : 0][DUAL ? j : 0] = dn_v4f{0, 0, 0, 0};
        }
    const int fr = lane & 15, fk = lane >> 4;
    gload(0);
    lstore(0);
    __syncthreads();
    const int KT = (K + 31) / 32;
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) gload((kt + 1) * 32);
        dn_v8bf a[4], bb[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = *(const dn_v8bf*)&sA[cur][wm * 64 + i * 16 + fr][fk * 8];
#pragma unroll
        for (int j = 0; j < 4; ++j) bb[j] = *(const dn_v8bf*)&sB[cur][wn * 64 + j * 16 + fr][fk * 8];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], bb[j], acc[i][j], 0, 0, 0);
        if (DUAL) {
#pragma unroll
            for (int j = 0; j < 4; ++j) bb[j] = *(const dn_v8bf*)&sB2[cur][wn * 64 + j * 16 + fr][fk * 8];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc2[DUAL ? i : 0][DUAL ? j : 0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], bb[j], acc2[DUAL ? i : 0][DUAL ? j : 0], 0, 0, 0);
        }
        if (kt + 1 < KT) lstore(cur ^ 1);
        __syncthreads();
    }
    float* C = p.C + b * p.c_batch;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int reg = 0; reg < 4; ++reg) {
            const int rl = wm * 64 + i * 16 + fk * 4 + reg;
            if (rl >= M) continue;
            const int64_t r = m0 + rl;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = n0 + wn * 64 + j * 16 + fr;
                if (c < N) C[r * p.ldc + c] = dn_epilogue<EPI>(p, acc[i][j][reg], DUAL ? acc2[DUAL ? i : 0][DUAL ? j : 0][reg] : 0.0f, b, r, c);
            }
        }
}

// ---------------------------------------------------------------------------------------------------------------------------
// M <= 8 rows.  The rows are rounded to bf16 into LDS once per workgroup (M * K halves); a wave takes CPW = 4 weight rows at a
// time, every lane 8 consecutive k of each per iteration (one 16-byte load per weight row), products in fp32.
template <int EPI>
__global__ __launch_bounds__(256) void linear_skinny_kernel(const i64h_linear p, const int cols_per_block) {
    constexpr bool DUAL = dn_dual(EPI);
    constexpr int CPW = 4, MR = I64H_SKINNY_ROWS;
    extern __shared__ __attribute__((aligned(16))) uint16_t sa[];  // [M][K]
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int64_t b = blockIdx.z;
    const int M = (int)p.M, N = p.N, K = p.K;
    for (int m = 0; m < M; ++m) {
        const int64_t arow = p.a_rows ? (int64_t)p.a_rows[m] : m;
        const float* pa = p.A + b * p.a_batch + arow * p.lda;
        for (int k = tid * 4; k < K; k += 1024) {
            const float4 v = *(const float4*)(pa + k);
            *(uint2*)&sa[m * K + k] = make_uint2(dn_bf16_rne(v.x) | (dn_bf16_rne(v.y) << 16), dn_bf16_rne(v.z) | (dn_bf16_rne(v.w) << 16));
        }
    }
    __syncthreads();
    const uint16_t* W = (const uint16_t*)p.W + b * p.w_batch;
    float* C = p.C + b * p.c_batch;
    const int c_end = min(N, (int)(blockIdx.x + 1) * cols_per_block);
    for (int c0 = blockIdx.x * cols_per_block + wid * CPW; c0 < c_end; c0 += 4 * CPW) {
        float acc[CPW][MR], acc2[DUAL ? CPW : 1][MR];
#pragma unroll
        for (int j = 0; j < CPW; ++j)
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                acc[j][m] = 0.0f;
                if (DUAL) acc2[j][m] = 0.0f;
            }
        for (int k = lane * 8; k < K; k += 512) {
            uint4 w[CPW], w2[DUAL ? CPW : 1];
#pragma unroll
            for (int j = 0; j < CPW; ++j) {
                const int c = min(c0 + j, N - 1);
                w[j] = *(const uint4*)(W + (int64_t)c * K + k);
                if (DUAL) w2[j] = *(const uint4*)(W + (int64_t)(c + N) * K + k);
            }
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                if (m >= M) break;
                const uint4 a = *(const uint4*)&sa[m * K + k];
                const uint32_t aw[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
                for (int j = 0; j < CPW; ++j) {
                    const uint32_t ww[4] = {w[j].x, w[j].y, w[j].z, w[j].w};
                    float s = acc[j][m];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        s = fmaf(__uint_as_float(aw[q] << 16), __uint_as_float(ww[q] << 16), s);
                        s = fmaf(__uint_as_float(aw[q] & 0xffff0000u), __uint_as_float(ww[q] & 0xffff0000u), s);
                    }
                    acc[j][m] = s;
                    if (DUAL) {
                        const uint32_t w2w[4] = {w2[j].x, w2[j].y, w2[j].z, w2[j].w};
                        float s2 = acc2[j][m];
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            s2 = fmaf(__uint_as_float(aw[q] << 16), __uint_as_float(w2w[q] << 16), s2);
                            s2 = fmaf(__uint_as_float(aw[q] & 0xffff0000u), __uint_as_float(w2w[q] & 0xffff0000u), s2);
                        }
                        acc2[j][m] = s2;
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < CPW; ++j)
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                if (m >= M) break;
                const float s = wave_sum(acc[j][m]);
                const float s2 = DUAL ? wave_sum(acc2[j][m]) : 0.0f;
                const int c = c0 + j;
                if (lane == 0 && c < c_end) C[(int64_t)m * p.ldc + c] = dn_epilogue<EPI>(p, s, s2, b, m, c);
            }
    }
}


// ---------------------------------------------------------------------------------------------------------------------------
// At most 64 rows (decode steps, small batches), bf16 form.  A workgroup owns 16 output columns; its four or eight waves deal the
// 32-wide k steps among them, each with up to four 16-row blocks of A against the one weight fragment, all operands read straight from memory
// as matrix-core fragments (no staging, no barrier inside the loop); the four partial tiles meet in LDS, then the epilogue.
// Many small workgroups fill the chip where a launch has few 64-column tiles, and the weights stream exactly once.
template <int EPI, int NW>
__global__ __launch_bounds__(64 * NW) void linear_rows64_kernel(const i64h_linear p) {
    constexpr bool DUAL = dn_dual(EPI);
    __shared__ float red[DUAL ? 2 : 1][NW][64][17];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int n = lane & 15, kg = lane >> 4;
    const int64_t b = blockIdx.z;
    const int n0 = blockIdx.x * 16;
    int M = (int)p.M;
    const int N = p.N, K = p.K;
    int64_t g0 = 0;      // this batch's first row among all rows, where the rows are dealt to the batches by group_off
    if (p.group_off) {
        g0 = p.group_off[b];
        M = min(M, p.group_off[b + 1] - (int)g0);
        if (M <= 0) return;
    }
    const int mblocks = (M + 15) / 16;
    const bool cok = n0 + n < N;
    const uint16_t* pw = (const uint16_t*)p.W + b * p.w_batch + (int64_t)(cok ? n0 + n : 0) * K;
    const uint16_t* pw2 = pw + (int64_t)N * K;
    const float* pa[4];
    bool rok[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = i * 16 + n;
        rok[i] = m < M;
        const int64_t arow = rok[i] ? (p.a_rows ? (int64_t)p.a_rows[g0 + m] : g0 + m) : 0;
        pa[i] = p.A + b * p.a_batch + arow * p.lda;
    }
    dn_v4f acc[4], acc2[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc[i] = dn_v4f{0, 0, 0, 0};
        acc2[i] = dn_v4f{0, 0, 0, 0};
    }
    const int KT = (K + 31) / 32;
    // U k steps per turn: the loads of all of them are requested before the first matrix instruction (four per turn measured slower:
    // 21 against 17 us on the gate / up launch of 64 rows - the registers cost a wave per SIMD)
    constexpr int U = 2;
    for (int kt = wv; kt < KT; kt += U * NW) {
        uint4 wf[U], wf2[U];
        float4 au[U][4], av[U][4];
#pragma unroll
        for (int h = 0; h < U; ++h) {
            const int k = (kt + h * NW) * 32 + kg * 8;
            const bool kin = kt + h * NW < KT && k < K;
            wf[h] = wf2[h] = make_uint4(0, 0, 0, 0);
            if (cok && kin) {
                wf[h] = *(const uint4*)(pw + k);
                if (DUAL) wf2[h] = *(const uint4*)(pw2 + k);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                au[h][i] = av[h][i] = make_float4(0, 0, 0, 0);
                if (i < mblocks && rok[i] && kin) {
                    au[h][i] = *(const float4*)(pa[i] + k);
                    av[h][i] = *(const float4*)(pa[i] + k + 4);
                }
            }
        }
#pragma unroll
        for (int h = 0; h < U; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (i < mblocks) {
                    const float4 u = au[h][i], v = av[h][i];
                    const uint4 af = make_uint4(dn_bf16_rne(u.x) | (dn_bf16_rne(u.y) << 16), dn_bf16_rne(u.z) | (dn_bf16_rne(u.w) << 16),
                                                dn_bf16_rne(v.x) | (dn_bf16_rne(v.y) << 16), dn_bf16_rne(v.z) | (dn_bf16_rne(v.w) << 16));
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dn_v8bf, af), __builtin_bit_cast(dn_v8bf, wf[h]), acc[i], 0, 0, 0);
                    if (DUAL) acc2[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dn_v8bf, af), __builtin_bit_cast(dn_v8bf, wf2[h]), acc2[i], 0, 0, 0);
                }
            }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            red[0][wv][i * 16 + kg * 4 + g][n] = acc[i][g];
            if (DUAL) red[DUAL ? 1 : 0][wv][i * 16 + kg * 4 + g][n] = acc2[i][g];
        }
    __syncthreads();
    float* C = p.C + b * p.c_batch;
    for (int e = tid; e < 64 * 16; e += 64 * NW) {
        const int m = e >> 4, c = e & 15;
        if (m >= M || n0 + c >= N) continue;
        float s = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            s += red[0][w][m][c];
            if (DUAL) s2 += red[DUAL ? 1 : 0][w][m][c];
        }
        C[(g0 + m) * p.ldc + n0 + c] = dn_epilogue<EPI>(p, s, s2, b, g0 + m, n0 + c);
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void embed_scaled_kernel(const int64_t* __restrict__ ids, const uint16_t* __restrict__ table, float scale,
                                                           float* __restrict__ out, int W, int64_t V) {
    const int64_t t = blockIdx.x;
    int64_t id = ids[t];
    id = id < 0 ? 0 : (id >= V ? V - 1 : id);
    const uint16_t* row = table + id * W;
    for (int c = threadIdx.x; c < W; c += 256) out[t * W + c] = dn_bf16_to_f32(row[c]) * scale;
}

// ---------------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gated_postnorm_kernel(const i64h_postnorm p) {
    extern __shared__ float sv[];  // [W] the row before the norm, then [groups] root mean squares
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int64_t m = blockIdx.x;
    const int W = p.W;
    const int64_t xr = p.x_rows ? (int64_t)p.x_rows[m] : m;
    const float* x = p.x + xr * W;
    for (int c = tid; c < W; c += 256) {
        float v = p.alpha * x[c];
        if (p.y) {
            float g = 1.0f;
            if (p.gate_pre) g = dn_sigmoid(p.gate_pre[m * p.ldg + c] + (p.gate_bias ? p.gate_bias[c] : 0.0f));
            v = v + g * p.y[m * p.ldy + c];
        }
        sv[c] = v;
    }
    __syncthreads();
    const int gs = W / p.groups;
    for (int g = wid; g < p.groups; g += 4) {
        float s = 0.0f;
        for (int c = lane; c < gs; c += 64) {
            const float v = sv[g * gs + c];
            s += v * v;
        }
        s = wave_sum(s);
        if (lane == 0) sv[W + g] = sqrtf(s / (float)gs + p.eps);
    }
    __syncthreads();
    const int64_t plane = p.n * (int64_t)W;
    if ((W & 3) == 0 && ((uintptr_t)p.norm_w & 15) == 0 && ((uintptr_t)p.out & 15) == 0 && ((uintptr_t)p.hist & 15) == 0 && ((uintptr_t)p.mix_out & 15) == 0 &&
        gs % 4 == 0) {
        // four columns per thread and 16-byte accesses; the history planes are read four at a time (independent loads in flight)
        for (int c = tid * 4; c < W; c += 1024) {
            const float den = sv[W + c / gs];
            const float4 nw = *(const float4*)(p.norm_w + c);
            float4 o;
            o.x = sv[c] / den * nw.x; o.y = sv[c + 1] / den * nw.y; o.z = sv[c + 2] / den * nw.z; o.w = sv[c + 3] / den * nw.w;
            if (p.out) *(float4*)(p.out + m * W + c) = o;
            if (p.mix_w) {
                const float* h = p.hist + m * W + c;
                *(float4*)(p.hist + p.hist_index * plane + m * W + c) = o;
                float4 a = make_float4(0, 0, 0, 0);
                int j = 0;
                for (; j + 4 <= p.hist_index; j += 4) {
                    float4 v[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) v[u] = *(const float4*)(h + (j + u) * plane);
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const float wj = p.mix_w[j + u];
                        a.x += wj * v[u].x; a.y += wj * v[u].y; a.z += wj * v[u].z; a.w += wj * v[u].w;
                    }
                }
                for (; j < p.hist_index; ++j) {
                    const float4 v = *(const float4*)(h + j * plane);
                    const float wj = p.mix_w[j];
                    a.x += wj * v.x; a.y += wj * v.y; a.z += wj * v.z; a.w += wj * v.w;
                }
                const float wl = p.mix_w[p.hist_index];
                a.x += wl * o.x; a.y += wl * o.y; a.z += wl * o.z; a.w += wl * o.w;
                *(float4*)(p.mix_out + m * W + c) = a;
            }
        }
        return;
    }
    for (int c = tid; c < W; c += 256) {
        const float o = sv[c] / sv[W + c / gs] * p.norm_w[c];
        if (p.out) p.out[m * W + c] = o;
        if (p.mix_w) {
            p.hist[p.hist_index * plane + m * W + c] = o;
            float a = 0.0f;
            for (int j = 0; j < p.hist_index; ++j) a += p.mix_w[j] * p.hist[j * plane + m * W + c];
            a += p.mix_w[p.hist_index] * o;
            p.mix_out[m * W + c] = a;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
// One workgroup per row.  Thresholds are found by bisection over the bits of the order-preserving integer image of a float:
// top-k: the largest key with at least k values at or above it; top-p: the largest key whose values at or above it hold at
// least p of the mass.  The draw walks the kept values in index order (each thread a contiguous range).
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

__global__ __launch_bounds__(256) void sample_rows_kernel(const float* __restrict__ logits, int64_t* __restrict__ out, int V,
                                                          const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
                                                          const float* __restrict__ top_p, const float* __restrict__ u) {
    __shared__ float red[4];
    __shared__ float smax[256];
    __shared__ int sidx[256];
    __shared__ float part[257];
    __shared__ int chosen;
    const int tid = threadIdx.x;
    const int64_t r = blockIdx.x;
    const float* x = logits + r * V;
    const float T = temperature ? temperature[r] : 0.0f;
    // the maximum and its first index
    float best = -INFINITY;
    int bi = V;
    for (int c = tid; c < V; c += 256) {
        const float v = x[c];
        if (v > best || (v == best && c < bi)) { best = v; bi = c; }
    }
    smax[tid] = best;
    sidx[tid] = bi;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (tid < s) {
            const float v = smax[tid + s];
            const int i = sidx[tid + s];
            if (v > smax[tid] || (v == smax[tid] && i < sidx[tid])) { smax[tid] = v; sidx[tid] = i; }
        }
        __syncthreads();
    }
    const float mx = smax[0];
    if (!(T > 0.0f)) {
        if (tid == 0) out[r] = sidx[0] < V ? sidx[0] : 0;
        return;
    }
    const float invT = 1.0f / T;
    uint32_t thr = 0;  // keep values whose key is >= thr
    const int k = top_k ? top_k[r] : 0;
    if (k > 0 && k < V) {
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = thr | (1u << bit);
            float cnt = 0.0f;
            for (int c = tid; c < V; c += 256) cnt += f32_to_ordered(x[c]) >= cand ? 1.0f : 0.0f;
            if (block_sum(cnt, red) >= (float)k) thr = cand;
        }
    }
    const float pp = top_p ? top_p[r] : 1.0f;
    if (pp < 1.0f) {
        float z = 0.0f;
        for (int c = tid; c < V; c += 256) z += f32_to_ordered(x[c]) >= thr ? expf((x[c] - mx) * invT) : 0.0f;
        const float need = pp * block_sum(z, red);
        uint32_t t2 = 0;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = t2 | (1u << bit), cut = cand > thr ? cand : thr;
            float s = 0.0f;
            for (int c = tid; c < V; c += 256) s += f32_to_ordered(x[c]) >= cut ? expf((x[c] - mx) * invT) : 0.0f;
            if (block_sum(s, red) >= need) t2 = cand;
        }
        thr = t2 > thr ? t2 : thr;
    }
    // draw
    const int per = (V + 255) / 256, lo = tid * per, hi = min(V, lo + per);
    float s = 0.0f;
    for (int c = lo; c < hi; ++c) s += f32_to_ordered(x[c]) >= thr ? expf((x[c] - mx) * invT) : 0.0f;
    part[tid + 1] = s;
    if (tid == 0) { part[0] = 0.0f; chosen = -1; }
    __syncthreads();
    if (tid == 0)
        for (int i = 1; i <= 256; ++i) part[i] += part[i - 1];
    __syncthreads();
    const float target = (u ? u[r] : 0.5f) * part[256];
    if (hi > lo && target >= part[tid] && target < part[tid + 1]) {
        float a = part[tid];
        int pick = -1;
        for (int c = lo; c < hi; ++c) {
            if (f32_to_ordered(x[c]) < thr) continue;
            a += expf((x[c] - mx) * invT);
            pick = c;
            if (a > target) break;
        }
        if (pick >= 0) chosen = pick;
    }
    __syncthreads();
    if (tid == 0) out[r] = chosen >= 0 ? chosen : sidx[0];  // rounding at the far end of the walk: the most likely token
}

// ---------------------------------------------------------------------------------------------------------------------------
template <bool EXACT>
static void launch_tile(const i64h_linear& d, dim3 grid, hipStream_t s, int vecA, int vecW) {
    switch (d.epilogue) {
        case I64H_EPI_GELU_MUL: hipLaunchKernelGGL((linear_tile_kernel<EXACT, I64H_EPI_GELU_MUL>), grid, dim3(256), 0, s, d, vecA, vecW); break;
        case I64H_EPI_SILU_MUL: hipLaunchKernelGGL((linear_tile_kernel<EXACT, I64H_EPI_SILU_MUL>), grid, dim3(256), 0, s, d, vecA, vecW); break;
        case I64H_EPI_MUL_SIGMOID: hipLaunchKernelGGL((linear_tile_kernel<EXACT, I64H_EPI_MUL_SIGMOID>), grid, dim3(256), 0, s, d, vecA, vecW); break;
        case I64H_EPI_SOFTCAP: hipLaunchKernelGGL((linear_tile_kernel<EXACT, I64H_EPI_SOFTCAP>), grid, dim3(256), 0, s, d, vecA, vecW); break;
        case I64H_EPI_GELU_ERF: hipLaunchKernelGGL((linear_tile_kernel<EXACT, I64H_EPI_GELU_ERF>), grid, dim3(256), 0, s, d, vecA, vecW); break;
        case I64H_EPI_XIELU: hipLaunchKernelGGL((linear_tile_kernel<EXACT, I64H_EPI_XIELU>), grid, dim3(256), 0, s, d, vecA, vecW); break;
        case I64H_EPI_RELU_SQ: hipLaunchKernelGGL((linear_tile_kernel<EXACT, I64H_EPI_RELU_SQ>), grid, dim3(256), 0, s, d, vecA, vecW); break;
        case I64H_EPI_SCALE: hipLaunchKernelGGL((linear_tile_kernel<EXACT, I64H_EPI_SCALE>), grid, dim3(256), 0, s, d, vecA, vecW); break;
        default: hipLaunchKernelGGL((linear_tile_kernel<EXACT, I64H_EPI_STORE>), grid, dim3(256), 0, s, d, vecA, vecW); break;
    }
}

// the large tile is off by default: at 4096 rows and 1024 to 8192 columns (256 to 1024 tiles) it measured 1.3 to 1.8 times SLOWER than
// the 64 x 64 kernel - one workgroup per CU leaves nothing to run while it waits at its barriers
static int g_skinny = 1, g_rows64 = 1, g_tile128 = 0;

extern "C" {

// tuning / test knob, bit 0: launches of at most 8 rows on the weight-streaming kernel; bit 1: launches of at most 64 rows on the
// fragment-streaming kernel; bit 2: launches of 256 or more 128 x 128 tiles on the large-tile kernel (default 3; 0 = every launch on
// the 64 x 64 tile kernel)
int i64h_set_linear_skinny(int32_t on) {
    g_skinny = on & 1;
    g_rows64 = (on >> 1) & 1;
    g_tile128 = (on >> 2) & 1;
    return 0;
}

int i64h_linear_run(const i64h_linear* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "linear: no descriptor");
    const i64h_linear& d = *dp;
    I64H_CHECK_ARG(d.M >= 0 && d.N > 0 && d.K > 0 && d.batch > 0, "linear: bad sizes M=%lld N=%d K=%d batch=%d", (long long)d.M, d.N, d.K, d.batch);
    I64H_CHECK_ARG(d.A && d.W && d.C, "linear: null operand");
    I64H_CHECK_ARG(d.epilogue >= 0 && d.epilogue <= I64H_EPI_RELU_SQ, "linear: epilogue %d", d.epilogue);
    I64H_CHECK_ARG(d.epilogue != I64H_EPI_MUL_SIGMOID || d.E, "linear: the sigmoid epilogue needs E");
    I64H_CHECK_ARG(d.epilogue != I64H_EPI_SOFTCAP || d.softcap > 0.0f, "linear: soft cap %g", (double)d.softcap);
    I64H_CHECK_ARG(!dn_dual(d.epilogue) || !d.bias, "linear: the gate / up epilogues take no bias");
    I64H_CHECK_ARG(d.lda >= d.K || d.M <= 1, "linear: lda %lld < K %d", (long long)d.lda, d.K);
    I64H_CHECK_ARG(d.batch <= 65535 && (d.M + 63) / 64 <= 65535, "linear: grid too large");
    if (d.M == 0) return 0;
    const int vecA = (uintptr_t)d.A % 16 == 0 && d.lda % 4 == 0 && d.a_batch % 4 == 0;
    const int vecW = (uintptr_t)d.W % 16 == 0 && d.K % 8 == 0 && d.w_batch % 8 == 0;
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)d.M * d.K * 2;
    if (g_skinny && !d.group_off && !d.exact && d.M <= I64H_SKINNY_ROWS && vecA && vecW && lds <= 64 * 1024) {
        int cpb = 64;  // columns per workgroup: at least about two workgroups per CU, a wave takes four columns at a time
        while (cpb > 16 && (int64_t)((d.N + cpb - 1) / cpb) * d.batch < 512) cpb >>= 1;
        const dim3 grid((unsigned)((d.N + cpb - 1) / cpb), 1, (unsigned)d.batch);
        switch (d.epilogue) {
            case I64H_EPI_GELU_MUL: hipLaunchKernelGGL((linear_skinny_kernel<I64H_EPI_GELU_MUL>), grid, dim3(256), lds, s, d, cpb); break;
            case I64H_EPI_SILU_MUL: hipLaunchKernelGGL((linear_skinny_kernel<I64H_EPI_SILU_MUL>), grid, dim3(256), lds, s, d, cpb); break;
            case I64H_EPI_MUL_SIGMOID: hipLaunchKernelGGL((linear_skinny_kernel<I64H_EPI_MUL_SIGMOID>), grid, dim3(256), lds, s, d, cpb); break;
            case I64H_EPI_SOFTCAP: hipLaunchKernelGGL((linear_skinny_kernel<I64H_EPI_SOFTCAP>), grid, dim3(256), lds, s, d, cpb); break;
            case I64H_EPI_GELU_ERF: hipLaunchKernelGGL((linear_skinny_kernel<I64H_EPI_GELU_ERF>), grid, dim3(256), lds, s, d, cpb); break;
            case I64H_EPI_XIELU: hipLaunchKernelGGL((linear_skinny_kernel<I64H_EPI_XIELU>), grid, dim3(256), lds, s, d, cpb); break;
            case I64H_EPI_RELU_SQ: hipLaunchKernelGGL((linear_skinny_kernel<I64H_EPI_RELU_SQ>), grid, dim3(256), lds, s, d, cpb); break;
            case I64H_EPI_SCALE: hipLaunchKernelGGL((linear_skinny_kernel<I64H_EPI_SCALE>), grid, dim3(256), lds, s, d, cpb); break;
            default: hipLaunchKernelGGL((linear_skinny_kernel<I64H_EPI_STORE>), grid, dim3(256), lds, s, d, cpb); break;
        }
        I64H_CHECK_LAUNCH();
        return 0;
    }
    if (g_rows64 && !d.exact && d.M <= 64 && vecA && vecW) {
        const dim3 grid((unsigned)((d.N + 15) / 16), 1, (unsigned)d.batch);
        switch (d.epilogue) {
            // eight waves share the k steps where one accumulator is kept (the gate / up pair needs twice the LDS: four)
            case I64H_EPI_GELU_MUL: hipLaunchKernelGGL((linear_rows64_kernel<I64H_EPI_GELU_MUL, 4>), grid, dim3(256), 0, s, d); break;
            case I64H_EPI_SILU_MUL: hipLaunchKernelGGL((linear_rows64_kernel<I64H_EPI_SILU_MUL, 4>), grid, dim3(256), 0, s, d); break;
            case I64H_EPI_MUL_SIGMOID: hipLaunchKernelGGL((linear_rows64_kernel<I64H_EPI_MUL_SIGMOID, 8>), grid, dim3(512), 0, s, d); break;
            case I64H_EPI_SOFTCAP: hipLaunchKernelGGL((linear_rows64_kernel<I64H_EPI_SOFTCAP, 8>), grid, dim3(512), 0, s, d); break;
            case I64H_EPI_GELU_ERF: hipLaunchKernelGGL((linear_rows64_kernel<I64H_EPI_GELU_ERF, 8>), grid, dim3(512), 0, s, d); break;
            case I64H_EPI_XIELU: hipLaunchKernelGGL((linear_rows64_kernel<I64H_EPI_XIELU, 8>), grid, dim3(512), 0, s, d); break;
            case I64H_EPI_RELU_SQ: hipLaunchKernelGGL((linear_rows64_kernel<I64H_EPI_RELU_SQ, 8>), grid, dim3(512), 0, s, d); break;
            case I64H_EPI_SCALE: hipLaunchKernelGGL((linear_rows64_kernel<I64H_EPI_SCALE, 8>), grid, dim3(512), 0, s, d); break;
            default: hipLaunchKernelGGL((linear_rows64_kernel<I64H_EPI_STORE, 8>), grid, dim3(512), 0, s, d); break;
        }
        I64H_CHECK_LAUNCH();
        return 0;
    }
    const int64_t tiles128 = ((d.N + 127) / 128) * ((d.M + 127) / 128) * (int64_t)d.batch;
    if (g_tile128 && !d.group_off && !d.exact && tiles128 >= 256) {     // at least a workgroup per CU: the large tile pays
        const dim3 grid((unsigned)((d.N + 127) / 128), (unsigned)((d.M + 127) / 128), (unsigned)d.batch);
        switch (d.epilogue) {
            case I64H_EPI_GELU_MUL: hipLaunchKernelGGL((linear_tile128_kernel<I64H_EPI_GELU_MUL>), grid, dim3(256), 0, s, d, vecA, vecW); break;
            case I64H_EPI_SILU_MUL: hipLaunchKernelGGL((linear_tile128_kernel<I64H_EPI_SILU_MUL>), grid, dim3(256), 0, s, d, vecA, vecW); break;
            case I64H_EPI_MUL_SIGMOID: hipLaunchKernelGGL((linear_tile128_kernel<I64H_EPI_MUL_SIGMOID>), grid, dim3(256), 0, s, d, vecA, vecW); break;
            case I64H_EPI_SOFTCAP: hipLaunchKernelGGL((linear_tile128_kernel<I64H_EPI_SOFTCAP>), grid, dim3(256), 0, s, d, vecA, vecW); break;
            case I64H_EPI_GELU_ERF: hipLaunchKernelGGL((linear_tile128_kernel<I64H_EPI_GELU_ERF>), grid, dim3(256), 0, s, d, vecA, vecW); break;
            case I64H_EPI_XIELU: hipLaunchKernelGGL((linear_tile128_kernel<I64H_EPI_XIELU>), grid, dim3(256), 0, s, d, vecA, vecW); break;
            case I64H_EPI_RELU_SQ: hipLaunchKernelGGL((linear_tile128_kernel<I64H_EPI_RELU_SQ>), grid, dim3(256), 0, s, d, vecA, vecW); break;
            case I64H_EPI_SCALE: hipLaunchKernelGGL((linear_tile128_kernel<I64H_EPI_SCALE>), grid, dim3(256), 0, s, d, vecA, vecW); break;
            default: hipLaunchKernelGGL((linear_tile128_kernel<I64H_EPI_STORE>), grid, dim3(256), 0, s, d, vecA, vecW); break;
        }
        I64H_CHECK_LAUNCH();
        return 0;
    }
    const dim3 grid((unsigned)((d.N + 63) / 64), (unsigned)((d.M + 63) / 64), (unsigned)d.batch);
    if (d.exact) launch_tile<true>(d, grid, s, vecA, vecW);
    else launch_tile<false>(d, grid, s, vecA, vecW);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_embed_scaled(const int64_t* ids, const void* table_bf16, float scale, float* out, int64_t n, int32_t W, int64_t V, void* stream) {
    I64H_CHECK_ARG(n >= 0 && W > 0 && V > 0, "embed_scaled: bad sizes");
    if (n == 0) return 0;
    hipLaunchKernelGGL(embed_scaled_kernel, dim3((unsigned)n), dim3(256), 0, (hipStream_t)stream, ids, (const uint16_t*)table_bf16, scale, out,
                       (int)W, V);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_gated_postnorm(const i64h_postnorm* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "gated_postnorm: no descriptor");
    const i64h_postnorm& d = *dp;
    I64H_CHECK_ARG(d.n >= 0 && d.W > 0 && d.groups > 0 && d.W % d.groups == 0, "gated_postnorm: W %d does not split into %d groups", d.W, d.groups);
    I64H_CHECK_ARG(d.x && d.norm_w, "gated_postnorm: null operand");
    I64H_CHECK_ARG(!d.mix_w || (d.hist && d.mix_out && d.hist_index >= 0), "gated_postnorm: the depth mix needs hist and mix_out");
    I64H_CHECK_ARG(d.out || d.mix_w, "gated_postnorm: no output");
    const size_t lds = ((size_t)d.W + d.groups) * 4;
    I64H_CHECK_ARG(lds <= 64 * 1024, "gated_postnorm: a row of %d values does not fit the kernel's LDS buffer", d.W);
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(gated_postnorm_kernel, dim3((unsigned)d.n), dim3(256), lds, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_sample_rows(const float* logits, int64_t* out, int64_t rows, int32_t V, const float* temperature, const int32_t* top_k,
                     const float* top_p, const float* u, void* stream) {
    I64H_CHECK_ARG(rows >= 0 && V > 0 && logits && out, "sample_rows: bad arguments");
    if (rows == 0) return 0;
    hipLaunchKernelGGL(sample_rows_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, logits, out, (int)V, temperature, top_k, top_p, u);
    I64H_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"
