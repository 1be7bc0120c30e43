// Latent attention of libi64hip_dense.so (include/i64h_dense.h): every token caches ONE row per layer - a normalised low-rank
// latent and a rotated key part shared by all heads.  The per-head key and value projections of the latent are never
// materialised: the caller carries the query through the key projection (q' = W_uk^T q, a batched Linear) and the attention
// output back through the value projection (a batched Linear over the summed latents), so a head's score is
// q'_latent . latent_j + q_rot . key_rot_j and all heads read the same cached rows.
//   latent_prep_kernel     : RMS norm of the latent, rotation of the shared key part and of every head's rotated query part,
//                            cache write - one workgroup per token
//   latent_attn_mfma_kernel: bf16 caches of aligned widths - 16 query vectors per wave (a token's heads, or a head's consecutive rows)
//                            on the bf16 matrix cores, see below
//   latent_attn_row_kernel : any width and cache type, true fp32 products: one wave per (token, head): 64 keys at a time, one key per lane for the scores (fp32 dot over the
//                            cached row), online softmax over the wave, weighted row sum with the columns spread over the lanes
#include "i64h_common.h"
#include "i64h_dense.h"

__device__ __forceinline__ float lt_load(const void* cache, int dtype, int64_t idx) {
    return dtype == 0 ? ((const float*)cache)[idx] : __uint_as_float((uint32_t)((const uint16_t*)cache)[idx] << 16);
}
__device__ __forceinline__ void lt_store(void* cache, int dtype, int64_t idx, float v) {
    if (dtype == 0) {
        ((float*)cache)[idx] = v;
    } else {
        uint32_t u = __float_as_uint(v);
        u = (u & 0x7fffffffu) > 0x7f800000u ? ((u >> 16) | 0x40u) : ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
        ((uint16_t*)cache)[idx] = (uint16_t)u;
    }
}

__global__ __launch_bounds__(256) void latent_prep_kernel(const i64h_latent_prep_args p) {
    __shared__ float red[4];
    const int tid = threadIdx.x;
    const int64_t t = blockIdx.x;
    const int pos = p.positions[t], slot = p.slot_ids[t];
    const int r = p.kv_rank, rd = p.rot_dim, D = r + rd, half = p.rot_dims / 2;
    const int64_t row = (int64_t)p.block_table[(int64_t)slot * p.max_blocks_per_seq + pos / p.block_size] * p.block_size + pos % p.block_size;
    const float* pr = p.P + t * p.ldp;
    const float* dkv = pr + p.dkv_off;
    float s = 0.0f;
    for (int c = tid; c < r; c += 256) s += dkv[c] * dkv[c];
    s = wave_sum(s);
    if ((tid & 63) == 0) red[tid >> 6] = s;
    __syncthreads();
    const float den = sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)r + p.eps);
    for (int c = tid; c < r; c += 256) lt_store(p.cache, p.cache_dtype, row * D + c, dkv[c] / den * p.c_norm_w[c]);
    const float fpos = (float)pos;
    // the shared key part and every head's query part: index 0 is the key, 1 + h the heads
    for (int e = tid; e < (p.heads + 1) * rd; e += 256) {
        const int who = e / rd, c = e % rd;
        const float* src = who == 0 ? dkv + r : pr + p.q_off + (int64_t)(who - 1) * (p.dim + rd) + p.dim;
        float v;
        if (c < 2 * half) {
            float sn, cs;
            sincosf(fpos * p.inv_freq[c >> 1], &sn, &cs);
            const float a = src[c & ~1], b = src[c | 1];
            v = (c & 1) ? (b * cs + a * sn) : (a * cs - b * sn);
        } else {
            v = src[c];
        }
        if (who == 0) lt_store(p.cache, p.cache_dtype, row * D + r + c, v);
        else p.Q[(t * p.heads + (who - 1)) * D + r + c] = v;
    }
}

#define LT_MAXC 16  // latent columns per lane: kv_rank <= 64 * LT_MAXC

__global__ __launch_bounds__(256) void latent_attn_row_kernel(const i64h_latent_attn_args p) {
    extern __shared__ float lds[];  // [4][D] scaled queries, [4][64] weights, [4][64] cache rows
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int64_t t = blockIdx.x;
    const int r = p.kv_rank, D = r + p.rot_dim;
    float* sq = lds + w * D;
    float* sp = lds + 4 * D + w * 64;
    int* srow = (int*)(lds + 4 * D + 256) + w * 64;
    const int h_raw = blockIdx.y * 4 + w;
    const bool active = h_raw < p.heads;
    const int h = active ? h_raw : p.heads - 1;
    const int pos = p.positions[t], slot = p.slot_ids[t];
    const float* q = p.Q + (t * p.heads + h) * D;
    for (int d = lane; d < D; d += 64) sq[d] = q[d] * p.scale;
    __syncthreads();
    const int j0 = p.window > 0 ? max(0, pos - p.window + 1) : 0;
    const int32_t* bt = p.block_table + (int64_t)slot * p.max_blocks_per_seq;
    // the sink: one more score (a learned one per head, or zero) that counts in the denominator and carries no value
    float m = p.sink ? (p.sink_w ? p.sink_w[h] : 0.0f) : -INFINITY, l = p.sink ? 1.0f : 0.0f, acc[LT_MAXC];
#pragma unroll
    for (int i = 0; i < LT_MAXC; ++i) acc[i] = 0.0f;
    for (int jb = j0; jb <= pos; jb += 64) {
        const int j = jb + lane;
        const bool valid = j <= pos;
        const int jj = valid ? j : pos;
        const int64_t rj = (int64_t)bt[jj / p.block_size] * p.block_size + jj % p.block_size;
        float s = 0.0f;
        if (p.cache_dtype == 0) {
            const float* kr = (const float*)p.cache + rj * D;
            if ((D & 3) == 0) {
                for (int d = 0; d < D; d += 4) {
                    const float4 kv = *(const float4*)(kr + d);
                    s += sq[d] * kv.x; s += sq[d + 1] * kv.y; s += sq[d + 2] * kv.z; s += sq[d + 3] * kv.w;
                }
            } else {
                for (int d = 0; d < D; ++d) s += sq[d] * kr[d];
            }
        } else {
            const uint16_t* kr = (const uint16_t*)p.cache + rj * D;
            if ((D & 7) == 0) {
                for (int d = 0; d < D; d += 8) {
                    const uint4 kv = *(const uint4*)(kr + d);
                    const uint32_t kw[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s += sq[d + 2 * i] * __uint_as_float(kw[i] << 16);
                        s += sq[d + 2 * i + 1] * __uint_as_float(kw[i] & 0xffff0000u);
                    }
                }
            } else {
                for (int d = 0; d < D; ++d) s += sq[d] * __uint_as_float((uint32_t)kr[d] << 16);
            }
        }
        if (p.softcap > 0.0f) s = p.softcap * tanhf(s / p.softcap);
        s = valid ? s : -INFINITY;
        const float mn = fmaxf(m, wave_max(s));
        const float alpha = expf(m - mn);
        const float pj = valid ? expf(s - mn) : 0.0f;
        l = l * alpha + wave_sum(pj);
        m = mn;
        __syncthreads();  // the previous block's weights have been read by every lane
        sp[lane] = pj;
        srow[lane] = (int)rj;
        __syncthreads();
        const int cnt = min(64, pos - jb + 1);
#pragma unroll
        for (int i = 0; i < LT_MAXC; ++i) acc[i] *= alpha;
        for (int k = 0; k < cnt; ++k) {
            const float pk = sp[k];
            const int64_t base = (int64_t)srow[k] * D;
#pragma unroll
            for (int i = 0; i < LT_MAXC; ++i) {
                const int c = lane + 64 * i;
                if (c < r) acc[i] += pk * lt_load(p.cache, p.cache_dtype, base + c);
            }
        }
    }
    if (active) {
        float* o = p.out + (t * p.heads + h) * r;
#pragma unroll
        for (int i = 0; i < LT_MAXC; ++i) {
            const int c = lane + 64 * i;
            if (c < r) o[c] = acc[i] / l;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
// Matrix-core form (bf16 cache).  One wave per task of 16 query vectors that walk the same cached rows:
//   head tiles: the (up to) 16 heads of a group of one token  - decode rows, one token per sequence;
//   row tiles : 16 consecutive rows of the step for one head   - portions of prompts; rows of a tile that belong to different
//               sequences are handled run by run (a run's keys are masked for every other row).
// Per tile of 32 keys: scores S[16, 32] = Q K^T on v_mfma_f32_16x16x32_bf16 with the cached rows read straight from memory as B
// fragments (8 consecutive values of one key per lane) and the scaled query carried as TWO bf16 terms (hi + lo, 16 mantissa bits),
// masking and the online softmax in fp32 on the accumulator layout, the weights again as two bf16 terms through LDS into the
// A layout, the tile's latent columns transposed through LDS (4 keys x 8 columns per lane and pass, 8-byte writes) into the B
// layout of the second product, out[16, kv_rank] += P V in fp32.  Every product of two bf16 values is exact in fp32.
#define LT_KD 10   // 32-wide steps over a cached row: kv_rank + rot_dim <= 320
#define LT_NB 16   // 16-column blocks of the output: kv_rank <= 256
#define LT_VLD 40  // halves per row of the transposed tile and of the weight planes (32 keys + 8: 16-byte aligned, conflict-poor)
typedef __bf16 lt_v8bf __attribute__((ext_vector_type(8)));
typedef float lt_v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t lt_rne(float f) {  // nearest even: the hardware conversion of this chip
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ void lt_split(float x, uint32_t& hi, uint32_t& lo) {
    hi = lt_rne(x);
    lo = lt_rne(x - __uint_as_float(hi << 16));
}

// KD, NB: 32-wide steps over a cached row and 16-column blocks of the output that the instance holds registers for (rows of at most
// 32 KD values, kv_rank <= 16 NB): the widest instance keeps two waves per SIMD, narrow rows leave room for more.
template <int KD, int NB>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2, KD > 4 ? 2 : 8))) void latent_attn_mfma_kernel(const i64h_latent_attn_args p, const int row_tiles, const int splits) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x, n = lane & 15, kg = lane >> 4;
    const int r = p.kv_rank, D = r + p.rot_dim, H = p.heads, bs = p.block_size, win = p.window;
    uint16_t* Vt = (uint16_t*)smem;           // [r][LT_VLD]
    uint16_t* Ph = Vt + r * LT_VLD;           // [16][LT_VLD]
    uint16_t* Pl = Ph + 16 * LT_VLD;
    int* info = (int*)(Pl + 16 * LT_VLD);     // [16] positions, [16] slots (-1: no such row), [32] cache rows of the tile's keys
    int* rowoff = info + 32;
    const int64_t task = blockIdx.x;
    const int split = blockIdx.y;
    // key heads side by side in a cached row (key-valued attention): a head tile takes 16 of the rep query heads of ONE key head
    const int G = p.kv_groups > 1 ? p.kv_groups : 1, rep = H / G, tpg = (rep + 15) / 16;
    const int hgroups = G * tpg;
    const int rstride = p.row_stride > 0 ? p.row_stride : D;
    const int coff = (row_tiles ? (int)(task % H) / rep : (int)(task % hgroups) / tpg) * D;
    const int hbase = row_tiles ? (int)(task % H) : ((int)(task % hgroups) / tpg) * rep + ((int)(task % hgroups) % tpg) * 16;
    auto row_of = [&](int m, int64_t& tok, int& head) -> bool {
        if (row_tiles) {     // the heads of a row tile are neighbours in the launch: they walk the same cached rows at the same time
            tok = (task / H) * 16 + m;
            head = hbase;
            return tok < p.n;
        }
        tok = task / hgroups;
        head = hbase + m;
        return ((int)(task % hgroups) % tpg) * 16 + m < rep;
    };
    int64_t tok_n;
    int head_n;
    const bool valid_n = row_of(n, tok_n, head_n);
    if (lane < 16) {
        info[lane] = valid_n ? p.positions[tok_n] : -1;
        info[16 + lane] = valid_n ? p.slot_ids[tok_n] : -1;
    }
    // the query of row n times scale * log2(e) (the softmax runs on powers of two), columns ks * 32 + kg * 8 .. + 7, as two bf16 terms
    uint4 Qh[KD], Ql[KD];
    {
        const float* q = p.Q + (tok_n * H + head_n) * D;
        const float qs = p.scale * 1.4426950408889634f;
#pragma unroll
        for (int ks = 0; ks < KD; ++ks) {
            const int d0 = ks * 32 + kg * 8;
            uint32_t h[8], l[8];
            if (valid_n && d0 < D) {
                const float4 a = *(const float4*)(q + d0), b = *(const float4*)(q + d0 + 4);
                const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
                for (int i = 0; i < 8; ++i) lt_split(v[i] * qs, h[i], l[i]);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = l[i] = 0;
            }
            Qh[ks] = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
            Ql[ks] = make_uint4(l[0] | (l[1] << 16), l[2] | (l[3] << 16), l[4] | (l[5] << 16), l[6] | (l[7] << 16));
        }
    }
    lt_v4f acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = lt_v4f{0, 0, 0, 0};
    float mrow[4], lrow[4];
    int lor[4], hrow[4];   // per row of the tile: the first position it sees, its head (for the bias table)
    const bool sink = p.sink && split == 0;     // the extra score of zero counts once: in the first share of the keys
    __syncthreads();
    const float capl = p.softcap * 1.4426950408889634f;     // the cap in the units of the scores (powers of two)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int pp = info[kg * 4 + g];
        lor[g] = p.chunk > 0 ? (max(pp, 0) / p.chunk) * p.chunk : (win > 0 ? max(0, pp - win + 1) : 0);
        hrow[g] = min(row_tiles ? hbase : hbase + kg * 4 + g, H - 1);
        mrow[g] = sink ? (p.sink_w ? p.sink_w[hrow[g]] * 1.4426950408889634f : 0.0f) : -INFINITY;
        lrow[g] = sink ? 1.0f : 0.0f;
    }
    const uint16_t* cache = (const uint16_t*)p.cache;
    int s0 = 0;
    while (s0 < 16) {
        const int sl = info[16 + s0];
        if (sl < 0) {
            ++s0;
            continue;
        }
        int s1 = s0 + 1;
        while (s1 < 16 && info[16 + s1] == sl) ++s1;
        int lo = 0x7fffffff, hi = -1;
        for (int i = s0; i < s1; ++i) {
            const int pp = info[i];
            hi = max(hi, pp);
            lo = min(lo, p.chunk > 0 ? (pp / p.chunk) * p.chunk : (win > 0 ? max(0, pp - win + 1) : 0));
        }
        const int32_t* bt = p.block_table + (int64_t)sl * p.max_blocks_per_seq;
        for (int kb = (lo & ~31) + 32 * split; kb <= hi; kb += 32 * splits) {
            if (lane < 32) {
                const int jc = min(kb + lane, hi);
                rowoff[lane] = bt[jc / bs] * bs + jc % bs;
            }
            __syncthreads();
            lt_v4f S[2];
            float ksc[2] = {1.0f, 1.0f};
            if (p.kscale) {
                ksc[0] = p.kscale[rowoff[n]];
                ksc[1] = p.kscale[rowoff[16 + n]];
            }
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                S[b] = lt_v4f{0, 0, 0, 0};
                const uint16_t* rowp = cache + (int64_t)rowoff[16 * b + n] * rstride + coff;
#pragma unroll
                for (int ks = 0; ks < KD; ++ks) {
                    if (ks * 32 < D) {
                        const int d0 = ks * 32 + kg * 8;
                        const uint4 kf = d0 < D ? *(const uint4*)(rowp + d0) : make_uint4(0, 0, 0, 0);
                        if ((ks + 1) * 32 > p.key_off) {     // (a step of value-only columns: the query is zero there)
                            S[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lt_v8bf, Qh[ks]), __builtin_bit_cast(lt_v8bf, kf), S[b], 0, 0, 0);
                            S[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lt_v8bf, Ql[ks]), __builtin_bit_cast(lt_v8bf, kf), S[b], 0, 0, 0);
                        }
                        if (d0 < r) {   // the same registers, transposed, are the second product's operand: column d0 + c of key 16 b + n
                            const uint32_t kw[4] = {kf.x, kf.y, kf.z, kf.w};
#pragma unroll
                            for (int c = 0; c < 8; ++c) Vt[(d0 + c) * LT_VLD + 16 * b + n] = (uint16_t)(kw[c >> 1] >> (16 * (c & 1)));
                        }
                    }
                }
            }
            float al[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int rr = kg * 4 + g;
                const int pr = info[rr];
                const bool in_run = rr >= s0 && rr < s1;
                float sv[2];
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    const int j = kb + 16 * b + n;
                    const bool vis = in_run && j <= pr && j >= lor[g];
                    float sc = S[b][g] * ksc[b];
                    if (capl > 0.0f) sc = capl * tanhf(sc / capl);
                    if (p.bias) sc += 1.4426950408889634f * p.bias[(int64_t)min(max(pr - j, 0), p.bias_rows - 1) * H + hrow[g]];
                    sv[b] = vis ? sc : -INFINITY;
                }
                const float mx = row16_max(fmaxf(sv[0], sv[1]));
                const float mn = fmaxf(mrow[g], mx);
                const float ms = mn == -INFINITY ? 0.0f : mn;
                al[g] = __builtin_amdgcn_exp2f(mrow[g] - ms);
                const float p0 = __builtin_amdgcn_exp2f(sv[0] - ms), p1 = __builtin_amdgcn_exp2f(sv[1] - ms);
                lrow[g] = lrow[g] * al[g] + group_sum(p0 + p1, 16);
                mrow[g] = mn;
                uint32_t h0, l0, h1, l1;
                lt_split(p0, h0, l0);
                lt_split(p1, h1, l1);
                Ph[rr * LT_VLD + n] = (uint16_t)h0;
                Pl[rr * LT_VLD + n] = (uint16_t)l0;
                Ph[rr * LT_VLD + 16 + n] = (uint16_t)h1;
                Pl[rr * LT_VLD + 16 + n] = (uint16_t)l1;
            }
            __syncthreads();
            const uint4 pah = *(const uint4*)&Ph[n * LT_VLD + kg * 8], pal = *(const uint4*)&Pl[n * LT_VLD + kg * 8];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                if (nb * 16 < r) {
                    const uint4 vf = *(const uint4*)&Vt[(nb * 16 + n) * LT_VLD + kg * 8];
#pragma unroll
                    for (int g = 0; g < 4; ++g) acc[nb][g] *= al[g];
                    acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lt_v8bf, pah), __builtin_bit_cast(lt_v8bf, vf), acc[nb], 0, 0, 0);
                    acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lt_v8bf, pal), __builtin_bit_cast(lt_v8bf, vf), acc[nb], 0, 0, 0);
                }
            }
            __syncthreads();
        }
        s0 = s1;
    }
    if (splits > 1) {
        // partial result of this share of the keys: [16 rows][kv_rank unnormalised sums | maximum (log2 units) | sum of weights]
        float* w = p.workspace + ((int64_t)task * splits + split) * 16 * (r + 2);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float* o = w + (kg * 4 + g) * (r + 2);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
                if (nb * 16 < r) o[nb * 16 + n] = acc[nb][g];
            if (n == 0) {
                o[r] = mrow[g];
                o[r + 1] = lrow[g];
            }
        }
        return;
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        int64_t tok;
        int head;
        if (!row_of(kg * 4 + g, tok, head)) continue;
        float* o = p.out + (tok * H + head) * r;
        const float inv = 1.0f / lrow[g];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
            if (nb * 16 < r) o[nb * 16 + n] = acc[nb][g] * inv;
    }
}

// The same products for rows that are one per sequence (every wave: one token, 16 heads, a share of the keys), arranged around the
// memory latency that dominates such launches: a tile's 18 fragment loads are requested together, the NEXT tile's are requested as
// soon as this tile's scores and transposed columns are done - under its softmax and second product - and the cache rows of the tile
// after that are looked up a tile ahead.  The workgroup is one wave, so LDS traffic needs program order only (no barrier, whose
// fence would wait for the loads in flight).  Registers: a whole SIMD's (one wave per SIMD is all such a launch has anyway).
template <int KD, int NB>
__global__ __launch_bounds__(64) void latent_attn_mfma_decode_kernel(const i64h_latent_attn_args p, const int splits) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x, n = lane & 15, kg = lane >> 4;
    const int r = p.kv_rank, D = r + p.rot_dim, H = p.heads, bs = p.block_size, win = p.window;
    uint16_t* Vt = (uint16_t*)smem;
    uint16_t* Ph = Vt + r * LT_VLD;
    uint16_t* Pl = Ph + 16 * LT_VLD;
    int* rowoff = (int*)(Pl + 16 * LT_VLD);   // [2][32] cache rows of two tiles' keys
    const int64_t task = blockIdx.x;
    const int split = blockIdx.y;
    const int G = p.kv_groups > 1 ? p.kv_groups : 1, rep = H / G, tpg = (rep + 15) / 16;
    const int hgroups = G * tpg;
    const int64_t tok = task / hgroups;
    const int sub = (int)(task % hgroups);
    const int hin = (sub % tpg) * 16;               // first of this wave's heads within its key head
    const int head0 = (sub / tpg) * rep + hin;
    const int rstride = p.row_stride > 0 ? p.row_stride : D;
    const int coff = (sub / tpg) * D;
    const int pos = p.positions[tok], slot = p.slot_ids[tok];
    const int lo = p.chunk > 0 ? (pos / p.chunk) * p.chunk : (win > 0 ? max(0, pos - win + 1) : 0), hi = pos;
    const int32_t* bt = p.block_table + (int64_t)slot * p.max_blocks_per_seq;
    const uint16_t* cache = (const uint16_t*)p.cache;
    const int step = 32 * splits;
    const int kb0 = (lo & ~31) + 32 * split;
    auto lookup = [&](int kb, int buf) {
        if (lane < 32) {
            const int jc = min(kb + lane, hi);
            rowoff[buf * 32 + lane] = bt[jc / bs] * bs + jc % bs;
        }
    };
    uint4 kf[2][KD];
    auto request = [&](int buf) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const uint16_t* rowp = cache + (int64_t)rowoff[buf * 32 + 16 * b + n] * rstride + coff;
#pragma unroll
            for (int ks = 0; ks < KD; ++ks) {
                const int d0 = ks * 32 + kg * 8;
                kf[b][ks] = (ks * 32 < D && d0 < D) ? *(const uint4*)(rowp + d0) : make_uint4(0, 0, 0, 0);
            }
        }
    };
    if (kb0 <= hi) {
        lookup(kb0, 0);
        if (kb0 + step <= hi) lookup(kb0 + step, 1);
        __builtin_amdgcn_wave_barrier();
        request(0);
    }
    // the query of row n (head head0 + n) times scale * log2(e), as two bf16 terms - converted while the first tile travels
    uint4 Qh[KD], Ql[KD];
    {
        const bool valid_n = hin + n < rep;
        const float* q = p.Q + (tok * H + head0 + n) * D;
        const float qs = p.scale * 1.4426950408889634f;
#pragma unroll
        for (int ks = 0; ks < KD; ++ks) {
            const int d0 = ks * 32 + kg * 8;
            uint32_t h[8], l[8];
            if (valid_n && d0 < D) {
                const float4 a = *(const float4*)(q + d0), b = *(const float4*)(q + d0 + 4);
                const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
                for (int i = 0; i < 8; ++i) lt_split(v[i] * qs, h[i], l[i]);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = l[i] = 0;
            }
            Qh[ks] = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
            Ql[ks] = make_uint4(l[0] | (l[1] << 16), l[2] | (l[3] << 16), l[4] | (l[5] << 16), l[6] | (l[7] << 16));
        }
    }
    lt_v4f acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = lt_v4f{0, 0, 0, 0};
    float mrow[4], lrow[4];
    int hrow[4];
    const bool sink = p.sink && split == 0;     // the extra score of zero counts once: in the first share of the keys
    const float capl = p.softcap * 1.4426950408889634f;     // the cap in the units of the scores (powers of two)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        hrow[g] = min(head0 + kg * 4 + g, H - 1);
        mrow[g] = sink ? (p.sink_w ? p.sink_w[hrow[g]] * 1.4426950408889634f : 0.0f) : -INFINITY;
        lrow[g] = sink ? 1.0f : 0.0f;
    }
    int it = 0;
    for (int kb = kb0; kb <= hi; kb += step, ++it) {
        const int cur = it & 1;
        lt_v4f S[2];
        float ksc[2] = {1.0f, 1.0f};
        if (p.kscale) {
            ksc[0] = p.kscale[rowoff[cur * 32 + n]];
            ksc[1] = p.kscale[rowoff[cur * 32 + 16 + n]];
        }
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            S[b] = lt_v4f{0, 0, 0, 0};
#pragma unroll
            for (int ks = 0; ks < KD; ++ks) {
                if (ks * 32 < D) {
                    const int d0 = ks * 32 + kg * 8;
                    const uint4 f = kf[b][ks];
                    if ((ks + 1) * 32 > p.key_off) {     // (a step of value-only columns: the query is zero there)
                        S[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lt_v8bf, Qh[ks]), __builtin_bit_cast(lt_v8bf, f), S[b], 0, 0, 0);
                        S[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lt_v8bf, Ql[ks]), __builtin_bit_cast(lt_v8bf, f), S[b], 0, 0, 0);
                    }
                    if (d0 < r) {
                        const uint32_t kw[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
                        for (int c = 0; c < 8; ++c) Vt[(d0 + c) * LT_VLD + 16 * b + n] = (uint16_t)(kw[c >> 1] >> (16 * (c & 1)));
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (kb + step <= hi) request(cur ^ 1);          // the next tile travels under this tile's softmax and second product
        float al[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int rr = kg * 4 + g;
            float sv[2];
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const int j = kb + 16 * b + n;
                float sc = S[b][g] * ksc[b];
                if (capl > 0.0f) sc = capl * tanhf(sc / capl);
                if (p.bias) sc += 1.4426950408889634f * p.bias[(int64_t)min(max(pos - j, 0), p.bias_rows - 1) * H + hrow[g]];
                sv[b] = (j <= pos && j >= lo) ? sc : -INFINITY;
            }
            const float mx = row16_max(fmaxf(sv[0], sv[1]));
            const float mn = fmaxf(mrow[g], mx);
            const float ms = mn == -INFINITY ? 0.0f : mn;
            al[g] = __builtin_amdgcn_exp2f(mrow[g] - ms);
            const float p0 = __builtin_amdgcn_exp2f(sv[0] - ms), p1 = __builtin_amdgcn_exp2f(sv[1] - ms);
            lrow[g] = lrow[g] * al[g] + group_sum(p0 + p1, 16);
            mrow[g] = mn;
            uint32_t h0, l0, h1, l1;
            lt_split(p0, h0, l0);
            lt_split(p1, h1, l1);
            Ph[rr * LT_VLD + n] = (uint16_t)h0;
            Pl[rr * LT_VLD + n] = (uint16_t)l0;
            Ph[rr * LT_VLD + 16 + n] = (uint16_t)h1;
            Pl[rr * LT_VLD + 16 + n] = (uint16_t)l1;
        }
        __builtin_amdgcn_wave_barrier();
        const uint4 pah = *(const uint4*)&Ph[n * LT_VLD + kg * 8], pal = *(const uint4*)&Pl[n * LT_VLD + kg * 8];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            if (nb * 16 < r) {
                const uint4 vf = *(const uint4*)&Vt[(nb * 16 + n) * LT_VLD + kg * 8];
#pragma unroll
                for (int g = 0; g < 4; ++g) acc[nb][g] *= al[g];
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lt_v8bf, pah), __builtin_bit_cast(lt_v8bf, vf), acc[nb], 0, 0, 0);
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lt_v8bf, pal), __builtin_bit_cast(lt_v8bf, vf), acc[nb], 0, 0, 0);
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (kb + 2 * step <= hi) lookup(kb + 2 * step, cur);   // rows of the tile after next, into the buffer this tile is done with
    }
    if (splits > 1) {
        float* w = p.workspace + ((int64_t)task * splits + split) * 16 * (r + 2);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float* o = w + (kg * 4 + g) * (r + 2);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
                if (nb * 16 < r) o[nb * 16 + n] = acc[nb][g];
            if (n == 0) {
                o[r] = mrow[g];
                o[r + 1] = lrow[g];
            }
        }
        return;
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int head = head0 + kg * 4 + g;
        if (hin + kg * 4 + g >= rep) continue;
        float* o = p.out + (tok * H + head) * r;
        const float inv = 1.0f / lrow[g];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
            if (nb * 16 < r) o[nb * 16 + n] = acc[nb][g] * inv;
    }
}

// the shares of a token's keys, merged: one wave per (token, head); lane s holds share s's maximum and weight sum (at most 64
// shares), then every lane sums its columns over the shares, eight loads in flight at a time
__global__ __launch_bounds__(64) void latent_attn_merge_kernel(const i64h_latent_attn_args p, const int splits) {
    __shared__ float sf[64];
    const int lane = threadIdx.x;
    const int r = p.kv_rank, H = p.heads;
    const int G = p.kv_groups > 1 ? p.kv_groups : 1, rep = H / G, tpg = (rep + 15) / 16;
    const int hgroups = G * tpg;
    const int64_t task = blockIdx.x, tok = task / hgroups;
    const int m = blockIdx.y;
    const int sub = (int)(task % hgroups);
    if ((sub % tpg) * 16 + m >= rep) return;
    const int head = (sub / tpg) * rep + (sub % tpg) * 16 + m;
    const float* w = p.workspace + (task * splits * 16 + m) * (r + 2);      // share s: + s * 16 * (r + 2)
    const int64_t stride = (int64_t)16 * (r + 2);
    const float* mine = w + (int64_t)min(lane, splits - 1) * stride;
    const float ms = lane < splits ? mine[r] : -INFINITY, ls = lane < splits ? mine[r + 1] : 0.0f;
    const float mx = wave_max(ms);
    const float f = __builtin_amdgcn_exp2f(ms - mx);      // share `lane`'s factor (0 for an empty share)
    const float den = wave_sum(f * ls);
    sf[lane] = lane < splits ? f : 0.0f;
    __syncthreads();
    for (int c = lane; c < r; c += 64) {
        float num = 0.0f;
        for (int s0 = 0; s0 < splits; s0 += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = s0 + u < splits ? w[(int64_t)(s0 + u) * stride + c] : 0.0f;
#pragma unroll
            for (int u = 0; u < 8; ++u) num += sf[(s0 + u) & 63] * v[u];
        }
        p.out[(tok * H + head) * r + c] = num / den;
    }
}

extern "C" {

int i64h_latent_prep(const i64h_latent_prep_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "latent_prep: no descriptor");
    const i64h_latent_prep_args& d = *dp;
    I64H_CHECK_ARG(d.n >= 0 && d.heads > 0 && d.dim > 0 && d.rot_dim >= 0 && d.kv_rank > 0 && d.block_size > 0, "latent_prep: bad sizes");
    I64H_CHECK_ARG(d.rot_dims >= 0 && d.rot_dims <= d.rot_dim && d.rot_dims % 2 == 0, "latent_prep: %d rotated dimensions of %d", d.rot_dims, d.rot_dim);
    I64H_CHECK_ARG(d.cache_dtype == 0 || d.cache_dtype == 2, "latent_prep: cache dtype %d", d.cache_dtype);
    I64H_CHECK_ARG(d.P && d.c_norm_w && d.positions && d.slot_ids && d.block_table && d.cache && d.Q && (d.inv_freq || d.rot_dims == 0), "latent_prep: null operand");
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(latent_prep_kernel, dim3((unsigned)d.n), dim3(256), 0, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

static int g_decode_form = 1;
int i64h_set_latent_attn_decode_form(int32_t on) {  // tuning / test knob: 0 = rows that are one per sequence on the general matrix-core kernel
    g_decode_form = on;
    return 0;
}

int64_t i64h_latent_attn_workspace_floats(int64_t n, int32_t heads, int32_t kv_rank, int32_t splits) {
    if (splits <= 1) return 0;
    return n * ((heads + 15) / 16) * (int64_t)(splits > 64 ? 64 : splits) * 16 * (kv_rank + 2);
}

int i64h_latent_attn(const i64h_latent_attn_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "latent_attn: no descriptor");
    const i64h_latent_attn_args& d = *dp;
    I64H_CHECK_ARG(d.n >= 0 && d.heads > 0 && d.kv_rank > 0 && d.rot_dim >= 0 && d.block_size > 0, "latent_attn: bad sizes");
    I64H_CHECK_ARG(d.kv_rank <= 64 * LT_MAXC, "latent_attn: kv_rank %d above %d", d.kv_rank, 64 * LT_MAXC);
    I64H_CHECK_ARG(d.cache_dtype == 0 || d.cache_dtype == 2, "latent_attn: cache dtype %d", d.cache_dtype);
    I64H_CHECK_ARG(d.Q && d.cache && d.block_table && d.slot_ids && d.positions && d.out, "latent_attn: null operand");
    I64H_CHECK_ARG(d.key_off >= 0 && d.key_off <= d.kv_rank, "latent_attn: %d value-only columns of %d value columns", d.key_off, d.kv_rank);
    if (d.n == 0) return 0;
    const int D = d.kv_rank + d.rot_dim;
    const bool mfma_ok = d.cache_dtype == 2 && D % 8 == 0 && d.kv_rank % 16 == 0 && d.kv_rank <= 16 * LT_NB && D <= 32 * LT_KD &&
                         (uintptr_t)d.Q % 16 == 0 && (uintptr_t)d.cache % 16 == 0 && d.row_stride % 8 == 0;
    I64H_CHECK_ARG(mfma_ok || (d.kv_groups <= 1 && d.row_stride <= 0 && d.chunk <= 0 && !d.kscale && !d.bias),
                   "latent_attn: key heads, chunks, key scales and bias are built for the matrix-core form only");
    I64H_CHECK_ARG(!d.sink_w || d.sink, "latent_attn: sink scores without the sink");
    if (d.mode != 1 && mfma_ok) {
        const int row_tiles = d.mode == 3;
        const int G = d.kv_groups > 1 ? d.kv_groups : 1;
        I64H_CHECK_ARG(d.heads % G == 0, "latent_attn: %d heads over %d key heads", d.heads, G);
        const int64_t tasks = row_tiles ? (d.n + 15) / 16 * d.heads : d.n * G * ((d.heads / G + 15) / 16);
        I64H_CHECK_ARG(tasks < (1ll << 31), "latent_attn: too many tiles");
        const int splits = (!row_tiles && d.workspace && d.splits > 1) ? (d.splits > 64 ? 64 : d.splits) : 1;
        const size_t bytes = (size_t)d.kv_rank * LT_VLD * 2 + 2 * 16 * LT_VLD * 2 + 64 * 4;
        const dim3 grid((unsigned)tasks, (unsigned)splits);
        hipStream_t st = (hipStream_t)stream;
        const int size = (D <= 64 && d.kv_rank <= 64) ? 0 : ((D <= 128 && d.kv_rank <= 128) ? 1 : 2);     // the narrowest instance that holds the rows
        if (row_tiles || !g_decode_form) {
            if (size == 0) hipLaunchKernelGGL((latent_attn_mfma_kernel<2, 4>), grid, dim3(64), bytes, st, d, row_tiles, splits);
            else if (size == 1) hipLaunchKernelGGL((latent_attn_mfma_kernel<4, 8>), grid, dim3(64), bytes, st, d, row_tiles, splits);
            else hipLaunchKernelGGL((latent_attn_mfma_kernel<LT_KD, LT_NB>), grid, dim3(64), bytes, st, d, row_tiles, splits);
        } else {
            if (size == 0) hipLaunchKernelGGL((latent_attn_mfma_decode_kernel<2, 4>), grid, dim3(64), bytes, st, d, splits);
            else if (size == 1) hipLaunchKernelGGL((latent_attn_mfma_decode_kernel<4, 8>), grid, dim3(64), bytes, st, d, splits);
            else hipLaunchKernelGGL((latent_attn_mfma_decode_kernel<LT_KD, LT_NB>), grid, dim3(64), bytes, st, d, splits);
        }
        I64H_CHECK_LAUNCH();
        if (splits > 1) {
            hipLaunchKernelGGL(latent_attn_merge_kernel, dim3((unsigned)tasks, 16), dim3(64), 0, (hipStream_t)stream, d, splits);
            I64H_CHECK_LAUNCH();
        }
        return 0;
    }
    const size_t lds = (size_t)(4 * D + 512) * 4;
    I64H_CHECK_ARG(lds <= 64 * 1024, "latent_attn: cached rows of %d values do not fit", D);
    hipLaunchKernelGGL(latent_attn_row_kernel, dim3((unsigned)d.n, (unsigned)((d.heads + 3) / 4)), dim3(256), lds, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"
