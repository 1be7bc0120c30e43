// Kernels of libi64hip_dense.so for gated linear recurrences and mixtures of experts (include/i64h_dense.h):
//   gla_gates_kernel   : query activation and bounded forget gate, in place on the projection rows
//   gla_scan_kernel    : linear attention with a decay per key channel, a head's matrix in registers (16 lanes per value column)
//   gdn_gates_kernel / gdn_scan_kernel : gated delta rule - unit-vector queries and keys, write strength and decay; the recurrence with the
//                        correction S^T k summed over the DPP row before the write, the read-out after it
//   route_topk_kernel  : softmax scores, corrected choice, groups of neighbours, top-k and normalised weights, one wave per row
//   moe_plan_kernel    : (token, choice) pairs grouped by expert: offsets, the token of every grouped row, the row of every pair
//   moe_combine_kernel : weighted sum of the chosen experts' rows, pass-through entries and the shared expert's row
// A row continues the row before it iff slot and position say so; state is taken as empty at position 0.  All arithmetic fp32.
#include "i64h_common.h"
#include "i64h_dense.h"

__device__ __forceinline__ float bl_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

// ---------------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gla_gates_kernel(const i64h_gla_args p) {
    const int64_t t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= p.heads * p.dim) return;
    float* row = p.P + t * p.ldp;
    if (p.q_act) {
        const float q = row[p.q_off + c];
        row[p.q_off + c] = q * bl_sigmoid(q);
    }
    const float lo = p.lower ? p.lower[c] : 0.0f;
    row[p.f_off + c] = lo + (1.0f - lo) * bl_sigmoid(row[p.f_off + c]);
}

// One workgroup per (head, 16 * CPT value columns, run of rows).  The 16 lanes of a DPP row share CPT neighbouring value columns and hold
// KPT consecutive key channels of each in registers; a wave has four such rows.  Per token a lane loads its slices of the query, the
// decay and (where it is not one minus the decay) the key once for its CPT columns, updates its states with fused multiply-adds and
// the row sums the partial outputs with DPP moves: no LDS and no barrier, the tokens of a run strictly in their order (the same sums in
// the same order however a prompt is cut).  Loads run GL_TG tokens ahead in two alternating register sets, so that a wave that is alone
// on its SIMD still has a group of tokens in flight while it computes one.  State layout [slot, head, value column, key channel].
#define GL_TG 4
template <int KPT, int CPT, bool HASK>
__global__ __launch_bounds__(256) void gla_scan_kernel(const i64h_gla_args p, const int ctiles, const int vec) {
    const int N = p.dim, P = p.vdim;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int nlane = lane & 15, cl = lane >> 4;
    const int a = blockIdx.x / ctiles, seg = blockIdx.y;
    const int cbase = (blockIdx.x % ctiles) * 16 * CPT + (w * 4 + cl) * CPT;
    const int64_t r0 = p.seg_start[seg], r1 = p.seg_start[seg + 1];
    if (r1 <= r0) return;
    const int n0 = nlane * KPT;
    float S[CPT][KPT];
    float* gS = p.state + ((int64_t)p.slot_ids[r0] * p.heads + a) * P * N + n0;      // + column * N
    const bool fresh = p.positions[r0] == 0;
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
        const bool cok = cbase + j < P;
        const float* src = gS + (int64_t)(cok ? cbase + j : 0) * N;
#pragma unroll
        for (int k = 0; k < KPT; ++k) S[j][k] = 0.0f;
        if (!fresh && cok) {
            if (vec) {
#pragma unroll
                for (int k = 0; k < KPT; k += 4)
                    if (n0 + k < N) {
                        const float4 v = *(const float4*)(src + k);
                        S[j][k] = v.x, S[j][k + 1] = v.y, S[j][k + 2] = v.z, S[j][k + 3] = v.w;
                    }
            } else {
#pragma unroll
                for (int k = 0; k < KPT; ++k)
                    if (n0 + k < N) S[j][k] = src[k];
            }
        }
    }
    const int qoff = p.q_off + a * N + n0, foff = p.f_off + a * N + n0, koff = HASK ? p.k_off + a * N + n0 : 0;
    struct Tok {
        float q[KPT], f[KPT], k[HASK ? KPT : 1], v[CPT];
    };
    auto fetch = [&](int64_t t, Tok& u) {
        if (t >= r1) return;
        const float* row = p.P + t * p.ldp;
        if (vec) {      // KPT % 4 == 0 and every slice starts at a multiple of four floats and lies inside the row
#pragma unroll
            for (int k = 0; k < KPT; k += 4) {
                float4 q = make_float4(0, 0, 0, 0), f = make_float4(1, 1, 1, 1), kk = q;
                if (n0 + k < N) {
                    q = *(const float4*)(row + qoff + k);
                    f = *(const float4*)(row + foff + k);
                    if (HASK) kk = *(const float4*)(row + koff + k);
                }
                u.q[k] = q.x, u.q[k + 1] = q.y, u.q[k + 2] = q.z, u.q[k + 3] = q.w;
                u.f[k] = f.x, u.f[k + 1] = f.y, u.f[k + 2] = f.z, u.f[k + 3] = f.w;
                if (HASK) u.k[k] = kk.x, u.k[k + 1] = kk.y, u.k[k + 2] = kk.z, u.k[k + 3] = kk.w;
            }
        } else {
#pragma unroll
            for (int k = 0; k < KPT; ++k) {
                const bool ok = n0 + k < N;
                u.q[k] = ok ? row[qoff + k] : 0.0f;
                u.f[k] = ok ? row[foff + k] : 1.0f;
                if (HASK) u.k[k] = ok ? row[koff + k] : 0.0f;
            }
        }
#pragma unroll
        for (int j = 0; j < CPT; ++j) u.v[j] = cbase + j < P ? row[p.v_off + a * P + cbase + j] : 0.0f;
    };
    auto step = [&](int64_t t, const Tok& u) {
        if (t >= r1) return;
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
            float part = 0.0f;
#pragma unroll
            for (int k = 0; k < KPT; ++k) {
                const float kk = HASK ? u.k[k] : 1.0f - u.f[k];
                S[j][k] = fmaf(u.f[k], S[j][k], kk * u.v[j]);
                part = fmaf(S[j][k], u.q[k], part);
            }
            part = group_sum(part, 16);
            if (nlane == 0 && cbase + j < P) p.out[t * p.ldo + a * P + cbase + j] = part;
        }
    };
    Tok A[GL_TG], B[GL_TG];
#pragma unroll
    for (int i = 0; i < GL_TG; ++i) fetch(r0 + i, A[i]);
    for (int64_t t = r0; t < r1; t += 2 * GL_TG) {
#pragma unroll
        for (int i = 0; i < GL_TG; ++i) fetch(t + GL_TG + i, B[i]);
#pragma unroll
        for (int i = 0; i < GL_TG; ++i) step(t + i, A[i]);
#pragma unroll
        for (int i = 0; i < GL_TG; ++i) fetch(t + 2 * GL_TG + i, A[i]);
#pragma unroll
        for (int i = 0; i < GL_TG; ++i) step(t + GL_TG + i, B[i]);
    }
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
        if (cbase + j >= P) continue;
        float* dst = gS + (int64_t)(cbase + j) * N;
        if (vec) {
#pragma unroll
            for (int k = 0; k < KPT; k += 4)
                if (n0 + k < N) *(float4*)(dst + k) = make_float4(S[j][k], S[j][k + 1], S[j][k + 2], S[j][k + 3]);
        } else {
#pragma unroll
            for (int k = 0; k < KPT; ++k)
                if (n0 + k < N) dst[k] = S[j][k];
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
// Gated delta rule.  gdn_gates_kernel: one workgroup per token - a wave per query / key head makes the head a unit vector in place (the
// query also scaled), and the first threads turn the raw gate projections into the write strength and the decay of every head.
__device__ __forceinline__ float bl_softplus(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

__global__ __launch_bounds__(256) void gdn_gates_kernel(const i64h_gdn_args p) {
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    float* row = p.X + t * p.ldx;
    if (p.unit_eps >= 0.0f || p.q_scale != 1.0f) {
        for (int u = wid; u < 2 * p.kv_heads; u += 4) {
            const bool isq = u < p.kv_heads;
            float* x = row + (isq ? p.q_off + u * p.dim : p.k_off + (u - p.kv_heads) * p.dim);
            float s = 0.0f;
            for (int d = lane; d < p.dim; d += 64) s += x[d] * x[d];
            s = wave_sum(s);
            float f = p.unit_eps >= 0.0f ? 1.0f / sqrtf(s + p.unit_eps) : 1.0f;
            if (isq) f *= p.q_scale;
            for (int d = lane; d < p.dim; d += 64) x[d] *= f;
        }
    }
    for (int a = threadIdx.x; a < p.heads; a += 256) {
        const float* r = p.R + t * p.ldr;
        p.G[t * 2 * p.heads + a] = bl_sigmoid(r[p.b_off + a]);
        p.G[t * 2 * p.heads + p.heads + a] = expf(-expf(p.A_log[a]) * bl_softplus(r[p.a_off + a] + p.dt_bias[a]));
    }
}

// gdn_scan_kernel: the layout of gla_scan_kernel (one workgroup per (head, 16 * CPT value columns, run of rows); the 16 lanes of a DPP
// row share CPT value columns and hold KPT key channels of each in registers).  Per token the state decays, the row sums S^T k with DPP
// moves (every lane of the row ends with the sum), the correction along k is written, and a second row sum reads the state out with
// the query - after the write.  No LDS and no barrier, the tokens of a run strictly in their order; loads run GL_TG tokens ahead.
template <int KPT, int CPT>
__global__ __launch_bounds__(256) void gdn_scan_kernel(const i64h_gdn_args p, const int ctiles, const int vec) {
    const int N = p.dim, P = p.vdim;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int nlane = lane & 15, cl = lane >> 4;
    const int a = blockIdx.x / ctiles, seg = blockIdx.y;
    const int kh = a / (p.heads / p.kv_heads);
    const int cbase = (blockIdx.x % ctiles) * 16 * CPT + (w * 4 + cl) * CPT;
    const int64_t r0 = p.seg_start[seg], r1 = p.seg_start[seg + 1];
    if (r1 <= r0) return;
    const int n0 = nlane * KPT;
    float S[CPT][KPT];
    float* gS = p.state + ((int64_t)p.slot_ids[r0] * p.heads + a) * P * N + n0;      // + column * N
    const bool fresh = p.positions[r0] == 0;
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
        const bool cok = cbase + j < P;
        const float* src = gS + (int64_t)(cok ? cbase + j : 0) * N;
#pragma unroll
        for (int k = 0; k < KPT; ++k) S[j][k] = 0.0f;
        if (!fresh && cok) {
            if (vec) {
#pragma unroll
                for (int k = 0; k < KPT; k += 4)
                    if (n0 + k < N) {
                        const float4 v = *(const float4*)(src + k);
                        S[j][k] = v.x, S[j][k + 1] = v.y, S[j][k + 2] = v.z, S[j][k + 3] = v.w;
                    }
            } else {
#pragma unroll
                for (int k = 0; k < KPT; ++k)
                    if (n0 + k < N) S[j][k] = src[k];
            }
        }
    }
    const int qoff = p.q_off + kh * N + n0, koff = p.k_off + kh * N + n0;
    struct Tok {
        float q[KPT], k[KPT], v[CPT], beta, g;
    };
    auto fetch = [&](int64_t t, Tok& u) {
        if (t >= r1) return;
        const float* row = p.X + t * p.ldx;
        if (vec) {      // KPT % 4 == 0 and every slice starts at a multiple of four floats and lies inside the row
#pragma unroll
            for (int k = 0; k < KPT; k += 4) {
                float4 q = make_float4(0, 0, 0, 0), kk = q;
                if (n0 + k < N) {
                    q = *(const float4*)(row + qoff + k);
                    kk = *(const float4*)(row + koff + k);
                }
                u.q[k] = q.x, u.q[k + 1] = q.y, u.q[k + 2] = q.z, u.q[k + 3] = q.w;
                u.k[k] = kk.x, u.k[k + 1] = kk.y, u.k[k + 2] = kk.z, u.k[k + 3] = kk.w;
            }
        } else {
#pragma unroll
            for (int k = 0; k < KPT; ++k) {
                const bool ok = n0 + k < N;
                u.q[k] = ok ? row[qoff + k] : 0.0f;
                u.k[k] = ok ? row[koff + k] : 0.0f;
            }
        }
#pragma unroll
        for (int j = 0; j < CPT; ++j) u.v[j] = cbase + j < P ? row[p.v_off + a * P + cbase + j] : 0.0f;
        u.beta = p.G[t * 2 * p.heads + a];
        u.g = p.G[t * 2 * p.heads + p.heads + a];
    };
    auto step = [&](int64_t t, const Tok& u) {
        if (t >= r1) return;
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
            float seen = 0.0f;
#pragma unroll
            for (int k = 0; k < KPT; ++k) {
                S[j][k] *= u.g;
                seen = fmaf(S[j][k], u.k[k], seen);
            }
            seen = group_sum(seen, 16);
            const float d = u.beta * (u.v[j] - seen);
            float part = 0.0f;
#pragma unroll
            for (int k = 0; k < KPT; ++k) {
                S[j][k] = fmaf(u.k[k], d, S[j][k]);
                part = fmaf(S[j][k], u.q[k], part);
            }
            part = group_sum(part, 16);
            if (nlane == 0 && cbase + j < P) p.out[t * p.ldo + a * P + cbase + j] = part;
        }
    };
    Tok A[GL_TG], B[GL_TG];
#pragma unroll
    for (int i = 0; i < GL_TG; ++i) fetch(r0 + i, A[i]);
    for (int64_t t = r0; t < r1; t += 2 * GL_TG) {
#pragma unroll
        for (int i = 0; i < GL_TG; ++i) fetch(t + GL_TG + i, B[i]);
#pragma unroll
        for (int i = 0; i < GL_TG; ++i) step(t + i, A[i]);
#pragma unroll
        for (int i = 0; i < GL_TG; ++i) fetch(t + 2 * GL_TG + i, A[i]);
#pragma unroll
        for (int i = 0; i < GL_TG; ++i) step(t + GL_TG + i, B[i]);
    }
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
        if (cbase + j >= P) continue;
        float* dst = gS + (int64_t)(cbase + j) * N;
        if (vec) {
#pragma unroll
            for (int k = 0; k < KPT; k += 4)
                if (n0 + k < N) *(float4*)(dst + k) = make_float4(S[j][k], S[j][k + 1], S[j][k + 2], S[j][k + 3]);
        } else {
#pragma unroll
            for (int k = 0; k < KPT; ++k)
                if (n0 + k < N) dst[k] = S[j][k];
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
// the lane that holds the largest value, ties to the lower index; (value, index) pairs with index < 0 do not take part
__device__ __forceinline__ int bl_wave_argmax(float v, int idx, float& best) {
    best = wave_max(idx >= 0 ? v : -INFINITY);
    const int cand = (idx >= 0 && v == best) ? idx : 0x7fffffff;
    return -wave_max_i(-cand);
}

#define RT_MAX_TOP 32
__global__ __launch_bounds__(256) void route_topk_kernel(const i64h_route_args p) {
    extern __shared__ float rt_lds[];   // per wave: [E] scores, [E] choice values, [groups] group flags
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int64_t t = (int64_t)blockIdx.x * 4 + wid;
    if (t >= p.n) return;     // (a whole wave leaves; no workgroup barrier below)
    const int E = p.E, G = p.groups > 1 ? p.groups : 1, gsz = E / G;
    // volatile: lanes read what another lane of the wave wrote (one wave: program order is enough, no barrier)
    volatile float* sc = rt_lds + (size_t)wid * (2 * E + G);
    volatile float* ch = sc + E;
    volatile float* gflag = ch + E;
    if (p.W) {      // the router's own products: eight entries at a time, every lane a share of the columns, fp32 throughout
        const float* h = p.h + t * p.ldh;
        const uint16_t* W = (const uint16_t*)p.W;
        const int K = p.K;
        const bool vec = (K & 3) == 0 && (p.ldh & 3) == 0 && ((uintptr_t)p.h & 15) == 0 && ((uintptr_t)p.W & 7) == 0;
        for (int e0 = 0; e0 < E; e0 += 8) {
            float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
            if (vec) {
                for (int k = lane * 4; k < K; k += 256) {
                    const float4 x = *(const float4*)(h + k);
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        if (e0 + j < E) {
                            const uint2 w = *(const uint2*)(W + (int64_t)(e0 + j) * K + k);
                            acc[j] = fmaf(x.x, __uint_as_float(w.x << 16), acc[j]);
                            acc[j] = fmaf(x.y, __uint_as_float(w.x & 0xffff0000u), acc[j]);
                            acc[j] = fmaf(x.z, __uint_as_float(w.y << 16), acc[j]);
                            acc[j] = fmaf(x.w, __uint_as_float(w.y & 0xffff0000u), acc[j]);
                        }
                    }
                }
            } else {
                for (int k = lane; k < K; k += 64) {
                    const float x = h[k];
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (e0 + j < E) acc[j] = fmaf(x, __uint_as_float((uint32_t)W[(int64_t)(e0 + j) * K + k] << 16), acc[j]);
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float v = wave_sum(acc[j]);
                if (lane == 0 && e0 + j < E) ch[e0 + j] = v;
            }
        }
    } else {
        const float* z = p.logits + t * p.ld;
        for (int e = lane; e < E; e += 64) ch[e] = z[e];
    }
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, ch[e]);
    mx = wave_max(mx);
    float sum = 0.0f;
    for (int e = lane; e < E; e += 64) {
        const float v = expf(ch[e] - mx);
        sc[e] = v;
        sum += v;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += 64) {
        const float s = sc[e] / sum;
        sc[e] = s;
        ch[e] = p.correction ? s + p.correction[e] : s;
    }
    if (G > 1) {   // a group's score: its largest choice value; the `keep` best groups stay, the entries of the others cannot be chosen
        for (int g = lane; g < G; g += 64) {
            float b = -INFINITY;
            for (int i = 0; i < gsz; ++i) b = fmaxf(b, ch[g * gsz + i]);
            gflag[g] = b;
        }
        // (LDS traffic of one wave needs program order only)
        for (int r = 0; r < p.keep; ++r) {
            float bv = -INFINITY;
            int bi = -1;
            for (int g = lane; g < G; g += 64) {
                const float v = gflag[g];
                if (!(v != v) && v != INFINITY && (bi < 0 || v > bv)) bv = v, bi = g;     // +inf marks a group already kept
            }
            float best;
            const int pick = bl_wave_argmax(bv, bi, best);
            if (pick != 0x7fffffff && lane == 0) gflag[pick] = INFINITY;
        }
        for (int e = lane; e < E; e += 64)
            if (gflag[e / gsz] != INFINITY) ch[e] = -INFINITY;
    }
    float wsum = 0.0f;
    float mine_w = 0.0f;      // lane k keeps the k-th choice
    int mine_i = 0;
    for (int k = 0; k < p.top; ++k) {
        float bv = -INFINITY;
        int bi = -1;
        for (int e = lane; e < E; e += 64) {
            const float v = ch[e];
            if (v == v && (bi < 0 || v > bv)) bv = v, bi = e;
        }
        float best;
        int pick = bl_wave_argmax(bv, bi, best);
        if (pick == 0x7fffffff) pick = 0;
        const float s = sc[pick];
        wsum += s;
        if (lane == k) mine_w = s, mine_i = pick;
        if (lane == 0) ch[pick] = __builtin_nanf("");     // taken: out of every later comparison
    }
    if (lane < p.top) {
        p.idx[t * p.top + lane] = mine_i;
        p.wgt[t * p.top + lane] = mine_w / (wsum + 1e-20f) * p.scale;
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void moe_plan_kernel(const i64h_moe_plan_args p) {
    extern __shared__ int pl_lds[];   // [experts + 1] counts, then offsets; [experts] cursors
    int* cnt = pl_lds;
    int* cur = pl_lds + p.experts + 1;
    const int tid = threadIdx.x;
    const int64_t pairs = p.n * p.top;
    for (int e = tid; e <= p.experts; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int64_t i = tid; i < pairs; i += 1024) {
        const int e = p.idx[i];
        if (e >= 0 && e < p.experts) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int e = 0; e < p.experts; ++e) {
            const int c = cnt[e];
            cnt[e] = run;
            cur[e] = run;
            run += c;
        }
        cnt[p.experts] = run;
    }
    __syncthreads();
    for (int e = tid; e <= p.experts; e += 1024) p.group_off[e] = cnt[e];
    for (int64_t i = tid; i < pairs; i += 1024) {
        const int e = p.idx[i];
        int r = -1;
        if (e >= 0 && e < p.experts) {
            r = atomicAdd(&cur[e], 1);
            p.pair_token[r] = (int)(i / p.top);
        }
        p.pair_row[i] = r;
    }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(const i64h_moe_combine_args p) {
    const int64_t t = blockIdx.x;
    const int W = p.W;
    for (int c = threadIdx.x; c < W; c += 256) {
        float a = 0.0f;
        for (int k = 0; k < p.top; ++k) {
            const int r = p.pair_row[t * p.top + k];
            const float v = r >= 0 ? p.Y[(int64_t)r * W + c] : p.h[t * W + c];
            a += p.wgt[t * p.top + k] * v;
        }
        if (p.shared) a += p.shared[t * W + c];
        p.out[t * W + c] = a;
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
extern "C" {

static int gla_check(const i64h_gla_args& d, const char* what) {
    I64H_CHECK_ARG(d.heads > 0 && d.dim > 0 && d.vdim > 0 && d.n >= 0, "%s: heads %d, dim %d, vdim %d", what, d.heads, d.dim, d.vdim);
    I64H_CHECK_ARG(d.P && d.q_off >= 0 && d.f_off >= 0 && d.v_off >= 0, "%s: null operand or negative column", what);
    return 0;
}

int i64h_gla_gates(const i64h_gla_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "gla_gates: no descriptor");
    const i64h_gla_args& d = *dp;
    if (gla_check(d, "gla_gates")) return 1;
    I64H_CHECK_ARG(d.n <= 65535, "gla_gates: %lld rows in one launch (at most 65535)", (long long)d.n);
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(gla_gates_kernel, dim3((unsigned)((d.heads * d.dim + 255) / 256), (unsigned)d.n), dim3(256), 0, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_gla_scan(const i64h_gla_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "gla_scan: no descriptor");
    const i64h_gla_args& d = *dp;
    if (gla_check(d, "gla_scan")) return 1;
    I64H_CHECK_ARG(d.seg_start && d.positions && d.slot_ids && d.state && d.out, "gla_scan: null operand");
    I64H_CHECK_ARG(d.dim <= 16 * 16, "gla_scan: dim %d above 256", d.dim);
    I64H_CHECK_ARG(d.nseg <= 65535, "gla_scan: %d runs in one launch", d.nseg);
    if (d.nseg <= 0 || d.n == 0) return 0;
    const int kpt = (d.dim + 15) / 16;
    // columns per lane: query, decay and key are loaded once for both - unless the launch would then leave most of the chip idle
    const int cpt = (d.vdim > 16 && (int64_t)d.heads * ((d.vdim + 31) / 32) * d.nseg >= 512) ? 2 : 1;
    const int ctiles = (d.vdim + 16 * cpt - 1) / (16 * cpt);
    const dim3 grid((unsigned)(d.heads * ctiles), (unsigned)d.nseg);
    const bool hask = d.k_off >= 0;
    auto launch = [&](auto kern, int K) {
        const int vec = K % 4 == 0 && d.dim % 4 == 0 && d.ldp % 4 == 0 && d.q_off % 4 == 0 && d.f_off % 4 == 0 && (!hask || d.k_off % 4 == 0) &&
                        (uintptr_t)d.P % 16 == 0 && (uintptr_t)d.state % 16 == 0;
        hipLaunchKernelGGL(kern, grid, dim3(256), 0, (hipStream_t)stream, d, ctiles, vec);
    };
#define GLA_PICK(C, HK)                                          \
    if (kpt <= 1) launch(gla_scan_kernel<1, C, HK>, 1);          \
    else if (kpt <= 2) launch(gla_scan_kernel<2, C, HK>, 2);     \
    else if (kpt <= 4) launch(gla_scan_kernel<4, C, HK>, 4);     \
    else if (kpt <= 8) launch(gla_scan_kernel<8, C, HK>, 8);     \
    else launch(gla_scan_kernel<16, C, HK>, 16);
    if (cpt == 2) {
        if (hask) { GLA_PICK(2, true) } else { GLA_PICK(2, false) }
    } else {
        if (hask) { GLA_PICK(1, true) } else { GLA_PICK(1, false) }
    }
#undef GLA_PICK
    I64H_CHECK_LAUNCH();
    return 0;
}

static int gdn_check(const i64h_gdn_args& d, const char* what) {
    I64H_CHECK_ARG(d.heads > 0 && d.kv_heads > 0 && d.heads % d.kv_heads == 0 && d.dim > 0 && d.vdim > 0 && d.n >= 0, "%s: heads %d, query / key heads %d, dim %d, vdim %d",
                   what, d.heads, d.kv_heads, d.dim, d.vdim);
    I64H_CHECK_ARG(d.X && d.G && d.q_off >= 0 && d.k_off >= 0 && d.v_off >= 0, "%s: null operand or negative column", what);
    return 0;
}

int i64h_gdn_gates(const i64h_gdn_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "gdn_gates: no descriptor");
    const i64h_gdn_args& d = *dp;
    if (gdn_check(d, "gdn_gates")) return 1;
    I64H_CHECK_ARG(d.R && d.A_log && d.dt_bias && d.b_off >= 0 && d.a_off >= 0, "gdn_gates: null operand or negative column");
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(gdn_gates_kernel, dim3((unsigned)d.n), dim3(256), 0, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_gdn_scan(const i64h_gdn_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "gdn_scan: no descriptor");
    const i64h_gdn_args& d = *dp;
    if (gdn_check(d, "gdn_scan")) return 1;
    I64H_CHECK_ARG(d.seg_start && d.positions && d.slot_ids && d.state && d.out, "gdn_scan: null operand");
    I64H_CHECK_ARG(d.dim <= 16 * 16, "gdn_scan: dim %d above 256", d.dim);
    I64H_CHECK_ARG(d.nseg <= 65535, "gdn_scan: %d runs in one launch", d.nseg);
    if (d.nseg <= 0 || d.n == 0) return 0;
    const int kpt = (d.dim + 15) / 16;
    // columns per lane: query and key are loaded once for both - unless the launch would then leave most of the chip idle
    // (two columns also give the two row sums of a token independent work to overlap: measured faster from 256 workgroups on)
    const int cpt = (d.vdim > 16 && (int64_t)d.heads * ((d.vdim + 31) / 32) * d.nseg >= 256) ? 2 : 1;
    const int ctiles = (d.vdim + 16 * cpt - 1) / (16 * cpt);
    const dim3 grid((unsigned)(d.heads * ctiles), (unsigned)d.nseg);
    auto launch = [&](auto kern, int K) {
        const int vec = K % 4 == 0 && d.dim % 4 == 0 && d.ldx % 4 == 0 && d.q_off % 4 == 0 && d.k_off % 4 == 0 && (uintptr_t)d.X % 16 == 0 && (uintptr_t)d.state % 16 == 0;
        hipLaunchKernelGGL(kern, grid, dim3(256), 0, (hipStream_t)stream, d, ctiles, vec);
    };
#define GDN_PICK(C)                                          \
    if (kpt <= 1) launch(gdn_scan_kernel<1, C>, 1);          \
    else if (kpt <= 2) launch(gdn_scan_kernel<2, C>, 2);     \
    else if (kpt <= 4) launch(gdn_scan_kernel<4, C>, 4);     \
    else if (kpt <= 8) launch(gdn_scan_kernel<8, C>, 8);     \
    else launch(gdn_scan_kernel<16, C>, 16);
    if (cpt == 2) { GDN_PICK(2) } else { GDN_PICK(1) }
#undef GDN_PICK
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_route_topk(const i64h_route_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "route_topk: no descriptor");
    const i64h_route_args& d = *dp;
    I64H_CHECK_ARG(d.E > 0 && d.E <= 1024 && d.top > 0 && d.top <= RT_MAX_TOP && d.top <= d.E, "route_topk: %d entries (at most 1024), top %d (at most %d)", d.E, d.top, RT_MAX_TOP);
    I64H_CHECK_ARG(d.groups <= 1 || (d.E % d.groups == 0 && d.keep >= 1 && d.keep <= d.groups), "route_topk: %d entries in %d groups, %d kept", d.E, d.groups, d.keep);
    I64H_CHECK_ARG(d.groups <= 1 || d.keep * (d.E / d.groups) >= d.top, "route_topk: %d kept groups of %d entries hold fewer than top %d", d.keep, d.E / (d.groups > 0 ? d.groups : 1), d.top);
    I64H_CHECK_ARG(d.idx && d.wgt && ((d.logits && d.ld >= d.E) || (d.W && d.h && d.K > 0 && d.ldh >= d.K)), "route_topk: null operand or row stride below the row");
    if (d.n == 0) return 0;
    const size_t lds = 4 * (size_t)(2 * d.E + (d.groups > 1 ? d.groups : 1)) * 4;
    hipLaunchKernelGGL(route_topk_kernel, dim3((unsigned)((d.n + 3) / 4)), dim3(256), lds, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_moe_plan(const i64h_moe_plan_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "moe_plan: no descriptor");
    const i64h_moe_plan_args& d = *dp;
    I64H_CHECK_ARG(d.experts > 0 && d.experts <= 4096 && d.top > 0 && d.n >= 0, "moe_plan: %d experts (at most 4096), top %d", d.experts, d.top);
    I64H_CHECK_ARG(d.idx && d.group_off && d.pair_token && d.pair_row, "moe_plan: null operand");
    I64H_CHECK_ARG(d.n * d.top < (1ll << 31), "moe_plan: too many pairs");
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), (size_t)(2 * d.experts + 1) * 4, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_moe_combine(const i64h_moe_combine_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "moe_combine: no descriptor");
    const i64h_moe_combine_args& d = *dp;
    I64H_CHECK_ARG(d.top > 0 && d.W > 0 && d.n >= 0, "moe_combine: top %d, width %d", d.top, d.W);
    I64H_CHECK_ARG(d.Y && d.pair_row && d.wgt && d.h && d.out, "moe_combine: null operand");
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)d.n), dim3(256), 0, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"
