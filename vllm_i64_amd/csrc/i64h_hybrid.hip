// Kernels of libi64hip_dense.so for recurrent and hybrid layers (include/i64h_dense.h, "recurrent and hybrid layers"):
//   embed_bigram_kernel / prev_token_kernel : token embedding + hashed bigram embedding; the previous token is per-sequence state
//   streams_kernel        : multi-stream residual write (a result may pass a norm of its own first, and the result as a whole an RMS or
//                           centred norm) + the next sublayer's weighted read
//                           and RMS norm, one workgroup per row
//   causal_conv_kernel / conv_carry_kernel : per-channel causal convolution over rows and carried inputs (+ silu, or added to its input);
//                           the carry update
//   ssm_scan_kernel       : state-space recurrence with a scalar decay per head, a head's matrix in registers (16 lanes per value column)
//   gate_norm_kernel      : y * silu(z) -> RMS norm in groups
//   mingru_scan_kernel    : element-wise gated recurrence, tiles of 64 tokens scanned by four waves and folded
//   kattn_prep_kernel     : whole-row RMS norms of query and key, key-norm weights / scale / temperature folded into the query,
//                           raw key row and its 1 / rms into the paged cache
//   kattn_row_kernel      : attention over the cached keys (which are also the values, or with the values in front of them in the
//                           same cached row) with distance bias, chunk mask and sink
//   kv_prep_kernel        : [q | k | v] projections -> the cached row [v | k] per key head and query rows with zeros in the value columns
//   rot_prep_kernel       : the same with whole-row or per-head query / key norms, rotation of a part of every head in either pair layout
//                           and values turned by their own position; rot_post_kernel turns a head's sum back and applies a gate per head
// A row continues the row before it iff slot and position say so; state is taken as empty at position 0.  All arithmetic fp32.
#include "i64h_common.h"
#include "i64h_dense.h"

__device__ __forceinline__ float hy_bf16(const void* p, int64_t i) { return __uint_as_float((uint32_t)((const uint16_t*)p)[i] << 16); }
__device__ __forceinline__ float hy_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float hy_silu(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float hy_softplus(float x) { return x > 20.0f ? x : log1pf(expf(x)); }
__device__ __forceinline__ bool hy_continues(const int32_t* slot, const int32_t* pos, int64_t t, int d) {
    // row t - d belongs to the same run of consecutive positions as row t
    return t - d >= 0 && slot[t - d] == slot[t] && pos[t - d] == pos[t] - d;
}

// sum over the 256 threads of a workgroup; red: 4 floats of LDS
__device__ __forceinline__ float hy_block_sum(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

// ---------------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void embed_bigram_kernel(const i64h_embed_bigram_args p) {
    const int64_t t = blockIdx.x;
    int64_t id = p.ids[t];
    id = id < 0 ? 0 : (id >= p.V ? p.V - 1 : id);
    const int W = p.W;
    int64_t brow = -1;
    if (p.bigram) {
        if (p.positions[t] == 0) brow = p.buckets;
        else {
            int64_t prev = hy_continues(p.slot_ids, p.positions, t, 1) ? p.ids[t - 1] : p.prev_token[p.slot_ids[t]];
            prev = prev < 0 ? 0 : (prev >= p.V ? p.V - 1 : prev);
            brow = (prev * p.mul_prev + id * p.mul_cur) % p.buckets;
        }
    }
    const int64_t plane = p.n * (int64_t)W;
    const int64_t prow = p.pos_table ? min(max((int64_t)p.positions[t], (int64_t)0), p.pos_rows - 1) : 0;
    for (int c = threadIdx.x; c < W; c += 256) {
        float v = hy_bf16(p.table, id * W + c) * p.scale;
        if (p.pos_table) v += hy_bf16(p.pos_table, prow * W + c);
        if (brow >= 0) v += hy_bf16(p.bigram, brow * W + c);
        for (int s = 0; s < p.copies; ++s) p.out[s * plane + t * W + c] = v;
    }
}

__global__ __launch_bounds__(256) void prev_token_kernel(const i64h_embed_bigram_args p) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= p.n) return;
    if (t + 1 < p.n && hy_continues(p.slot_ids, p.positions, t + 1, 1)) return;   // not the last row of its run
    p.prev_token[p.slot_ids[t]] = p.ids[t];
}

// ---------------------------------------------------------------------------------------------------------------------------
#define HY_MAX_STREAMS 8
#define HY_MAX_TAPS 16
__global__ __launch_bounds__(256) void streams_kernel(const i64h_streams_args p) {
    extern __shared__ float sv[];   // [W] the weighted read of the row, then 4 floats for reductions
    const int tid = threadIdx.x;
    const int W = p.W, S = p.S;
    float* red = sv + W;
    const int64_t m = blockIdx.x;
    const int64_t r = p.rows ? (int64_t)p.rows[m] : m;
    const int64_t plane = p.n * (int64_t)W;
    float* xs = p.streams + r * W;
    float ya = 1.0f, yb = 1.0f;
    if (p.y && p.y2) {   // the two side-by-side results, each divided by its root mean square
        float a = 0.0f, b = 0.0f;
        for (int c = tid; c < W; c += 256) {
            const float u = p.y[m * p.ldy + c], v = p.y2[m * p.ldy2 + c];
            a += u * u;
            b += v * v;
        }
        a = hy_block_sum(a, red);
        b = hy_block_sum(b, red);
        ya = 1.0f / sqrtf(a / (float)W + p.y_eps);
        yb = 1.0f / sqrtf(b / (float)W + p.y_eps);
    } else if (p.y && p.yn_w) {   // one result with a norm of its own (the norm behind a sublayer)
        float a = 0.0f;
        for (int c = tid; c < W; c += 256) {
            const float u = p.y[m * p.ldy + c];
            a += u * u;
        }
        a = hy_block_sum(a, red);
        ya = sqrtf(a / (float)W + p.y_eps);     // divided by, as the norm in front is
    }
    // the result as the residual receives it: both side-by-side parts normed and averaged, or the one result with its own norm, or as it is
    auto result = [&](int c) -> float {
        float v = p.y[m * p.ldy + c];
        if (p.y2) v = 0.5f * (v * ya * p.yn_w[c] + p.y2[m * p.ldy2 + c] * yb * p.y2n_w[c]);
        else if (p.yn_w) v = v / ya * p.yn_w[c];
        return v;
    };
    float pmean = 0.0f, pden = 1.0f;
    if (p.y && p.post_w) {   // a norm over the whole result: the row waits in LDS, mean first, then the squared deviations
        float a = 0.0f;
        for (int c = tid; c < W; c += 256) {
            const float v = result(c);
            sv[c] = v;
            a += v;
        }
        if (p.post_center) pmean = hy_block_sum(a, red) / (float)W;
        float b = 0.0f;
        for (int c = tid; c < W; c += 256) {
            const float u = sv[c] - pmean;
            b += u * u;
        }
        b = hy_block_sum(b, red);
        pden = sqrtf(b / (float)W + p.y_eps);
    }
    float ss = 0.0f, su = 0.0f;
    for (int c = tid; c < W; c += 256) {
        float x[HY_MAX_STREAMS];
#pragma unroll
        for (int s = 0; s < HY_MAX_STREAMS; ++s) x[s] = s < S ? xs[s * plane + c] : 0.0f;
        if (p.y) {
            const float v = p.post_w ? (sv[c] - pmean) / pden * p.post_w[c] : result(c);
            float nx[HY_MAX_STREAMS];
#pragma unroll
            for (int t = 0; t < HY_MAX_STREAMS; ++t) {
                float a = 0.0f;
                if (t < S) {
                    if (p.mix) {
#pragma unroll
                        for (int s = 0; s < HY_MAX_STREAMS; ++s)
                            if (s < S) a += p.mix[s * S + t] * x[s];
                    } else a = x[t];
                    a += p.out_w[t] * v;
                    xs[t * plane + c] = a;
                }
                nx[t] = a;
            }
#pragma unroll
            for (int t = 0; t < HY_MAX_STREAMS; ++t) x[t] = nx[t];
        }
        if (p.h) {
            float u = 0.0f;
#pragma unroll
            for (int s = 0; s < HY_MAX_STREAMS; ++s)
                if (s < S) u += (p.in_w ? p.in_w[s] : 1.0f) * x[s];
            sv[c] = u;
            ss += u * u;
            su += u;
        }
    }
    if (!p.h) return;
    float mean = 0.0f;
    if (p.h_center) {        // the centred norm: the squared deviations from the mean, summed in a pass of their own
        mean = hy_block_sum(su, red) / (float)W;
        ss = 0.0f;
        for (int c = tid; c < W; c += 256) {
            const float u = sv[c] - mean;
            ss += u * u;
        }
    }
    ss = hy_block_sum(ss, red);
    const float den = sqrtf(ss / (float)W + p.eps);
    for (int c = tid; c < W; c += 256) p.h[m * W + c] = (sv[c] - mean) / den * p.norm_w[p.norm_w_len == 1 ? 0 : c];
}

// ---------------------------------------------------------------------------------------------------------------------------
// the input of channel c, d positions before row t (d >= 1); `before` = rows of this step that continue into row t (at most taps - 1 counted)
__device__ __forceinline__ float conv_input(const i64h_causal_conv_args& p, int64_t t, int d, int before, int c) {
    if (p.positions[t] - d < 0) return 0.0f;
    if (d <= before) return p.P[(t - d) * p.ldp + p.off + c];
    return p.state[((int64_t)p.slot_ids[t] * (p.taps - 1) + (p.taps - 1 + before - d)) * p.channels + c];
}
__device__ __forceinline__ int conv_rows_before(const i64h_causal_conv_args& p, int64_t t) {
    int before = 0;
    while (before < p.taps - 1 && hy_continues(p.slot_ids, p.positions, t, before + 1)) ++before;
    return before;
}

__global__ __launch_bounds__(256) void causal_conv_kernel(const i64h_causal_conv_args p) {
    const int64_t t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= p.channels) return;
    const int before = conv_rows_before(p, t);
    float a = p.bias ? p.bias[c] : 0.0f;
    for (int k = 0; k < p.taps - 1; ++k) a += p.w[(int64_t)c * p.taps + k] * conv_input(p, t, p.taps - 1 - k, before, c);
    const float x = p.P[t * p.ldp + p.off + c];
    a += p.w[(int64_t)c * p.taps + p.taps - 1] * x;
    p.out[t * p.ldo + c] = p.mode == 1 ? x + a : hy_silu(a);
    if (p.single_rows && p.taps > 1) {      // no other row of the launch reads or writes this sequence's carried inputs
        float v[HY_MAX_TAPS];
        for (int d = 1; d < p.taps - 1; ++d) v[d] = conv_input(p, t, d, before, c);
        float* st = p.state + (int64_t)p.slot_ids[t] * (p.taps - 1) * p.channels + c;
        for (int d = 1; d < p.taps - 1; ++d) st[(int64_t)(p.taps - 2 - d) * p.channels] = v[d];
        st[(int64_t)(p.taps - 2) * p.channels] = x;
    }
}

// the same for 2 .. 8 taps: a thread walks CV_ROWS consecutive rows of its channel with the weights and the last TAPS - 1 inputs in
// registers; only the first row of the walk and the first row of a run look back through memory
#define CV_ROWS 16
template <int TAPS>
__global__ __launch_bounds__(256) void causal_conv_walk_kernel(const i64h_causal_conv_args p) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= p.channels) return;
    const int64_t t0 = (int64_t)blockIdx.y * CV_ROWS, t1 = min(p.n, t0 + CV_ROWS);
    float w[TAPS], win[TAPS - 1];     // win[d - 1]: the input d positions back
#pragma unroll
    for (int k = 0; k < TAPS; ++k) w[k] = p.w[(int64_t)c * TAPS + k];
    const float bias = p.bias ? p.bias[c] : 0.0f;
    for (int64_t t = t0; t < t1; ++t) {
        if (t == t0 || !hy_continues(p.slot_ids, p.positions, t, 1)) {
            const int before = conv_rows_before(p, t);
#pragma unroll
            for (int d = 1; d < TAPS; ++d) win[d - 1] = conv_input(p, t, d, before, c);
        }
        const float x = p.P[t * p.ldp + p.off + c];
        float a = bias;
#pragma unroll
        for (int k = 0; k < TAPS - 1; ++k) a += w[k] * win[TAPS - 2 - k];
        a += w[TAPS - 1] * x;
        p.out[t * p.ldo + c] = p.mode == 1 ? x + a : hy_silu(a);
#pragma unroll
        for (int d = TAPS - 2; d > 0; --d) win[d] = win[d - 1];
        win[0] = x;
    }
}

__global__ __launch_bounds__(256) void conv_carry_kernel(const i64h_causal_conv_args p) {
    const int64_t t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (t + 1 < p.n && hy_continues(p.slot_ids, p.positions, t + 1, 1)) return;   // only the last row of a run
    if (c >= p.channels) return;
    const int before = conv_rows_before(p, t);
    float v[HY_MAX_TAPS];   // the inputs 0 .. taps - 2 positions back, read before any is overwritten
    for (int d = 0; d < p.taps - 1; ++d) v[d] = d == 0 ? p.P[t * p.ldp + p.off + c] : conv_input(p, t, d, before, c);
    for (int d = 0; d < p.taps - 1; ++d) p.state[((int64_t)p.slot_ids[t] * (p.taps - 1) + (p.taps - 2 - d)) * p.channels + c] = v[d];
}

// ---------------------------------------------------------------------------------------------------------------------------
// One workgroup per (head, 16 * CPT value columns, run of rows).  The 16 lanes of a DPP row share CPT neighbouring columns and hold KPT
// consecutive state indices of each in registers; a wave has four such rows.  Per token a lane loads its own slices of B and C once
// for its CPT columns (the next token's while this one is computed), updates its states with fused multiply-adds and the row sums the
// partial outputs with DPP moves: no LDS and no barrier, the tokens of a run strictly in their order (the same sums in the same order
// however a prompt is cut).  Step sizes and decays of 64 tokens are computed at once, a token per lane, and read back lane by lane.
// State layout [slot, head, value column, state index].
template <int KPT, int CPT>
__global__ __launch_bounds__(256) void ssm_scan_kernel(const i64h_ssm_scan_args p, const int ctiles, const int vec) {
    const int N = p.state, P = p.vdim;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int nlane = lane & 15, cl = lane >> 4;
    const int a = blockIdx.x / ctiles, seg = blockIdx.y;
    const int cbase = (blockIdx.x % ctiles) * 16 * CPT + (w * 4 + cl) * CPT;
    const int g = a / (p.heads / p.groups);
    const int64_t r0 = p.seg_start[seg], r1 = p.seg_start[seg + 1];
    if (r1 <= r0) return;
    const int n0 = nlane * KPT;
    const int inner = p.heads * P;
    float S[CPT][KPT];
    float* gS = p.ssm_state + ((int64_t)p.slot_ids[r0] * p.heads + a) * P * N + n0;      // + column * N
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
    const float dtb = p.dt_bias[a], Aneg = -expf(p.A_log[a]), Dk = p.Dskip[a];
    const int boff = inner + g * N + n0, coff = inner + (p.groups + g) * N + n0;
    struct Tok {
        float B[KPT], C[KPT], x[CPT];
    };
    auto fetch = [&](int64_t t, Tok& q) {
        const float* row = p.xbc + t * p.ldx;
        if (vec) {      // KPT % 4 == 0 and every slice starts at a multiple of four floats and lies inside the row
#pragma unroll
            for (int k = 0; k < KPT; k += 4) {
                float4 b = make_float4(0, 0, 0, 0), c = b;
                if (n0 + k < N) {
                    b = *(const float4*)(row + boff + k);
                    c = *(const float4*)(row + coff + k);
                }
                q.B[k] = b.x, q.B[k + 1] = b.y, q.B[k + 2] = b.z, q.B[k + 3] = b.w;
                q.C[k] = c.x, q.C[k + 1] = c.y, q.C[k + 2] = c.z, q.C[k + 3] = c.w;
            }
        } else {
#pragma unroll
            for (int k = 0; k < KPT; ++k) {
                const bool ok = n0 + k < N;
                q.B[k] = ok ? row[boff + k] : 0.0f;
                q.C[k] = ok ? row[coff + k] : 0.0f;
            }
        }
#pragma unroll
        for (int j = 0; j < CPT; ++j) q.x[j] = cbase + j < P ? row[a * P + cbase + j] : 0.0f;
    };
    auto step = [&](int64_t t, const Tok& q, float dt, float decay) {
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
            const float xv = dt * q.x[j];
            float part = 0.0f;
#pragma unroll
            for (int k = 0; k < KPT; ++k) {
                S[j][k] = fmaf(decay, S[j][k], q.B[k] * xv);
                part = fmaf(S[j][k], q.C[k], part);
            }
            part = group_sum(part, 16);
            if (nlane == 0 && cbase + j < P) p.y[t * p.ldy + a * P + cbase + j] = part + Dk * q.x[j];
        }
    };
    auto lane_value = [](float v, int i) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), i)); };
    for (int64_t tb = r0; tb < r1; tb += 64) {
        const int cnt = (int)min((int64_t)64, r1 - tb);
        float dtv = 0.0f, dec = 1.0f;
        if (lane < cnt) {
            dtv = hy_softplus(p.dt[(tb + lane) * p.lddt + a] + dtb);
            dec = expf(Aneg * dtv);
        }
        Tok q0, q1;
        fetch(tb, q0);
        for (int i = 0; i < cnt; i += 2) {
            if (i + 1 < cnt) fetch(tb + i + 1, q1);
            step(tb + i, q0, lane_value(dtv, i), lane_value(dec, i));
            if (i + 1 < cnt) {
                if (i + 2 < cnt) fetch(tb + i + 2, q0);
                step(tb + i + 1, q1, lane_value(dtv, i + 1), lane_value(dec, i + 1));
            }
        }
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
__global__ __launch_bounds__(256) void gate_norm_kernel(const i64h_gate_norm_args p) {
    extern __shared__ float sv[];   // [width] gated values, [groups] root mean squares
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int64_t m = blockIdx.x;
    const int W = p.width;
    for (int c = tid; c < W; c += 256) {
        float v = p.y[m * p.ldy + c];
        if (p.z && !p.gate_after) v *= hy_silu(p.z[m * p.ldz + c]);
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
    for (int c = tid; c < W; c += 256) {
        float v = sv[c] / sv[W + c / gs] * p.w[p.w_len > 0 ? c % p.w_len : c];
        if (p.z && p.gate_after) v *= hy_silu(p.z[m * p.ldz + c]);
        p.out[m * p.ldo + c] = v;
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
// One workgroup per (64 channels, run of rows), tiles of 4 x GR_TL tokens: every wave scans GR_TL consecutive tokens of the tile from
// an empty state, keeping per token the pair (A_t, B_t) of S_t = A_t * S_in + B_t, the waves' end pairs meet in LDS, every wave folds
// the pairs before its own onto the tile's incoming state and finishes its tokens.  All loads of a tile are in flight together.
#define GR_TL 16
__global__ __launch_bounds__(256) void mingru_scan_kernel(const i64h_mingru_scan_args p) {
    __shared__ float sA[2][4][64], sB[2][4][64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + lane;
    const bool cok = c < p.width;
    const int seg = blockIdx.y;
    const int64_t r0 = p.seg_start[seg], r1 = p.seg_start[seg + 1];
    if (r1 <= r0) return;
    float* st = p.state + (int64_t)p.slot_ids[r0] * p.width + (cok ? c : 0);
    float carry = (p.positions[r0] == 0 || !cok) ? 0.0f : *st;
    int buf = 0;
    for (int64_t t0 = r0; t0 < r1; t0 += 4 * GR_TL, buf ^= 1) {
        const int64_t tb = t0 + w * GR_TL;
        const int cnt = cok ? (int)max((int64_t)0, min((int64_t)GR_TL, r1 - tb)) : 0;
        float z[GR_TL], u[GR_TL], G[GR_TL], A[GR_TL], Bv[GR_TL];
#pragma unroll
        for (int i = 0; i < GR_TL; ++i) {
            z[i] = u[i] = G[i] = 0.0f;
            if (i < cnt) {
                const float* row = p.P + (tb + i) * p.ldp;
                z[i] = row[p.z_off + c];
                u[i] = row[p.x_off + c];
                G[i] = row[p.g_off + c];
            }
        }
        float a = 1.0f, b = 0.0f;
#pragma unroll
        for (int i = 0; i < GR_TL; ++i) {
            const float zz = i < cnt ? hy_sigmoid(z[i]) : 0.0f;      // past the end: the identity step
            const float cand = u[i] >= 0.0f ? u[i] + 0.5f : hy_sigmoid(u[i]);
            a = (1.0f - zz) * a;
            b = (1.0f - zz) * b + zz * cand;
            A[i] = a;
            Bv[i] = b;
        }
        sA[buf][w][lane] = a;
        sB[buf][w][lane] = b;
        __syncthreads();      // (the buffers alternate: the next tile's writes cannot overtake this tile's reads)
        float sin = carry, mine = carry;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            if (v == w) mine = sin;
            sin = sA[buf][v][lane] * sin + sB[buf][v][lane];
        }
        carry = sin;
#pragma unroll
        for (int i = 0; i < GR_TL; ++i)
            if (i < cnt) p.out[(tb + i) * p.ldo + c] = (A[i] * mine + Bv[i]) * hy_silu(G[i]);
    }
    if (w == 0 && cok) *st = carry;
}

// ---------------------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ int64_t cache_row(const int32_t* bt, int mbs, int bs, int slot, int pos) {
    return (int64_t)bt[(int64_t)slot * mbs + pos / bs] * bs + pos % bs;
}

__global__ __launch_bounds__(256) void kattn_prep_kernel(const i64h_kattn_prep_args p) {
    __shared__ float red[4];
    const int tid = threadIdx.x;
    const int64_t t = blockIdx.x;
    const int nq = p.heads * p.dim, nk = p.kv_heads * p.dim;
    const float* q = p.P + t * p.ldp + p.q_off;
    const float* k = p.P + t * p.ldp + p.k_off;
    float a = 0.0f, b = 0.0f;
    for (int c = tid; c < nq; c += 256) a += q[c] * q[c];
    for (int c = tid; c < nk; c += 256) b += k[c] * k[c];
    a = hy_block_sum(a, red);
    b = hy_block_sum(b, red);
    const float qr = 1.0f / sqrtf(a / (float)nq + p.eps);
    const float kr = 1.0f / sqrtf(b / (float)nk + p.eps);
    const int rep = p.heads / p.kv_heads;
    for (int c = tid; c < nq; c += 256) {
        const int h = c / p.dim, d = c % p.dim;
        float v = q[c] * qr * p.q_norm_w[c] * p.k_norm_w[(h / rep) * p.dim + d] * p.scale;
        if (p.temp) v *= p.temp[h];
        p.Q[t * nq + c] = v;
    }
    const int64_t row = cache_row(p.block_table, p.max_blocks_per_seq, p.block_size, p.slot_ids[t], p.positions[t]);
    if (p.cache_dtype == 0) {
        float* dst = (float*)p.cache + row * nk;
        for (int c = tid; c < nk; c += 256) dst[c] = k[c];
    } else {
        __bf16* dst = (__bf16*)p.cache + row * nk;
        for (int c = tid; c < nk; c += 256) dst[c] = (__bf16)k[c];
    }
    if (tid == 0) p.kscale[row] = kr;
}

// one wave per (row, head): the lanes take 64 keys at a time for the scores, then the value columns for the weighted sum.  With
// vdim > 0 a key head's part of a cached row is [vdim values | dim key values] and the query sits behind vdim zeros in its Q row;
// otherwise the dim key values are the values too.
#define KA_MAX_DIM 256
template <typename T>
__global__ __launch_bounds__(256) void kattn_row_kernel(const i64h_kattn_args p) {
    __shared__ float sq[4][KA_MAX_DIM];
    __shared__ float sp[4][64];
    __shared__ int64_t srow[4][64];
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int64_t item = (int64_t)blockIdx.x * 4 + wid;
    if (item >= p.n * p.heads) return;     // (a whole wave leaves; no workgroup barrier below)
    const int64_t t = item / p.heads;
    const int h = (int)(item % p.heads);
    const int g = h / (p.heads / p.kv_heads);
    const int dim = p.dim, vd = p.vdim > 0 ? p.vdim : dim, koff = p.vdim > 0 ? p.vdim : 0, gs = koff + dim;
    const int nk = p.kv_heads * gs;
    const int pos = p.positions[t], slot = p.slot_ids[t];
    const int lo = p.chunk > 0 ? (pos / p.chunk) * p.chunk : 0;
    const T* cache = (const T*)p.cache;
    for (int d = lane; d < dim; d += 64) sq[wid][d] = p.Q[(t * p.heads + h) * gs + koff + d];
    float m = p.sink ? 0.0f : -INFINITY, l = p.sink ? 1.0f : 0.0f;
    float acc[KA_MAX_DIM / 64] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int j0 = lo; j0 <= pos; j0 += 64) {
        const int j = j0 + lane;
        float s = -INFINITY;
        int64_t row = 0;
        if (j <= pos) {
            row = cache_row(p.block_table, p.max_blocks_per_seq, p.block_size, slot, j);
            const T* kr = cache + row * nk + g * gs + koff;
            float dot = 0.0f;
            for (int d = 0; d < dim; ++d) dot += sq[wid][d] * (float)kr[d];
            s = p.kscale ? dot * p.kscale[row] : dot;
            if (p.softcap > 0.0f) s = p.softcap * tanhf(s / p.softcap);
            if (p.bias) s += p.bias[(int64_t)min(pos - j, p.bias_rows - 1) * p.heads + h];
        }
        srow[wid][lane] = row;
        const float mn = fmaxf(m, wave_max(s));
        const float w = j <= pos ? expf(s - mn) : 0.0f;
        const float f = expf(m - mn);      // m is finite or the first tile has a key (mn finite): no inf - inf
        l = l * f + wave_sum(w);
        m = mn;
        sp[wid][lane] = w;
        const int cnt = min(64, pos - j0 + 1);
#pragma unroll
        for (int i = 0; i < KA_MAX_DIM / 64; ++i) {
            const int d = lane + 64 * i;
            if (d < vd) {
                float a = acc[i] * f;
                for (int u = 0; u < cnt; ++u) a += sp[wid][u] * (float)cache[srow[wid][u] * nk + g * gs + d];
                acc[i] = a;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < KA_MAX_DIM / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < vd) p.out[(t * p.heads + h) * vd + d] = acc[i] / l;
    }
}

// [q | k | v] projections -> the paged cache row [v | k] per key head and the query rows [0 | q * scale]
__global__ __launch_bounds__(256) void kv_prep_kernel(const i64h_kv_prep_args p) {
    const int tid = threadIdx.x;
    const int64_t t = blockIdx.x;
    const int gs = p.vdim + p.dim;
    const float* row = p.P + t * p.ldp;
    float* Q = p.Q + t * p.heads * gs;
    for (int c = tid; c < p.heads * gs; c += 256) {
        const int h = c / gs, d = c % gs;
        Q[c] = d < p.vdim ? 0.0f : row[p.q_off + h * p.dim + d - p.vdim] * p.scale;
    }
    if (!p.cache) return;
    const int64_t cr = cache_row(p.block_table, p.max_blocks_per_seq, p.block_size, p.slot_ids[t], p.positions[t]);
    const int nk = p.kv_heads * gs;
    for (int c = tid; c < nk; c += 256) {
        const int g = c / gs, d = c % gs;
        const float v = d < p.vdim ? row[p.v_off + g * p.vdim + d] : row[p.k_off + g * p.dim + d - p.vdim];
        if (p.cache_dtype == 0) ((float*)p.cache)[cr * nk + c] = v;
        else ((__bf16*)p.cache)[cr * nk + c] = (__bf16)v;
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
// [q | k | v] projections -> whole-row norms, rotation (two pair layouts, a part of every head), per-head norms, rotated values ->
// the paged cache row [v | k] per key head and the query rows [0 | q * scale].  The normed and rotated queries and keys wait in LDS
// for the per-head sums.
__device__ __forceinline__ void rot_pair(int d, int dims, int interleaved, int& a, int& b, int& i, bool& second) {
    // the pair of dimension d < dims: a the first member, b the second, i the pair's index; second: d is b
    if (interleaved) {
        i = d >> 1, a = d & ~1, b = d | 1, second = d & 1;
    } else {
        const int half = dims >> 1;
        second = d >= half, i = second ? d - half : d, a = i, b = i + half;
    }
}

// One workgroup per token, two passes: the raw queries and keys go to LDS while their squares are summed (a rotation keeps the sum of
// squares of a pair, so the per-head sums behind the rotation are those in front of it, the rotated part times rot_mult^2); the second
// pass norms and rotates out of LDS straight into the query rows and the cached row.
template <int NT>
__global__ __launch_bounds__(NT) void rot_prep_kernel(const i64h_rot_prep_args p) {
    extern __shared__ float sv[];   // [heads * dim + kv_heads * dim] raw queries and keys, [heads + kv_heads] 1 / rms per head, 8 for
                                    // reductions, [rot_dims] cosines and sines of the row's angles, [vdim] those of the values' angles
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int64_t t = blockIdx.x;
    const int dim = p.dim, vd = p.vdim, gs = vd + dim;
    const int nq = p.heads * dim, nk = p.kv_heads * dim;
    const int half = p.rot_dims >> 1, vhalf = p.v_freq ? vd >> 1 : 0;
    float* inv = sv + nq + nk;
    float* red = inv + p.heads + p.kv_heads;
    float* rcs = red + 8;           // [half] cosines, [half] sines: every head turns by the same angles
    float* vcs = rcs + 2 * half;    // [vhalf] cosines, [vhalf] sines
    const float* q = p.P + t * p.ldp + p.q_off;
    const float* k = p.P + t * p.ldp + p.k_off;
    const float* v = p.P + t * p.ldp + p.v_off;
    const int pos = p.positions[t];
    const float fpos = (float)pos;
    float a = 0.0f, b = 0.0f;
    for (int c = tid; c < nq + nk; c += NT) {
        const float x = c < nq ? q[c] : k[c - nq];
        sv[c] = x;
        if (c < nq) a += x * x;
        else b += x * x;
    }
    for (int i = tid; i < half + vhalf; i += NT) {
        float sn, cs;
        if (i < half) {
            sincosf(fpos * p.inv_freq[i], &sn, &cs);
            rcs[i] = cs * p.rot_mult, rcs[half + i] = sn * p.rot_mult;
        } else {
            sincosf(fpos * p.v_freq[i - half], &sn, &cs);
            vcs[i - half] = cs, vcs[vhalf + i - half] = sn;
        }
    }
    float qr = 1.0f, kr = 1.0f;
    if (p.q_norm_w) {   // (both sums through one exchange)
        a = wave_sum(a), b = wave_sum(b);
        __syncthreads();
        if (lane == 0) red[wid] = a, red[4 + wid] = b;
        __syncthreads();
        float sa = 0.0f, sb = 0.0f;
#pragma unroll
        for (int w = 0; w < NT / 64; ++w) sa += red[w], sb += red[4 + w];
        qr = 1.0f / sqrtf(sa / (float)nq + p.eps);
        kr = 1.0f / sqrtf(sb / (float)nk + p.eps);
    }
    __syncthreads();
    if (p.head_norm) {
        const float m2 = p.rot_mult * p.rot_mult;
        for (int h = wid; h < p.heads + p.kv_heads; h += NT / 64) {
            float s = 0.0f;
            for (int d = lane; d < dim; d += 64) {
                const float x = sv[h * dim + d];
                s += d < p.rot_dims ? x * x * m2 : x * x;
            }
            s = wave_sum(s);
            if (lane == 0) inv[h] = 1.0f / sqrtf(s / (float)dim + p.eps);
        }
        __syncthreads();
    }
    float* Q = p.Q + t * p.heads * gs;
    const int64_t cr = cache_row(p.block_table, p.max_blocks_per_seq, p.block_size, p.slot_ids[t], pos);
    const int nkv = p.kv_heads * gs;
    // every head's part of a query row and of the cached row: [vdim zeros or values | dim rotated values]; a wave takes whole heads, so
    // that what depends on the head only is the same for all its lanes and no lane divides
    for (int h = wid; h < p.heads + p.kv_heads; h += NT / 64) {
        const bool isq = h < p.heads;
        const int h0 = h * dim;                      // (the keys' raw values lie behind the queries': head index heads + g)
        const float* nw = isq ? p.q_norm_w : p.k_norm_w;
        const float r = isq ? qr : kr;
        const int w0 = isq ? h0 : h0 - nq;
        const float hn = (p.head_norm ? inv[h] : 1.0f) * (isq ? p.scale : 1.0f);
        const int g = h - p.heads;
        for (int d = lane; d < gs; d += 64) {
            float o;
            if (d >= vd) {
                const int e = d - vd;
                auto val = [&](int idx) { return nw ? sv[h0 + idx] * r * nw[w0 + idx] : sv[h0 + idx]; };
                if (e < p.rot_dims) {
                    int ia, ib, i;
                    bool second;
                    rot_pair(e, p.rot_dims, p.interleaved, ia, ib, i, second);
                    const float cs = rcs[i], sn = rcs[half + i];
                    const float u = val(ia), w = val(ib);
                    o = second ? w * cs + u * sn : u * cs - w * sn;
                } else {
                    o = val(e);
                }
                if (p.head_norm || isq) o *= hn;
            } else if (isq) {
                o = 0.0f;
            } else if (p.v_freq) {
                int ia, ib, i;
                bool second;
                rot_pair(d, vd, p.interleaved, ia, ib, i, second);
                const float cs = vcs[i], sn = vcs[vhalf + i];
                const float u = v[g * vd + ia], w = v[g * vd + ib];
                o = second ? w * cs + u * sn : u * cs - w * sn;
            } else {
                o = v[g * vd + d];
            }
            if (isq) Q[h * gs + d] = o;
            else if (p.cache_dtype == 0) ((float*)p.cache)[cr * nkv + g * gs + d] = o;
            else ((__bf16*)p.cache)[cr * nkv + g * gs + d] = (__bf16)o;
        }
    }
}

// the attention output of every head turned back by the row's own position and multiplied by the head's sigmoid gate, in place:
// a thread takes whole pairs
__global__ __launch_bounds__(256) void rot_post_kernel(const i64h_rot_post_args p) {
    extern __shared__ float sv[];   // [vdim / 2] cosines, [vdim / 2] sines: every head turns by the same angles
    const int64_t t = blockIdx.x;
    const int vd = p.vdim, half = vd >> 1;
    float* O = p.O + t * p.heads * vd;
    if (p.v_freq) {
        const float fpos = (float)p.positions[t];
        for (int i = threadIdx.x; i < half; i += 256) sincosf(fpos * p.v_freq[i], &sv[half + i], &sv[i]);
        __syncthreads();
    }
    const int items = p.v_freq ? p.heads * half : p.heads * vd;
    for (int e = threadIdx.x; e < items; e += 256) {
        if (p.v_freq) {
            const int h = e / half, i = e % half;
            const int a = p.interleaved ? 2 * i : i, b = p.interleaved ? 2 * i + 1 : i + half;
            const float g = p.gate ? hy_sigmoid(p.gate[t * p.ldg + h]) : 1.0f;
            const float cs = sv[i], sn = sv[half + i];
            const float u = O[h * vd + a], w = O[h * vd + b];
            O[h * vd + a] = (u * cs + w * sn) * g;      // the turn by the negative angle
            O[h * vd + b] = (w * cs - u * sn) * g;
        } else {
            O[e] *= hy_sigmoid(p.gate[t * p.ldg + e / vd]);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
extern "C" {

int i64h_embed_bigram(const i64h_embed_bigram_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "embed_bigram: no descriptor");
    const i64h_embed_bigram_args& d = *dp;
    I64H_CHECK_ARG(d.n >= 0 && d.W > 0 && d.V > 0 && d.copies >= 1, "embed_bigram: bad sizes");
    I64H_CHECK_ARG(d.ids && d.table && d.out && d.positions && d.slot_ids, "embed_bigram: null operand");
    I64H_CHECK_ARG(!d.bigram || (d.buckets > 0 && d.prev_token), "embed_bigram: the bigram table needs buckets and the previous tokens");
    I64H_CHECK_ARG(!d.pos_table || d.pos_rows > 0, "embed_bigram: an empty position table");
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(embed_bigram_kernel, dim3((unsigned)d.n), dim3(256), 0, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    if (d.bigram) {
        hipLaunchKernelGGL(prev_token_kernel, dim3((unsigned)((d.n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, d);
        I64H_CHECK_LAUNCH();
    }
    return 0;
}

int i64h_streams_step(const i64h_streams_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "streams: no descriptor");
    const i64h_streams_args& d = *dp;
    I64H_CHECK_ARG(d.S >= 1 && d.S <= HY_MAX_STREAMS && d.W > 0 && d.n >= 0, "streams: %d streams (at most %d), width %d", d.S, HY_MAX_STREAMS, d.W);
    I64H_CHECK_ARG(d.streams && (d.y || d.h), "streams: nothing to do");
    I64H_CHECK_ARG(!d.y || d.out_w, "streams: the write needs out_w");
    I64H_CHECK_ARG(!d.y2 || (d.y && d.yn_w && d.y2n_w), "streams: two results need both norm weights");
    I64H_CHECK_ARG(!d.h || (d.norm_w && (d.norm_w_len == 1 || d.norm_w_len == d.W)), "streams: the read needs a norm weight of 1 or W values");
    I64H_CHECK_ARG(!d.rows || !d.y, "streams: gathered rows are read only");
    const int64_t rows = d.rows ? d.m_rows : d.n;
    const size_t lds = ((size_t)d.W + 4) * 4;
    I64H_CHECK_ARG(lds <= 64 * 1024, "streams: a row of %d values does not fit the kernel's LDS buffer", d.W);
    if (rows == 0) return 0;
    hipLaunchKernelGGL(streams_kernel, dim3((unsigned)rows), dim3(256), lds, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_causal_conv(const i64h_causal_conv_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "causal_conv: no descriptor");
    const i64h_causal_conv_args& d = *dp;
    I64H_CHECK_ARG(d.channels > 0 && d.taps >= 1 && d.taps <= HY_MAX_TAPS && d.n >= 0, "causal_conv: %d channels, %d taps (at most %d)", d.channels, d.taps, HY_MAX_TAPS);
    I64H_CHECK_ARG(d.P && d.w && d.out && d.positions && d.slot_ids && (d.state || d.taps == 1), "causal_conv: null operand");
    I64H_CHECK_ARG(d.n <= 65535, "causal_conv: %lld rows in one launch (at most 65535)", (long long)d.n);
    I64H_CHECK_ARG(d.mode == 0 || d.mode == 1, "causal_conv: mode %d", d.mode);
    if (d.n == 0) return 0;
    const dim3 grid((unsigned)((d.channels + 255) / 256), (unsigned)d.n);
    const dim3 walk((unsigned)((d.channels + 255) / 256), (unsigned)((d.n + CV_ROWS - 1) / CV_ROWS));
    hipStream_t s = (hipStream_t)stream;
    switch ((d.n >= 32 * CV_ROWS && !d.single_rows) ? d.taps : 0) {     // few rows: a thread per row and channel fills the chip better
        case 2: hipLaunchKernelGGL(causal_conv_walk_kernel<2>, walk, dim3(256), 0, s, d); break;
        case 3: hipLaunchKernelGGL(causal_conv_walk_kernel<3>, walk, dim3(256), 0, s, d); break;
        case 4: hipLaunchKernelGGL(causal_conv_walk_kernel<4>, walk, dim3(256), 0, s, d); break;
        case 5: hipLaunchKernelGGL(causal_conv_walk_kernel<5>, walk, dim3(256), 0, s, d); break;
        case 6: hipLaunchKernelGGL(causal_conv_walk_kernel<6>, walk, dim3(256), 0, s, d); break;
        case 7: hipLaunchKernelGGL(causal_conv_walk_kernel<7>, walk, dim3(256), 0, s, d); break;
        case 8: hipLaunchKernelGGL(causal_conv_walk_kernel<8>, walk, dim3(256), 0, s, d); break;
        default: hipLaunchKernelGGL(causal_conv_kernel, grid, dim3(256), 0, s, d); break;
    }
    I64H_CHECK_LAUNCH();
    if (d.taps > 1 && !d.single_rows) {
        hipLaunchKernelGGL(conv_carry_kernel, grid, dim3(256), 0, (hipStream_t)stream, d);
        I64H_CHECK_LAUNCH();
    }
    return 0;
}

int i64h_ssm_scan(const i64h_ssm_scan_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "ssm_scan: no descriptor");
    const i64h_ssm_scan_args& d = *dp;
    I64H_CHECK_ARG(d.heads > 0 && d.vdim > 0 && d.state > 0 && d.groups > 0 && d.heads % d.groups == 0,
                   "ssm_scan: heads %d, groups %d, state %d, vdim %d", d.heads, d.groups, d.state, d.vdim);
    I64H_CHECK_ARG(d.xbc && d.dt && d.dt_bias && d.A_log && d.Dskip && d.seg_start && d.positions && d.slot_ids && d.ssm_state && d.y, "ssm_scan: null operand");
    I64H_CHECK_ARG(d.state <= 16 * 16, "ssm_scan: state %d above 256", d.state);
    I64H_CHECK_ARG(d.nseg <= 65535, "ssm_scan: %d runs in one launch", d.nseg);
    if (d.nseg <= 0 || d.n == 0) return 0;
    const int kpt = (d.state + 15) / 16;
    const int cpt = d.vdim > 16 ? 2 : 1;             // columns per lane: B and C are loaded once for both
    const int ctiles = (d.vdim + 16 * cpt - 1) / (16 * cpt);
    const dim3 grid((unsigned)(d.heads * ctiles), (unsigned)d.nseg);
    const int inner = d.heads * d.vdim;
    auto launch = [&](auto kern, int K) {
        const int vec = K % 4 == 0 && d.state % 4 == 0 && d.ldx % 4 == 0 && inner % 4 == 0 && (uintptr_t)d.xbc % 16 == 0 && (uintptr_t)d.ssm_state % 16 == 0;
        hipLaunchKernelGGL(kern, grid, dim3(256), 0, (hipStream_t)stream, d, ctiles, vec);
    };
    if (cpt == 2) {
        if (kpt <= 1) launch(ssm_scan_kernel<1, 2>, 1);
        else if (kpt <= 2) launch(ssm_scan_kernel<2, 2>, 2);
        else if (kpt <= 4) launch(ssm_scan_kernel<4, 2>, 4);
        else if (kpt <= 8) launch(ssm_scan_kernel<8, 2>, 8);
        else launch(ssm_scan_kernel<16, 2>, 16);
    } else {
        if (kpt <= 1) launch(ssm_scan_kernel<1, 1>, 1);
        else if (kpt <= 2) launch(ssm_scan_kernel<2, 1>, 2);
        else if (kpt <= 4) launch(ssm_scan_kernel<4, 1>, 4);
        else if (kpt <= 8) launch(ssm_scan_kernel<8, 1>, 8);
        else launch(ssm_scan_kernel<16, 1>, 16);
    }
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_gate_norm(const i64h_gate_norm_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "gate_norm: no descriptor");
    const i64h_gate_norm_args& d = *dp;
    I64H_CHECK_ARG(d.width > 0 && d.groups > 0 && d.width % d.groups == 0, "gate_norm: width %d does not split into %d groups", d.width, d.groups);
    I64H_CHECK_ARG(d.y && d.w && d.out, "gate_norm: null operand");
    const size_t lds = ((size_t)d.width + d.groups) * 4;
    I64H_CHECK_ARG(lds <= 64 * 1024, "gate_norm: a row of %d values does not fit the kernel's LDS buffer", d.width);
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(gate_norm_kernel, dim3((unsigned)d.n), dim3(256), lds, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_mingru_scan(const i64h_mingru_scan_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "mingru_scan: no descriptor");
    const i64h_mingru_scan_args& d = *dp;
    I64H_CHECK_ARG(d.width > 0 && d.P && d.seg_start && d.positions && d.slot_ids && d.state && d.out, "mingru_scan: bad arguments");
    I64H_CHECK_ARG(d.nseg <= 65535, "mingru_scan: %d runs in one launch", d.nseg);
    if (d.nseg <= 0 || d.n == 0) return 0;
    hipLaunchKernelGGL(mingru_scan_kernel, dim3((unsigned)((d.width + 63) / 64), (unsigned)d.nseg), dim3(256), 0, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_kattn_prep(const i64h_kattn_prep_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "kattn_prep: no descriptor");
    const i64h_kattn_prep_args& d = *dp;
    I64H_CHECK_ARG(d.heads > 0 && d.kv_heads > 0 && d.heads % d.kv_heads == 0 && d.dim > 0, "kattn_prep: heads %d, kv heads %d, dim %d", d.heads, d.kv_heads, d.dim);
    I64H_CHECK_ARG(d.P && d.q_norm_w && d.k_norm_w && d.positions && d.slot_ids && d.block_table && d.cache && d.kscale && d.Q, "kattn_prep: null operand");
    I64H_CHECK_ARG(d.cache_dtype == 0 || d.cache_dtype == 2, "kattn_prep: cache type %d", d.cache_dtype);
    I64H_CHECK_ARG(d.block_size > 0 && d.max_blocks_per_seq > 0, "kattn_prep: bad paging");
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(kattn_prep_kernel, dim3((unsigned)d.n), dim3(256), 0, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int64_t i64h_kattn_workspace_floats(int64_t n, int32_t heads, int32_t kv_heads, int32_t dim, int32_t splits) {
    if (splits <= 1 || kv_heads <= 0) return 0;
    return n * kv_heads * ((heads / kv_heads + 15) / 16) * (int64_t)(splits > 64 ? 64 : splits) * 16 * (dim + 2);
}

int i64h_kattn(const i64h_kattn_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "kattn: no descriptor");
    const i64h_kattn_args& d = *dp;
    I64H_CHECK_ARG(d.heads > 0 && d.kv_heads > 0 && d.heads % d.kv_heads == 0 && d.dim > 0 && d.dim <= KA_MAX_DIM, "kattn: heads %d, kv heads %d, dim %d (at most %d)",
                   d.heads, d.kv_heads, d.dim, KA_MAX_DIM);
    I64H_CHECK_ARG(d.vdim >= 0 && d.vdim <= KA_MAX_DIM, "kattn: vdim %d (at most %d)", d.vdim, KA_MAX_DIM);
    I64H_CHECK_ARG(d.Q && d.cache && (d.kscale || d.vdim > 0) && d.block_table && d.slot_ids && d.positions && d.out, "kattn: null operand");
    I64H_CHECK_ARG(d.cache_dtype == 0 || d.cache_dtype == 2, "kattn: cache type %d", d.cache_dtype);
    I64H_CHECK_ARG(!d.bias || d.bias_rows > 0, "kattn: an empty bias table");
    I64H_CHECK_ARG(d.block_size > 0 && d.max_blocks_per_seq > 0, "kattn: bad paging");
    if (d.n == 0) return 0;
    // the matrix-core kernel of the latent attention scores against a whole cached row part and sums its first columns: the keys as values
    // (all columns) or [values | keys] with zeros in the query's value columns
    const int vals = d.vdim > 0 ? d.vdim : d.dim, gs = d.vdim > 0 ? d.vdim + d.dim : d.dim;
    if (d.mode != 1 && d.cache_dtype == 2 && vals % 16 == 0 && vals <= 256 && gs % 8 == 0 && gs <= 320 && (uintptr_t)d.Q % 16 == 0 && (uintptr_t)d.cache % 16 == 0) {
        i64h_latent_attn_args a = {};
        a.Q = d.Q, a.cache = d.cache, a.cache_dtype = d.cache_dtype, a.block_table = d.block_table, a.max_blocks_per_seq = d.max_blocks_per_seq;
        a.block_size = d.block_size, a.slot_ids = d.slot_ids, a.positions = d.positions, a.window = 0, a.scale = 1.0f, a.out = d.out, a.n = d.n;
        a.heads = d.heads, a.kv_rank = vals, a.rot_dim = gs - vals, a.mode = d.mode == 3 ? 3 : 2, a.splits = d.splits, a.workspace = d.workspace;
        a.row_stride = d.kv_heads * gs, a.kv_groups = d.kv_heads, a.chunk = d.chunk, a.kscale = d.kscale, a.bias = d.bias, a.bias_rows = d.bias_rows;
        a.sink = d.sink, a.softcap = d.softcap;
        a.key_off = d.vdim > 0 ? d.vdim : 0;
        return i64h_latent_attn(&a, stream);
    }
    const int64_t items = d.n * d.heads;
    const dim3 grid((unsigned)((items + 3) / 4));
    if (d.cache_dtype == 0) hipLaunchKernelGGL((kattn_row_kernel<float>), grid, dim3(256), 0, (hipStream_t)stream, d);
    else hipLaunchKernelGGL((kattn_row_kernel<__bf16>), grid, dim3(256), 0, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_kv_prep(const i64h_kv_prep_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "kv_prep: no descriptor");
    const i64h_kv_prep_args& d = *dp;
    I64H_CHECK_ARG(d.heads > 0 && d.kv_heads > 0 && d.heads % d.kv_heads == 0 && d.dim > 0 && d.vdim > 0, "kv_prep: heads %d, kv heads %d, dim %d, vdim %d",
                   d.heads, d.kv_heads, d.dim, d.vdim);
    I64H_CHECK_ARG(d.P && d.Q && d.positions && d.slot_ids, "kv_prep: null operand");
    I64H_CHECK_ARG(!d.cache || (d.block_table && d.block_size > 0 && d.max_blocks_per_seq > 0 && (d.cache_dtype == 0 || d.cache_dtype == 2)), "kv_prep: bad paging or cache type");
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(kv_prep_kernel, dim3((unsigned)d.n), dim3(256), 0, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_rot_prep(const i64h_rot_prep_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "rot_prep: no descriptor");
    const i64h_rot_prep_args& d = *dp;
    I64H_CHECK_ARG(d.heads > 0 && d.kv_heads > 0 && d.heads % d.kv_heads == 0 && d.dim > 0 && d.vdim > 0, "rot_prep: heads %d, kv heads %d, dim %d, vdim %d",
                   d.heads, d.kv_heads, d.dim, d.vdim);
    I64H_CHECK_ARG(d.rot_dims >= 0 && d.rot_dims <= d.dim && d.rot_dims % 2 == 0 && (d.rot_dims == 0 || d.inv_freq), "rot_prep: %d rotated dimensions of %d", d.rot_dims, d.dim);
    I64H_CHECK_ARG(!d.v_freq || d.vdim % 2 == 0, "rot_prep: rotated values of an odd size %d", d.vdim);
    I64H_CHECK_ARG((d.q_norm_w == nullptr) == (d.k_norm_w == nullptr), "rot_prep: the whole-row norms come together");
    I64H_CHECK_ARG(d.P && d.Q && d.positions && d.slot_ids && d.block_table && d.cache, "rot_prep: null operand");
    I64H_CHECK_ARG(d.block_size > 0 && d.max_blocks_per_seq > 0 && (d.cache_dtype == 0 || d.cache_dtype == 2), "rot_prep: bad paging or cache type");
    const size_t lds = ((size_t)(d.heads + d.kv_heads) * (d.dim + 1) + 8 + d.rot_dims + (d.v_freq ? d.vdim : 0)) * 4;
    I64H_CHECK_ARG(lds <= 64 * 1024, "rot_prep: %d + %d heads of %d values do not fit the kernel's LDS buffer", d.heads, d.kv_heads, d.dim);
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(rot_prep_kernel<256>, dim3((unsigned)d.n), dim3(256), lds, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_rot_post(const i64h_rot_post_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "rot_post: no descriptor");
    const i64h_rot_post_args& d = *dp;
    I64H_CHECK_ARG(d.heads > 0 && d.vdim > 0 && (!d.v_freq || d.vdim % 2 == 0), "rot_post: heads %d, vdim %d", d.heads, d.vdim);
    I64H_CHECK_ARG(d.O && d.positions && (d.v_freq || d.gate), "rot_post: null operand or nothing to do");
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(rot_post_kernel, dim3((unsigned)d.n), dim3(256), (size_t)d.vdim * 4, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"
