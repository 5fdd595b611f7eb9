// hybrid_ops.hip: the fp32 row kernels of hybrid attention / recurrent decoders (ops/hybrid.py): embedding gather,
// offset RMS norm, output norm + residual add, rotary + head norm (+ weights, query temperature) + paged append, causal
// convolution with carried tails, unit-length heads, decay / write-strength coefficients, per-channel decays, gated
// group norm, gated linear unit with per-group factors, expert routing.
//
// All statistics, angles, gates, routing and the residual are fp32; 16-bit (bf16) appears only on outputs that feed a
// GEMM and in the paged pools. Launchers are `extern "C" int mxh_*(..., hipStream_t)`, return the launch's
// hipError_t, never allocate or synchronise (safe under stream capture) and check the shapes their grids assume.
#include "../mx_common.h"

namespace {

constexpr int NT = 256;

template <bool B16>
MX_DEV float ld_elem(const void* p, long i) {
    if constexpr (B16) return bf16_to_f32(((const bf16_t*)p)[i]);
    else return ((const float*)p)[i];
}
template <bool B16>
MX_DEV void st_elem(void* p, long i, float v) {
    if constexpr (B16) ((bf16_t*)p)[i] = f32_to_bf16(v);
    else ((float*)p)[i] = v;
}

MX_DEV float silu_acc(float x) { return x / (1.f + expf(-x)); }
MX_DEV float sigmoid_acc(float x) { return 1.f / (1.f + expf(-x)); }
MX_DEV float softplus_acc(float x) { return x > 30.f ? x : log1pf(expf(x)); }

// sum over the threads of a block of blockDim.x = 64 * k threads (k <= 16), returned to every thread
MX_DEV float block_sum_dyn(float v, float* red) {
    v = wave_sum(v);
    const int nw = blockDim.x >> 6;
    if (nw == 1) return v;
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.f;
    for (int i = 0; i < nw; ++i) s += red[i];
    return s;
}

template <bool B16>
__global__ __launch_bounds__(NT) void embed_rows_kernel(const void* table, int V, const int* tokens, float* out,
                                                        int ldo, int accumulate, int C, bf16_t* o16, int ld16) {
    const int t = blockIdx.x;
    int tok = tokens[t];
    if (tok < 0 || tok >= V) tok = 0;
    const long base = (long)tok * C;
    float* o = out + (long)t * ldo;
    for (int c = threadIdx.x; c < C; c += NT) {
        float v = ld_elem<B16>(table, base + c);
        if (accumulate) v += o[c];
        o[c] = v;
        if (o16) o16[(long)t * ld16 + c] = f32_to_bf16(v);
    }
}

constexpr int RC = 16;  // rows of up to NT * RC numbers are read once and kept in registers

__global__ __launch_bounds__(NT) void offset_norm_kernel(const float* x, int ldx, const int* rows, const float* w,
                                                         float offset, float eps, float* o32, int ld32, bf16_t* o16,
                                                         int ld16, int C) {
    __shared__ float red[NT / 64];
    const int i = blockIdx.x;
    const float* xr = x + (long)(rows ? rows[i] : i) * ldx;
    const bool cached = C <= NT * RC;
    float keep[RC], wk[RC];
    float ss = 0.f;
    if (cached) {
#pragma unroll
        for (int k = 0; k < RC; ++k) {  // clamped addresses: straight-line loads, all in flight together
            const int c = threadIdx.x + k * NT;
            const float v = xr[min(c, C - 1)];
            wk[k] = w[min(c, C - 1)];  // requested with the row, not after the reduction
            keep[k] = c < C ? v : 0.f;
            ss += keep[k] * keep[k];
        }
    } else {
        for (int c = threadIdx.x; c < C; c += NT) {
            const float v = xr[c];
            ss += v * v;
        }
    }
    ss = block_sum_dyn(ss, red);
    const float sc = 1.f / sqrtf(ss / (float)C + eps);
    if (cached) {
#pragma unroll
        for (int k = 0; k < RC; ++k) {
            const int c = threadIdx.x + k * NT;
            if (c < C) {
                const float v = keep[k] * sc * (offset + wk[k]);
                if (o32) o32[(long)i * ld32 + c] = v;
                if (o16) o16[(long)i * ld16 + c] = f32_to_bf16(v);
            }
        }
        return;
    }
    for (int c = threadIdx.x; c < C; c += NT) {
        const float v = xr[c] * sc * (offset + w[c]);
        if (o32) o32[(long)i * ld32 + c] = v;
        if (o16) o16[(long)i * ld16 + c] = f32_to_bf16(v);
    }
}

// x[t] += y[t] / rms(y[t]) * (offset + w); o16 (optional) = the new x[t] rounded. One block per row (256 or 1024
// threads: the launcher keeps the loads per thread few), the row of y kept in registers when it fits.
template <int RK>
__global__ __launch_bounds__(1024) void norm_add_kernel(const float* y, int ldy, const float* w, float offset, float eps,
                                                        float* x, int ldx, bf16_t* o16, int ld16, int C) {
    __shared__ float red[16];
    const int i = blockIdx.x, nt = blockDim.x;
    const float* yr = y + (long)i * ldy;
    float* xr = x + (long)i * ldx;
    const bool cached = C <= nt * RK;
    float keep[RK], wk[RK], xk[RK];
    float ss = 0.f;
    if (cached) {
#pragma unroll
        for (int k = 0; k < RK; ++k) {  // clamped addresses: straight-line loads, all in flight together
            const int c = min((int)threadIdx.x + k * nt, C - 1);
            const float v = yr[c];
            wk[k] = w[c];
            xk[k] = xr[c];
            keep[k] = (int)threadIdx.x + k * nt < C ? v : 0.f;
            ss += keep[k] * keep[k];
        }
    } else {
        for (int c = threadIdx.x; c < C; c += nt) {
            const float v = yr[c];
            ss += v * v;
        }
    }
    ss = block_sum_dyn(ss, red);
    const float sc = 1.f / sqrtf(ss / (float)C + eps);
    if (cached) {
#pragma unroll
        for (int k = 0; k < RK; ++k) {
            const int c = threadIdx.x + k * nt;
            if (c < C) {
                const float v = xk[k] + keep[k] * sc * (offset + wk[k]);
                xr[c] = v;
                if (o16) o16[(long)i * ld16 + c] = f32_to_bf16(v);
            }
        }
        return;
    }
    for (int c = threadIdx.x; c < C; c += nt) {
        const float v = xr[c] + yr[c] * sc * (offset + w[c]);
        xr[c] = v;
        if (o16) o16[(long)i * ld16 + c] = f32_to_bf16(v);
    }
}

// grid (T, H + G + Gv), one wave per (token, head): query heads, then key heads, then the Gv value heads. Element
// e < rot_dims of a query / key head turns with its neighbour e ^ 1 by angle pos * base^(-(e / 2) * 2 / rot_dims); with
// `half` the pairs are (i, i + rot_dims / 2) instead and pair i turns by pos * base^(-i * 2 / rot_dims).
constexpr int HEAD_E = 8;  // elements per lane: heads of up to 512 numbers
template <bool Q16, bool C16>
__global__ __launch_bounds__(64) void rope_norm_append_kernel(const float* qi, const float* ki, const float* vi,
                                                              int ldq, int ldk, int ldv, const int* positions, int H,
                                                              int G, int dk, int dv, int rot, float neg_log_base,
                                                              int norm, float eps, void* qo, int ldqo, void* kc,
                                                              void* vc, const int* slots, const float* qw,
                                                              const float* kw, float temp_coef, int temp_every,
                                                              int half, int Gv) {
    const int t = blockIdx.x, u = blockIdx.y, lane = threadIdx.x;
    if (u >= H + G) {  // value head: plain copy into the pool
        const int sl = slots[t];
        if (sl < 0) return;
        const int g = u - H - G;
        const float* src = vi + (long)t * ldv + (long)g * dv;
        const long dst = ((long)sl * Gv + g) * dv;
        for (int e = lane; e < dv; e += 64) st_elem<C16>(vc, dst + e, src[e]);
        return;
    }
    const bool isq = u < H;
    const int hd = isq ? u : u - H;
    int sl = 0;
    if (!isq) {
        sl = slots[t];
        if (sl < 0) return;
    }
    const float* src = isq ? qi + (long)t * ldq + (long)hd * dk : ki + (long)t * ldk + (long)hd * dk;
    const float pos = (float)positions[t];
    float val[HEAD_E];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < HEAD_E; ++k) {
        const int e = lane + k * 64;
        float v = 0.f;
        if (e < dk) {
            v = src[e];
            if (e < rot) {
                const int n2 = rot >> 1;
                const bool second = half ? e >= n2 : (e & 1);  // the pair's second member turns as v cos + u sin
                const int mate = half ? (second ? e - n2 : e + n2) : (e ^ 1);
                const int pi = half ? (second ? e - n2 : e) : (e >> 1);
                const float other = src[mate];
                const float f = expf((float)pi * (2.f / (float)rot) * neg_log_base);
                float s, c;
                sincosf(pos * f, &s, &c);
                v = second ? v * c + other * s : v * c - other * s;
            }
        }
        val[k] = v;
        ss += v * v;
    }
    float sc = 1.f;
    if (norm) sc = 1.f / sqrtf(wave_sum(ss) / (float)dk + eps);
    // the head norm's weight (shared by the heads) and, for queries, the temperature of the position
    const float* hw = isq ? qw : kw;
    if (isq && temp_coef != 0.f) sc *= 1.f + temp_coef * logf((float)((positions[t] + 1) / temp_every + 1));
    const long dst = isq ? (long)t * ldqo + (long)hd * dk : ((long)sl * G + hd) * dk;
#pragma unroll
    for (int k = 0; k < HEAD_E; ++k) {
        const int e = lane + k * 64;
        if (e < dk) {
            const float v = hw ? val[k] * sc * hw[e] : val[k] * sc;
            if (isq) st_elem<Q16>(qo, dst + e, v);
            else st_elem<C16>(kc, dst + e, v);
        }
    }
}

// grid (ceil(C / NT), sequences, ceil(T / CONV_ROWS)): thread = channel. Reads the tails only; conv_tails_kernel
// rolls them afterwards
constexpr int CONV_ROWS = 8;
__global__ __launch_bounds__(NT) void causal_conv_kernel(const float* x, int ldx, const float* w, const float* bias,
                                                         int taps, int silu, float* tails, const int* state,
                                                         const int* positions, int n_dec, const int* pf_cu, float* out,
                                                         int ldo, int C) {
    const int c = blockIdx.x * NT + threadIdx.x;
    const int s = blockIdx.y;
    int row0, n;
    if (s < n_dec) {
        row0 = s;
        n = 1;
    } else {
        const int k = s - n_dec;
        row0 = n_dec + pf_cu[k];
        n = pf_cu[k + 1] - pf_cu[k];
    }
    const int t0 = blockIdx.z * CONV_ROWS;
    if (t0 >= n || c >= C) return;
    const int slot = state[s];
    const int nt = taps - 1;
    const bool fresh = positions[row0] == 0 || slot < 0;
    float* tail = tails + ((long)(slot < 0 ? 0 : slot) * (nt > 0 ? nt : 1)) * C + c;  // entry i at tail[i * C]
    float wr[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) wr[j] = j < taps ? w[(long)c * taps + j] : 0.f;
    const float b = bias ? bias[c] : 0.f;
    const int t1 = min(n, t0 + CONV_ROWS);
    for (int t = t0; t < t1; ++t) {
        float acc = b;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            if (j < taps) {
                const int tau = t - nt + j;  // input index within the chunk; < 0: carried from earlier steps
                float v;
                if (tau >= 0) v = x[(long)(row0 + tau) * ldx + c];
                else v = fresh ? 0.f : tail[(long)(nt + tau) * C];
                acc += wr[j] * v;
            }
        }
        out[(long)(row0 + t) * ldo + c] = silu ? silu_acc(acc) : acc;
    }
}

// second pass of the convolution (launched after it on the same stream): new tails = last taps-1 inputs
__global__ __launch_bounds__(NT) void conv_tails_kernel(const float* x, int ldx, int taps, float* tails, const int* state,
                                                        const int* positions, int n_dec, const int* pf_cu, int C) {
    const int c = blockIdx.x * NT + threadIdx.x;
    const int s = blockIdx.y;
    int row0, n;
    if (s < n_dec) {
        row0 = s;
        n = 1;
    } else {
        const int k = s - n_dec;
        row0 = n_dec + pf_cu[k];
        n = pf_cu[k + 1] - pf_cu[k];
    }
    const int slot = state[s];
    const int nt = taps - 1;
    if (c >= C || n <= 0 || slot < 0 || nt <= 0) return;
    const bool fresh = positions[row0] == 0;
    float* tail = tails + (long)slot * nt * C + c;
    for (int i = 0; i < nt; ++i) {
        const int tau = n - nt + i;
        float v;
        if (tau >= 0) v = x[(long)(row0 + tau) * ldx + c];
        else v = fresh ? 0.f : tail[(long)(nt + tau) * C];  // index n + i > i: not yet overwritten
        tail[(long)i * C] = v;
    }
}

// grid (T, heads), one wave per head; heads from `split` on take scale2
__global__ __launch_bounds__(64) void unit_norm_kernel(float* x, int ldx, int dim, float eps, float scale, int split,
                                                       float scale2) {
    float* p = x + (long)blockIdx.x * ldx + (long)blockIdx.y * dim;
    float ss = 0.f;
    for (int e = threadIdx.x; e < dim; e += 64) ss += p[e] * p[e];
    const float sc = ((int)blockIdx.y < split ? scale : scale2) / sqrtf(wave_sum(ss) + eps);
    for (int e = threadIdx.x; e < dim; e += 64) p[e] *= sc;
}

__global__ __launch_bounds__(NT) void scan_coefs_kernel(const float* a, int lda, const float* b, int ldb,
                                                        const float* A_log, const float* dt_bias, float* decay,
                                                        float* coef, int T, int H) {
    const int i = blockIdx.x * NT + threadIdx.x;
    if (i >= T * H) return;
    const int t = i / H, h = i - t * H;
    const float s = softplus_acc(a[(long)t * lda + h] + dt_bias[h]);
    decay[i] = expf(-expf(A_log[h]) * s);
    coef[i] = b ? sigmoid_acc(b[(long)t * ldb + h]) : s;
}

// out = exp(log_sigmoid(x) * inv_tau) = sigmoid(x)^(1 / tau) with x = z + bias, or, with a projection proj [R, C],
// x = sum_r z[t, r] proj[r, c] + bias[c] (the second half of a low-rank projection, summed in fp32 in a fixed order)
// With rate_log (one per head of `per` channels): out = exp(-exp(rate_log[c / per]) * softplus(x)) instead.
__global__ __launch_bounds__(NT) void channel_decay_kernel(const float* z, int ldz, const float* bias, float inv_tau,
                                                           float* out, int C, const float* proj, int R,
                                                           const float* rate_log, int per) {
    extern __shared__ float zr[];  // the token's R inputs of the projection
    const int c = blockIdx.y * NT + threadIdx.x, t = blockIdx.x;
    if (proj) {
        for (int r = threadIdx.x; r < R; r += NT) zr[r] = z[(long)t * ldz + r];
        __syncthreads();
    }
    if (c >= C) return;
    float x = bias ? bias[c] : 0.f;
    if (proj) {
        for (int r = 0; r < R; ++r) x += zr[r] * proj[(long)r * C + c];
    } else {
        x += z[(long)t * ldz + c];
    }
    out[(long)t * C + c] = rate_log ? expf(-expf(rate_log[c / per]) * softplus_acc(x)) : expf(-softplus_acc(-x) * inv_tau);
}

// grid (T, C / group): one block per (token, group of columns). Groups of up to blockDim * GC numbers are read once
// (straight-line clamped loads, all in flight together) and kept in registers with their gates; the launcher picks
// the smallest GC that holds the group
// sigm: the gate's activation is a sigmoid instead of a SiLU. proj [R, C]: the gate row holds R numbers and column
// c's pre-activation is sum_r gate[t, r] proj[r, c], summed in fp32 in a fixed order (a low-rank gate's second half).
MX_DEV float gate_act(float x, int sigm) { return sigm ? sigmoid_acc(x) : silu_acc(x); }
MX_DEV float gate_pre(const float* gr, const float* proj, int R, int C, int c, const float* zr) {
    if (!proj) return gr[c];
    float x = 0.f;
    for (int r = 0; r < R; ++r) x += zr[r] * proj[(long)r * C + c];
    return x;
}
template <bool B16, int GC>
__global__ void gated_group_norm_kernel(const float* y, int ldy, const float* gate, int ldg, const float* w, int wlen,
                                        float eps, int group, int gate_first, float out_scale, void* out, int ldo,
                                        int sigm, const float* proj, int R, int C) {
    __shared__ float red[16];
    extern __shared__ float zr[];  // the token's R inputs of the gate projection
    const int t = blockIdx.x, c0 = blockIdx.y * group;
    const float* yr = y + (long)t * ldy + c0;
    const float* gr = gate + (long)t * ldg + (proj ? 0 : c0);
    const int nt = blockDim.x;
    if (proj) {  // the general form below, with the projected gate
        for (int r = threadIdx.x; r < R; r += nt) zr[r] = gr[r];
        __syncthreads();
        float ss = 0.f;
        for (int e = threadIdx.x; e < group; e += nt) {
            float v = yr[e];
            if (gate_first) v *= gate_act(gate_pre(gr, proj, R, C, c0 + e, zr), sigm);
            ss += v * v;
        }
        ss = block_sum_dyn(ss, red);
        const float sc = out_scale / sqrtf(ss / (float)group + eps);
        for (int e = threadIdx.x; e < group; e += nt) {
            const float g = gate_act(gate_pre(gr, proj, R, C, c0 + e, zr), sigm);
            float v = yr[e];
            if (gate_first) v *= g;
            v = v * sc * w[(c0 + e) % wlen];
            if (!gate_first) v *= g;
            st_elem<B16>(out, (long)t * ldo + c0 + e, v);
        }
        return;
    }
    if (group <= nt * GC) {
        float z[GC], gs[GC];
        float ss = 0.f;
#pragma unroll
        for (int k = 0; k < GC; ++k) {  // no branch in this loop: the loads are requested back to back
            const int ec = min((int)threadIdx.x + k * nt, group - 1);
            z[k] = yr[ec];
            gs[k] = gr[ec];
        }
#pragma unroll
        for (int k = 0; k < GC; ++k) {
            const int e = threadIdx.x + k * nt;
            gs[k] = gate_act(gs[k], sigm);
            z[k] = e < group ? (gate_first ? z[k] * gs[k] : z[k]) : 0.f;
            ss += z[k] * z[k];
        }
        ss = block_sum_dyn(ss, red);
        const float sc = out_scale / sqrtf(ss / (float)group + eps);
#pragma unroll
        for (int k = 0; k < GC; ++k) {
            const int e = threadIdx.x + k * nt;
            if (k * nt < group && e < group) {
                float v = z[k] * sc * w[(c0 + e) % wlen];
                if (!gate_first) v *= gs[k];
                st_elem<B16>(out, (long)t * ldo + c0 + e, v);
            }
        }
        return;
    }
    float ss = 0.f;
    for (int e = threadIdx.x; e < group; e += nt) {
        float v = yr[e];
        if (gate_first) v *= gate_act(gr[e], sigm);
        ss += v * v;
    }
    ss = block_sum_dyn(ss, red);
    const float sc = out_scale / sqrtf(ss / (float)group + eps);
    for (int e = threadIdx.x; e < group; e += nt) {
        const float g = gate_act(gr[e], sigm);
        float v = yr[e];
        if (gate_first) v *= g;
        v = v * sc * w[(c0 + e) % wlen];
        if (!gate_first) v *= g;
        st_elem<B16>(out, (long)t * ldo + c0 + e, v);
    }
}

// grid (T, ceil(F / NT))
// act 0: silu(x) * y * factor; 1: gelu_tanh(x) * y * factor; 2 (no second operand): relu(factor * x)^2
MX_DEV float gelu_tanh_acc(float x) {
    return 0.5f * x * (1.f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
}
template <bool B16>
__global__ __launch_bounds__(NT) void glu_kernel(const float* a, int lda, const float* b, int ldb, const float* ba,
                                                 const float* bb, const float* scale, int lds, int group,
                                                 int scale_sigmoid, void* out, int ldo, int F, int act) {
    const int f = blockIdx.y * NT + threadIdx.x, t = blockIdx.x;
    if (f >= F) return;
    float fac = 1.f;
    if (scale) {
        fac = scale[(long)t * lds + f / group];
        if (scale_sigmoid) fac = sigmoid_acc(fac);
        if (fac == 0.f) {  // an expert the router did not choose: nothing to evaluate
            st_elem<B16>(out, (long)t * ldo + f, 0.f);
            return;
        }
    }
    const float x = a[(long)t * lda + f] + (ba ? ba[f] : 0.f);
    if (act == 2) {
        const float r = fmaxf(fac * x, 0.f);
        st_elem<B16>(out, (long)t * ldo + f, r * r);
        return;
    }
    const float y = b[(long)t * ldb + f] + (bb ? bb[f] : 0.f);
    st_elem<B16>(out, (long)t * ldo + f, (act == 1 ? gelu_tanh_acc(x) : silu_acc(x)) * y * fac);
}

// one wave per token; lane l holds experts l, l + 64, ... (up to 16 each)
constexpr int ROUTE_E = 16;
// sigm: the chosen experts keep sigmoid(logit) * scale as their weights (no softmax, no renormalisation)
__global__ __launch_bounds__(64) void moe_route_kernel(const float* logits, int ld, const float* bias, int E, int top,
                                                       float scale, float eps, float* weights, int sigm) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (long)t * ld;
    float v[ROUTE_E];
    float m = -INFINITY;
#pragma unroll
    for (int k = 0; k < ROUTE_E; ++k) {
        const int e = lane + k * 64;
        v[k] = e < E ? z[e] + (bias ? bias[e] : 0.f) : -INFINITY;
        m = fmaxf(m, v[k]);
    }
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < ROUTE_E; ++k) {
        v[k] = (lane + k * 64) < E ? expf(v[k] - m) : -1.f;  // scores are >= 0; -1 marks absent or taken
        sum += fmaxf(v[k], 0.f);
    }
    sum = wave_sum(sum);
    float* wr = weights + (long)t * E;
    for (int e = lane; e < E; e += 64) wr[e] = 0.f;
    float mine[ROUTE_E];  // score of the experts this lane holds that were chosen (else 0)
#pragma unroll
    for (int k = 0; k < ROUTE_E; ++k) mine[k] = 0.f;
    float chosen = 0.f;
    for (int r = 0; r < top; ++r) {
        float best = -1.f;
        int bi = 0x7fffffff;
#pragma unroll
        for (int k = 0; k < ROUTE_E; ++k) {
            if (v[k] > best) {  // strict: the lowest index of equal scores within the lane
                best = v[k];
                bi = lane + k * 64;
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ob > best || (ob == best && oi < bi)) {
                best = ob;
                bi = oi;
            }
        }
        chosen += best / sum;
#pragma unroll
        for (int k = 0; k < ROUTE_E; ++k) {
            if (lane + k * 64 == bi) {
                mine[k] = v[k] / sum;
                v[k] = -1.f;
            }
        }
    }
    const float norm = scale / (chosen + eps);
#pragma unroll
    for (int k = 0; k < ROUTE_E; ++k) {
        const int e = lane + k * 64;
        if (e < E && v[k] < 0.f) {  // the taken ones (absent ones have e >= E)
            // exp(z - m) orders the experts as their logits do, so the same `top` are taken in both modes
            wr[e] = sigm ? scale * sigmoid_acc(z[e] + (bias ? bias[e] : 0.f)) : mine[k] * norm;
        }
    }
}

}  // namespace

#define MXH_CHECK(cond) \
    if (!(cond)) return (int)hipErrorInvalidValue

extern "C" int mxh_embed_rows(const void* table, int is16, int V, const int* tokens, float* out, int ldo,
                              int accumulate, bf16_t* o16, int ld16, int T, int C, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(table && tokens && out && C > 0 && V > 0 && ldo >= C && (!o16 || ld16 >= C));
    if (is16) embed_rows_kernel<true><<<T, NT, 0, st>>>(table, V, tokens, out, ldo, accumulate, C, o16, ld16);
    else embed_rows_kernel<false><<<T, NT, 0, st>>>(table, V, tokens, out, ldo, accumulate, C, o16, ld16);
    return (int)hipGetLastError();
}

extern "C" int mxh_offset_norm(const float* x, int ldx, const int* rows, const float* w, float offset, float eps,
                               float* o32, int ld32, bf16_t* o16, int ld16, int M, int C, hipStream_t st) {
    if (M <= 0) return 0;
    MXH_CHECK(x && w && (o32 || o16) && C > 0 && ldx >= C && (!o32 || ld32 >= C) && (!o16 || ld16 >= C));
    offset_norm_kernel<<<M, NT, 0, st>>>(x, ldx, rows, w, offset, eps, o32, ld32, o16, ld16, C);
    return (int)hipGetLastError();
}

extern "C" int mxh_norm_add(const float* y, int ldy, const float* w, float offset, float eps, float* x, int ldx,
                            bf16_t* o16, int ld16, int T, int C, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(y && w && x && C > 0 && ldy >= C && ldx >= C && (!o16 || ld16 >= C));
    if (C <= 1024) norm_add_kernel<4><<<T, 256, 0, st>>>(y, ldy, w, offset, eps, x, ldx, o16, ld16, C);
    else if (C <= 4096) norm_add_kernel<4><<<T, 1024, 0, st>>>(y, ldy, w, offset, eps, x, ldx, o16, ld16, C);
    else norm_add_kernel<16><<<T, 1024, 0, st>>>(y, ldy, w, offset, eps, x, ldx, o16, ld16, C);
    return (int)hipGetLastError();
}

extern "C" int mxh_rope_norm_append(const float* qi, const float* ki, const float* vi, int ldq, int ldk, int ldv,
                                    const int* positions, int H, int G, int dk, int dv, int rot, float base, int norm,
                                    float eps, void* qo, int ldqo, int q16, void* kc, void* vc, int c16,
                                    const int* slots, const float* qw, const float* kw, float temp_coef,
                                    int temp_every, int half, int Gv, int T, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(qi && ki && vi && positions && qo && kc && vc && slots && temp_every >= 1);
    // G == 0: queries only (keys and values of another layer are read). Gv value heads (the pool's row is Gv * dv)
    MXH_CHECK(H > 0 && G >= 0 && Gv >= 0 && (G > 0) == (Gv > 0) && dk > 0 && dv > 0 && dk <= 64 * HEAD_E && rot >= 0 &&
              rot <= dk && rot % 2 == 0);
    MXH_CHECK(ldq >= H * dk && ldk >= G * dk && ldv >= Gv * dv && ldqo >= H * dk && base > 0.f && H + G + Gv <= 65535);
    const dim3 grid(T, H + G + Gv);
    const float nlb = -logf(base);
#define GO(Q, C)                                                                                                   \
    rope_norm_append_kernel<Q, C><<<grid, 64, 0, st>>>(qi, ki, vi, ldq, ldk, ldv, positions, H, G, dk, dv, rot, nlb, \
                                                       norm, eps, qo, ldqo, kc, vc, slots, qw, kw, temp_coef, temp_every, \
                                                       half, Gv)
    if (q16 && c16) GO(true, true);
    else if (q16) GO(true, false);
    else if (c16) GO(false, true);
    else GO(false, false);
#undef GO
    return (int)hipGetLastError();
}

extern "C" int mxh_causal_conv(const float* x, int ldx, const float* w, const float* bias, int taps, int silu,
                               float* tails, const int* state, const int* positions, int n_dec, const int* pf_cu,
                               int n_pf, float* out, int ldo, int T, int C, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(x && w && tails && state && positions && out && C > 0 && taps >= 1 && taps <= 16);
    MXH_CHECK(ldx >= C && ldo >= C && n_dec >= 0 && n_pf >= 0 && n_dec + n_pf > 0 && (n_pf == 0 || pf_cu));
    const int rows = n_pf ? T - n_dec : 1;
    const dim3 grid((C + NT - 1) / NT, n_dec + n_pf, (max(rows, 1) + CONV_ROWS - 1) / CONV_ROWS);
    causal_conv_kernel<<<grid, NT, 0, st>>>(x, ldx, w, bias, taps, silu, tails, state, positions, n_dec, pf_cu, out,
                                            ldo, C);
    if (taps > 1) {
        const dim3 g2((C + NT - 1) / NT, n_dec + n_pf);
        conv_tails_kernel<<<g2, NT, 0, st>>>(x, ldx, taps, tails, state, positions, n_dec, pf_cu, C);
    }
    return (int)hipGetLastError();
}

extern "C" int mxh_unit_norm(float* x, int ldx, int heads, int dim, float eps, float scale, int split, float scale2,
                             int T, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(x && heads > 0 && heads <= 65535 && dim > 0 && ldx >= heads * dim);
    unit_norm_kernel<<<dim3(T, heads), 64, 0, st>>>(x, ldx, dim, eps, scale, split, scale2);
    return (int)hipGetLastError();
}

extern "C" int mxh_scan_coefs(const float* a, int lda, const float* b, int ldb, const float* A_log,
                              const float* dt_bias, float* decay, float* coef, int T, int H, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(a && A_log && dt_bias && decay && coef && H > 0 && lda >= H && (!b || ldb >= H));
    scan_coefs_kernel<<<(T * H + NT - 1) / NT, NT, 0, st>>>(a, lda, b, ldb, A_log, dt_bias, decay, coef, T, H);
    return (int)hipGetLastError();
}

extern "C" int mxh_channel_decay(const float* z, int ldz, const float* bias, float inv_tau, float* out, int T, int C,
                                 const float* proj, int R, const float* rate_log, int per, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(z && out && C > 0 && inv_tau > 0.f && C <= 65535 * NT && (!rate_log || (per > 0 && C % per == 0)));
    MXH_CHECK(proj ? (R > 0 && R <= 8192 && ldz >= R) : ldz >= C);
    channel_decay_kernel<<<dim3(T, (C + NT - 1) / NT), NT, proj ? R * sizeof(float) : 0, st>>>(z, ldz, bias, inv_tau, out,
                                                                                            C, proj, R, rate_log, per);
    return (int)hipGetLastError();
}

extern "C" int mxh_gated_group_norm(const float* y, int ldy, const float* gate, int ldg, const float* w, int wlen,
                                    float eps, int group, int gate_first, float out_scale, void* out, int ldo,
                                    int o16, int T, int C, int sigm, const float* proj, int R, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(y && gate && w && out && C > 0 && group > 0 && C % group == 0 && wlen > 0 && C % wlen == 0);
    MXH_CHECK(ldy >= C && ldo >= C && (proj ? (R > 0 && R <= 8192 && ldg >= R) : ldg >= C) && C / group <= 65535);
    const dim3 grid(T, C / group);
    const size_t dyn = proj ? R * sizeof(float) : 0;
#define GO(B, G_, nt_)                                                                                              \
    gated_group_norm_kernel<B, G_><<<grid, nt_, dyn, st>>>(y, ldy, gate, ldg, w, wlen, eps, group, gate_first, out_scale, \
                                                           out, ldo, sigm, proj, R, C)
#define PICK(B)                              \
    do {                                     \
        if (group <= 256) GO(B, 4, 64);      \
        else if (group <= 2048) GO(B, 8, NT); \
        else if (group <= 8192) GO(B, 8, 1024); \
        else GO(B, 32, 1024);                \
    } while (0)
    if (o16) PICK(true);
    else PICK(false);
#undef PICK
#undef GO
    return (int)hipGetLastError();
}

extern "C" int mxh_glu(const float* a, int lda, const float* b, int ldb, const float* ba, const float* bb,
                       const float* scale, int lds, int group, int scale_sigmoid, void* out, int ldo, int o16, int T,
                       int F, int act, hipStream_t st) {
    if (T <= 0 || F <= 0) return 0;
    MXH_CHECK(a && out && lda >= F && ldo >= F && group > 0 && F <= 65535 * NT && act >= 0 && act <= 2);
    MXH_CHECK(act == 2 ? !b : (b && ldb >= F));  // the squared ReLU has one operand
    MXH_CHECK(!scale || (F % group == 0 && lds >= F / group));
    const dim3 grid(T, (F + NT - 1) / NT);
    if (o16)
        glu_kernel<true><<<grid, NT, 0, st>>>(a, lda, b, ldb, ba, bb, scale, lds, group, scale_sigmoid, out, ldo, F, act);
    else
        glu_kernel<false><<<grid, NT, 0, st>>>(a, lda, b, ldb, ba, bb, scale, lds, group, scale_sigmoid, out, ldo, F, act);
    return (int)hipGetLastError();
}

extern "C" int mxh_moe_route(const float* logits, int ld, const float* bias, int T, int E, int top, float scale,
                             float eps, float* weights, int sigm, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(logits && weights && E > 0 && E <= 64 * ROUTE_E && top > 0 && top <= E && ld >= E);
    moe_route_kernel<<<T, 64, 0, st>>>(logits, ld, bias, E, top, scale, eps, weights, sigm);
    return (int)hipGetLastError();
}
