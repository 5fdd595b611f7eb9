// hybrid_streams.hip: row kernels of decoders whose residual is several streams (ops/hybrid.py embed_pair, hyper_step,
// rope_rows, diff_group_norm).
//
// embed_pair_kernel: x = scale * embed[token] + pair[hash(previous token, token)], written `copies` times side by side.
// The previous token of a chunk's first row is the sequence's carried one (last[slot]); position 0 has none and takes
// the pair table's extra last row. The block of a chunk's first row leaves the chunk's last token in last[slot] after
// reading the old one.
// hyper_step_kernel<S>: one block per row of S streams [S][C]. With y: all streams at once from the old ones,
// x_t <- sum_s mix[s][t] x_s + out[t] y. With in: u = sum_t in[t] x_t of the new streams, h = u / rms(u) * (offset + w)
// as fp32 and / or bf16. Optionally the sum of the new streams. The row is read once: u stays in registers between the
// statistics and the output (columns beyond the register budget are recomputed from the streams just written). More
// than 8 streams take hyper_step_any_kernel, which keeps coefficients and a column's old values in LDS.
// rope_rows_kernel: rotary positions in place on fp32 heads, neighbouring pairs or the pairs (i, i + rot / 2).
// diff_group_norm_kernel: unit-RMS norm over groups of columns of a - lam * b.
//
// Launchers are `extern "C" int mxh_*(..., hipStream_t)`, return the launch's hipError_t, never allocate or
// synchronise (safe under stream capture) and check the shapes their grids assume.
#include "../mx_common.h"

namespace {

constexpr int NT = 256;

template <bool B16>
MX_DEV float ld_e(const void* p, long i) {
    if constexpr (B16) return bf16_to_f32(((const bf16_t*)p)[i]);
    else return ((const float*)p)[i];
}

// sum over the threads of a block of blockDim.x = 64 * k threads (k <= 16), returned to every thread
MX_DEV float block_sum_any(float v, float* red) {
    v = wave_sum(v);
    const int nw = blockDim.x >> 6;
    __syncthreads();  // red may still be read from an earlier call
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.f;
    for (int i = 0; i < nw; ++i) s += red[i];
    return s;
}

template <bool B16>
__global__ __launch_bounds__(1024) void embed_pair_kernel(const void* __restrict__ table, const void* __restrict__ pair,
                                                          int V, const int* __restrict__ tokens,
                                                          const int* __restrict__ seq_state,
                                                          const int* __restrict__ positions, int n_dec,
                                                          const int* __restrict__ pf_cu, int n_pf, int* last,
                                                          float scale, int mp, int mc, int buckets,
                                                          float* __restrict__ out, int copies, int C) {
    const int t = blockIdx.x, nt = blockDim.x;
    // what does not depend on the row's chunk is asked for at once: the token, its position, the token above, and
    // (decode rows) the slot; the chunk search of prompt rows follows
    const int raw = tokens[t];
    const int pos = pair ? positions[t] : 0;
    const int above = pair && t > 0 ? tokens[t - 1] : 0;
    const int tok = (raw < 0 || raw >= V) ? 0 : raw;
    long prow = -1;
    if (pair) {
        int s = t, first = t, end = t;  // decode rows: a chunk of one
        if (t >= n_dec) {
            const int r = t - n_dec;
            int lo = 0, hi = n_pf - 1;  // last i with pf_cu[i] <= r (empty chunks before it are passed over)
            while (lo < hi) {
                const int mid = (lo + hi + 1) >> 1;
                if (pf_cu[mid] <= r) lo = mid;
                else hi = mid - 1;
            }
            s = n_dec + lo;
            first = n_dec + pf_cu[lo];
            end = n_dec + pf_cu[lo + 1] - 1;
        }
        const int slot = seq_state[s];
        if (pos == 0) {
            prow = buckets;
        } else {
            const long prev = t == first ? (slot >= 0 ? last[slot] : 0) : above;
            const long hsh = (prev * mp + (long)raw * mc) % buckets;
            prow = hsh < 0 ? hsh + buckets : hsh;
        }
        if (t == first && slot >= 0) {
            __syncthreads();  // every thread of this block has read the carried token
            if (threadIdx.x == 0) last[slot] = tokens[end];
        }
    }
    const long base = (long)tok * C;
    float* o = out + (long)t * copies * C;
    for (int c = threadIdx.x; c < C; c += nt) {
        float v = ld_e<B16>(table, base + c) * scale;
        if (prow >= 0) v += ld_e<B16>(pair, prow * C + c);
        for (int k = 0; k < copies; ++k) o[(long)k * C + c] = v;
    }
}

template <int S>
__global__ __launch_bounds__(1024) void hyper_step_kernel(float* xs, const float* y, int ldy, const float* mix,
                                                          const float* ow, const float* iw, const float* nw,
                                                          float offset, float eps, float* h32, int ld32, bf16_t* h16,
                                                          int ld16, float* total, int ldt, int C) {
    // columns per thread whose old values are requested together and whose weighted sum stays in registers
    constexpr int HS_RK = S <= 2 ? 8 : 4;
    __shared__ float red[16];
    const int t = blockIdx.x, nt = blockDim.x;
    float* xr = xs + (long)t * S * C;
    const float* yr = y ? y + (long)t * ldy : nullptr;
    float m[S][S], wo[S], wi[S];
#pragma unroll
    for (int a = 0; a < S; ++a) {
        wo[a] = y ? ow[a] : 0.f;
        wi[a] = iw ? iw[a] : 0.f;
#pragma unroll
        for (int b = 0; b < S; ++b) m[a][b] = y ? mix[a * S + b] : (a == b ? 1.f : 0.f);
    }
    // one column from its old values: the streams' update (stored), their sum (stored when asked for), and the next
    // input's weighted sum
    auto column = [&](int c, const float (&x)[S], float yv) -> float {
        float nx[S];
        float u = 0.f, sum = 0.f;
        if (yr) {
#pragma unroll
            for (int b = 0; b < S; ++b) {
                float v = 0.f;
#pragma unroll
                for (int a = 0; a < S; ++a) v += m[a][b] * x[a];
                nx[b] = v + wo[b] * yv;
                xr[(long)b * C + c] = nx[b];
            }
        } else {
#pragma unroll
            for (int b = 0; b < S; ++b) nx[b] = x[b];
        }
#pragma unroll
        for (int b = 0; b < S; ++b) {
            u += wi[b] * nx[b];
            sum += nx[b];
        }
        if (total) total[(long)t * ldt + c] = sum;
        return u;
    };
    // the stores of one column may not pass the loads of the next (the compiler sees the same array): the loads of
    // all register columns go first, clamped and without branches, so that they are in flight together
    float xo[HS_RK][S], yo[HS_RK], u[HS_RK];
#pragma unroll
    for (int k = 0; k < HS_RK; ++k) {
        const int cc = min((int)threadIdx.x + k * nt, C - 1);
#pragma unroll
        for (int a = 0; a < S; ++a) xo[k][a] = xr[(long)a * C + cc];
        yo[k] = yr ? yr[cc] : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < HS_RK; ++k) {
        const int c = threadIdx.x + k * nt;
        u[k] = c < C ? column(c, xo[k], yo[k]) : 0.f;
        ss += u[k] * u[k];
    }
    for (int c = threadIdx.x + HS_RK * nt; c < C; c += nt) {
        float x[S];
#pragma unroll
        for (int a = 0; a < S; ++a) x[a] = xr[(long)a * C + c];
        const float v = column(c, x, yr ? yr[c] : 0.f);
        ss += v * v;
    }
    if (!iw) return;
    ss = block_sum_any(ss, red);
    const float sc = 1.f / sqrtf(ss / (float)C + eps);
    auto emit = [&](int c, float v) {
        v = v * sc * (offset + nw[c]);
        if (h32) h32[(long)t * ld32 + c] = v;
        if (h16) h16[(long)t * ld16 + c] = f32_to_bf16(v);
    };
#pragma unroll
    for (int k = 0; k < HS_RK; ++k) {
        const int c = threadIdx.x + k * nt;
        if (c < C) emit(c, u[k]);
    }
    for (int c = threadIdx.x + HS_RK * nt; c < C; c += nt) {  // the streams this thread has just written
        float v = 0.f;
#pragma unroll
        for (int b = 0; b < S; ++b) v += wi[b] * xr[(long)b * C + c];
        emit(c, v);
    }
}

// More than 8 streams (up to 32): the same pass with the coefficients and a column's old values in LDS instead of
// registers, one column at a time per thread; the next input is recomputed from the streams just written.
__global__ __launch_bounds__(NT) void hyper_step_any_kernel(float* xs, const float* y, int ldy, const float* mix,
                                                            const float* ow, const float* iw, const float* nw,
                                                            float offset, float eps, float* h32, int ld32, bf16_t* h16,
                                                            int ld16, float* total, int ldt, int S, int C) {
    extern __shared__ float sm[];  // mix [S][S], out [S], in [S], old values [S][NT]
    __shared__ float red[16];
    float* cm = sm;
    float* co = cm + S * S;
    float* ci = co + S;
    float* old = ci + S;
    const int t = blockIdx.x, tid = threadIdx.x;
    float* xr = xs + (long)t * S * C;
    const float* yr = y ? y + (long)t * ldy : nullptr;
    for (int i = tid; i < S * S; i += NT) cm[i] = y ? mix[i] : 0.f;
    for (int i = tid; i < S; i += NT) {
        co[i] = y ? ow[i] : 0.f;
        ci[i] = iw ? iw[i] : 0.f;
    }
    __syncthreads();
    float ss = 0.f;
    for (int c = tid; c < C; c += NT) {
        for (int a = 0; a < S; ++a) old[a * NT + tid] = xr[(long)a * C + c];
        const float yv = yr ? yr[c] : 0.f;
        float u = 0.f, sum = 0.f;
        for (int b = 0; b < S; ++b) {
            float v = old[b * NT + tid];
            if (yr) {
                v = 0.f;
                for (int a = 0; a < S; ++a) v += cm[a * S + b] * old[a * NT + tid];
                v += co[b] * yv;
                xr[(long)b * C + c] = v;
            }
            u += ci[b] * v;
            sum += v;
        }
        if (total) total[(long)t * ldt + c] = sum;
        ss += u * u;
    }
    if (!iw) return;
    ss = block_sum_any(ss, red);
    const float sc = 1.f / sqrtf(ss / (float)C + eps);
    for (int c = tid; c < C; c += NT) {  // the streams this thread has just written
        float v = 0.f;
        for (int b = 0; b < S; ++b) v += ci[b] * xr[(long)b * C + c];
        v = v * sc * (offset + nw[c]);
        if (h32) h32[(long)t * ld32 + c] = v;
        if (h16) h16[(long)t * ld16 + c] = f32_to_bf16(v);
    }
}

// grid (T, heads), one wave per (token, head)
constexpr int HEAD_E = 8;  // elements per lane: heads of up to 512 numbers
__global__ __launch_bounds__(64) void rope_rows_kernel(float* x, int ldx, const int* positions, int dim, int rot,
                                                       float neg_log_base, int half, float scale, int split,
                                                       float scale2) {
    const int t = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x;
    float* p = x + (long)t * ldx + (long)hd * dim;
    const float pos = (float)positions[t];
    const float sc = hd < split ? scale : scale2;
    const int n2 = rot >> 1;
    float val[HEAD_E];
#pragma unroll
    for (int k = 0; k < HEAD_E; ++k) {
        const int e = lane + k * 64;
        float v = 0.f;
        if (e < dim) {
            v = p[e];
            if (e < rot) {
                // the pair's first member turns as u cos - v sin, its second as v cos + u sin
                const bool second = half ? e >= n2 : (e & 1);
                const int mate = half ? (second ? e - n2 : e + n2) : (e ^ 1);
                const int i = half ? (second ? e - n2 : e) : (e >> 1);
                const float other = p[mate];
                const float f = expf((float)i * (2.f / (float)rot) * neg_log_base);
                float s, c;
                sincosf(pos * f, &s, &c);
                v = second ? v * c + other * s : v * c - other * s;
            }
        }
        val[k] = v * sc;
    }
    // a wave runs in lockstep through the loads above (no lane stores before every lane has read its mate), but the
    // compiler does not know that the stores below alias those loads across lanes: keep them apart
    __syncthreads();
#pragma unroll
    for (int k = 0; k < HEAD_E; ++k) {
        const int e = lane + k * 64;
        if (e < dim) p[e] = val[k];
    }
}

// grid (T, C / group)
template <bool B16>
__global__ __launch_bounds__(256) void diff_group_norm_kernel(const float* a, int lda, const float* b, int ldb, float lam,
                                                             float eps, int group, float out_scale, void* out,
                                                             int ldo) {
    __shared__ float red[16];
    const int t = blockIdx.x, c0 = blockIdx.y * group, nt = blockDim.x;
    const float* ar = a + (long)t * lda + c0;
    const float* br = b + (long)t * ldb + c0;
    constexpr int GC = 4;  // groups of up to blockDim * GC numbers stay in registers
    float z[GC];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < GC; ++k) {
        const int e = min((int)threadIdx.x + k * nt, group - 1);  // (clamped: both loads of all GC without a branch)
        z[k] = ar[e] - lam * br[e];
    }
#pragma unroll
    for (int k = 0; k < GC; ++k) {
        if ((int)threadIdx.x + k * nt >= group) z[k] = 0.f;
        ss += z[k] * z[k];
    }
    for (int e = threadIdx.x + GC * nt; e < group; e += nt) {
        const float v = ar[e] - lam * br[e];
        ss += v * v;
    }
    ss = block_sum_any(ss, red);
    const float sc = out_scale / sqrtf(ss / (float)group + eps);
    auto put = [&](int e, float v) {
        if constexpr (B16) ((bf16_t*)out)[(long)t * ldo + c0 + e] = f32_to_bf16(v * sc);
        else ((float*)out)[(long)t * ldo + c0 + e] = v * sc;
    };
#pragma unroll
    for (int k = 0; k < GC; ++k) {
        const int e = threadIdx.x + k * nt;
        if (e < group) put(e, z[k]);
    }
    for (int e = threadIdx.x + GC * nt; e < group; e += nt) put(e, ar[e] - lam * br[e]);
}

}  // namespace

#define MXH_CHECK(cond) \
    if (!(cond)) return (int)hipErrorInvalidValue

extern "C" int mxh_embed_pair(const void* table, const void* pair, int is16, int V, const int* tokens,
                              const int* seq_state, const int* positions, int n_dec, const int* pf_cu, int n_pf,
                              int* last, float scale, int mul_prev, int mul_cur, int buckets, float* out, int copies,
                              int T, int C, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(table && tokens && out && V > 0 && C > 0 && copies >= 1 && n_dec >= 0 && n_dec <= T);
    MXH_CHECK(!pair || (seq_state && positions && last && buckets > 0 && (n_dec == T || (pf_cu && n_pf > 0))));
    const int threads = C <= 1024 ? 256 : 1024;
    if (is16)
        embed_pair_kernel<true><<<T, threads, 0, st>>>(table, pair, V, tokens, seq_state, positions, n_dec, pf_cu, n_pf,
                                                       last, scale, mul_prev, mul_cur, buckets, out, copies, C);
    else
        embed_pair_kernel<false><<<T, threads, 0, st>>>(table, pair, V, tokens, seq_state, positions, n_dec, pf_cu, n_pf,
                                                        last, scale, mul_prev, mul_cur, buckets, out, copies, C);
    return (int)hipGetLastError();
}

extern "C" int mxh_hyper_step(float* xs, const float* y, int ldy, const float* mix, const float* ow, const float* iw,
                              const float* nw, float offset, float eps, float* h32, int ld32, void* h16, int ld16,
                              float* total, int ldt, int T, int S, int C, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(xs && S >= 1 && S <= 32 && C > 0);
    MXH_CHECK((!y || (mix && ow && ldy >= C)) && (!iw || (nw && (h32 || h16))) && (!h32 || ld32 >= C) &&
              (!h16 || ld16 >= C) && (!total || ldt >= C));
    if (S > 8) {
        const size_t dyn = (size_t)(S * S + 2 * S + S * NT) * sizeof(float);
        hyper_step_any_kernel<<<T, NT, dyn, st>>>(xs, y, ldy, mix, ow, iw, nw, offset, eps, h32, ld32, (bf16_t*)h16, ld16,
                                                  total, ldt, S, C);
        return (int)hipGetLastError();
    }
    const int threads = C <= 1024 ? 256 : 1024;
#define GO(S_)                                                                                                        \
    case S_:                                                                                                          \
        hyper_step_kernel<S_><<<T, threads, 0, st>>>(xs, y, ldy, mix, ow, iw, nw, offset, eps, h32, ld32, (bf16_t*)h16, \
                                                     ld16, total, ldt, C);                                            \
        break
    switch (S) {
        GO(1);
        GO(2);
        GO(3);
        GO(4);
        GO(5);
        GO(6);
        GO(7);
        GO(8);
    }
#undef GO
    return (int)hipGetLastError();
}

extern "C" int mxh_rope_rows(float* x, int ldx, const int* positions, int heads, int dim, int rot, float base, int half,
                             float scale, int split, float scale2, int T, hipStream_t st) {
    if (T <= 0 || heads <= 0) return 0;
    MXH_CHECK(x && positions && dim > 0 && dim <= 64 * HEAD_E && rot >= 0 && rot <= dim && rot % 2 == 0 && base > 0.f);
    MXH_CHECK(ldx >= heads * dim && heads <= 65535);
    rope_rows_kernel<<<dim3(T, heads), 64, 0, st>>>(x, ldx, positions, dim, rot, -logf(base), half, scale, split, scale2);
    return (int)hipGetLastError();
}

extern "C" int mxh_diff_group_norm(const float* a, int lda, const float* b, int ldb, float lam, float eps, int group,
                                   float out_scale, void* out, int ldo, int o16, int T, int C, hipStream_t st) {
    if (T <= 0) return 0;
    MXH_CHECK(a && b && out && group > 0 && C % group == 0 && C / group <= 65535 && lda >= C && ldb >= C && ldo >= C);
    const dim3 grid(T, C / group);
    const int threads = group <= 256 ? 64 : NT;  // one wave for a head of ordinary size
    if (o16) diff_group_norm_kernel<true><<<grid, threads, 0, st>>>(a, lda, b, ldb, lam, eps, group, out_scale, out, ldo);
    else diff_group_norm_kernel<false><<<grid, threads, 0, st>>>(a, lda, b, ldb, lam, eps, group, out_scale, out, ldo);
    return (int)hipGetLastError();
}
