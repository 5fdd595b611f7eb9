// hybrid_scan.hip: the linear recurrence of gated-delta-rule and state-space (duality form) layers (ops/hybrid.py
// state_scan). Per sequence and head, over the step's rows in order:
//     S <- a_t S;   u = c_t (v_t - S^T k_t)  [delta]   or   u = c_t v_t;   S <- S + k_t u^T;   o_t = S^T q_t (+ D v_t)
// S has N numbers for each of the head's P value columns, fp32, stored column-major: state [slots, H, P, N]. The
// columns never mix, so a column belongs to LPC neighbouring lanes (4, or the 16 of one DPP row) that each keep NPL
// consecutive numbers of it in registers for the whole chunk: a step costs 4 NPL vector operations and two LPC-wide
// sums done with DPP moves, and a lane's part of the state is one contiguous run in memory (a column's lanes read N
// contiguous floats, a wave's columns are adjacent). k_t and q_t are the same for every column of a head: the block
// stages them in LDS together with the tokens' decays, write strengths and values, 8 or 16 tokens at a time in two
// buffers; the next tokens' numbers are requested from memory before the current ones are worked on and wait in
// registers meanwhile, so memory latency and the barrier are paid once per 8 or 16 steps. The state is read from the
// sequence's slot unless the chunk starts at position 0, and written back after the chunk's last row: a decode row is
// a chunk of one, a prompt chunk walks its rows inside one launch.
// CHD (gated linear attention): the decay is one number per head and state row, a_t[n], staged beside k_t and q_t:
// S[n][p] <- a_t[n] S[n][p] + k_t[n] u[p]; with DELTA as well, the delta rule's read follows that per-row decay. A
// missing write strength means 1, one given as pre-activations (coef_sigmoid, row stride ldc) passes a sigmoid when
// staged; q_t is multiplied by q_scale when staged. A decay row stride of 0 (ldd) is one constant per head for every
// token (retention).
#include "../mx_common.h"

namespace {

template <int CTRL>
MX_DEV float dpp_add(float v) {
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
// sum over the LPC (4 or 16) neighbouring lanes of a column, returned to each of them
template <int LPC>
MX_DEV float lanes_sum(float v) {
    v = dpp_add<0xB1>(v);  // quad_perm [1, 0, 3, 2]
    v = dpp_add<0x4E>(v);  // quad_perm [2, 3, 0, 1]
    if constexpr (LPC == 16) {
        v = dpp_add<0x124>(v);  // row_ror 4
        v = dpp_add<0x128>(v);  // row_ror 8
    }
    return v;
}

// grid (column blocks, H, sequences); block = 256 threads = 256 / LPC columns
template <int NPL, int LPC, bool DELTA, bool CHD>
__global__ __launch_bounds__(256) void state_scan_kernel(const float* k, int ldk, const float* q, int ldq,
                                                         const float* v, int ldv, const float* decay, int ldd,
                                                         const float* coef, int ldc, int coef_sigmoid,
                                                         const float* skip, float* state, const int* seq_state,
                                                         const int* positions, int n_dec, const int* pf_cu, float* out,
                                                         int ldo, int H, int G, int N, int P, float q_scale) {
    static_assert(LPC == 4 || LPC == 16, "a column's lanes are a quad or a DPP row");
    constexpr int NT = 256;
    constexpr int NP = NPL * LPC;  // padded N
    constexpr int COLS = NT / LPC;
    constexpr int TB = NP <= 128 ? 16 : 8;  // tokens staged together
    constexpr int NW = CHD ? 3 : 2;  // vectors of N numbers staged per token: k, q (, channel decays)
    constexpr int KQ_PT = TB * NW * NP / NT, V_PT = (TB * COLS + NT - 1) / NT;
    __shared__ float kq[2][TB][NW][NP];
    __shared__ float vs[2][TB][COLS];
    __shared__ float ac[2][TB][2];
    const int cl = threadIdx.x / LPC;
    const int col = blockIdx.x * COLS + cl;
    const int part = threadIdx.x % LPC;
    const int h = blockIdx.y, s = blockIdx.z;
    int row0, n;
    if (s < n_dec) {
        row0 = s;
        n = 1;
    } else {
        const int i = s - n_dec;
        row0 = n_dec + pf_cu[i];
        n = pf_cu[i + 1] - pf_cu[i];
    }
    if (n <= 0) return;
    const int slot = seq_state[s];
    const bool fresh = positions[row0] == 0 || slot < 0;
    const bool live = col < P;
    const int g = h / (H / G);
    // addresses are clamped so that every load below is unconditional (all in flight together); what a lane must not
    // use is replaced by zero afterwards
    const int colc = min(col, P - 1);
    float* sp = state + (((long)(slot < 0 ? 0 : slot) * H + h) * P + colc) * N;
    const bool whole = N == NP && (N & 3) == 0;  // no padding: a lane's run is NPL aligned floats
    float S[NPL];
    if (whole) {
        const float4* s4 = (const float4*)(sp + part * NPL);
#pragma unroll
        for (int j = 0; j < NPL / 4; ++j) {
            const float4 x = s4[j];
            S[4 * j] = x.x;
            S[4 * j + 1] = x.y;
            S[4 * j + 2] = x.z;
            S[4 * j + 3] = x.w;
        }
    } else {
#pragma unroll
        for (int j = 0; j < NPL; ++j) S[j] = sp[min(part * NPL + j, N - 1)];
    }
    const bool keep = !fresh && live;
#pragma unroll
    for (int j = 0; j < NPL; ++j) S[j] = (keep && part * NPL + j < N) ? S[j] : 0.f;
    const float* kp = k + (long)g * N;
    const float* qp = q + (long)g * N;
    const float sk = skip ? skip[h] : 0.f;
    const int last = row0 + n - 1;
    // TB tokens' k, q, value, decay and write strength wait in registers while the TB tokens before them are worked
    // on, then move to LDS: memory latency is paid once per TB steps, and a barrier too
    float st_kq[KQ_PT], st_v[V_PT], st_ac = 0.f;
    // a round's loads are unconditional (clamped addresses, all in flight together) except that whole groups of NT
    // loads beyond the round's tokens are skipped by a block-uniform test: a decode row asks for one token's numbers,
    // not TB copies of them
    auto fetch = [&](int c) {
        const int r0 = row0 + c * TB;
        const int ntc = min(TB, n - c * TB);
#pragma unroll
        for (int i = 0; i < KQ_PT; ++i) {
            float x = 0.f;
            const int idx = threadIdx.x + i * NT;
            const int e = idx % NP;
            if (i * NT < ntc * NW * NP) {
                const int tt = idx / (NW * NP), w = (idx / NP) % NW;
                const long row = min(r0 + tt, last);
                const int ec = min(e, N - 1);
                if (CHD && w == 2) x = decay[row * ((long)H * N) + (long)h * N + ec];
                else x = w ? qp[row * ldq + ec] * q_scale : kp[row * ldk + ec];
            }
            st_kq[i] = e < N ? x : 0.f;
        }
#pragma unroll
        for (int i = 0; i < V_PT; ++i) {
            st_v[i] = 0.f;
            if (i * NT < ntc * COLS) {
                const int idx = min(threadIdx.x + i * NT, TB * COLS - 1);
                const int tt = idx / COLS, cc = idx % COLS;
                const long row = min(r0 + tt, last);
                st_v[i] = v[row * ldv + (long)h * P + min((int)blockIdx.x * COLS + cc, P - 1)];
            }
        }
        if (threadIdx.x < 2 * TB) {
            const long row = min(r0 + (int)threadIdx.x / 2, last);
            if (threadIdx.x & 1) {
                st_ac = coef ? coef[row * ldc + h] : 1.f;
                if (coef && coef_sigmoid) st_ac = 1.f / (1.f + expf(-st_ac));
            } else {
                st_ac = CHD ? 1.f : decay[row * ldd + h];
            }
        }
    };
    auto publish = [&](int b) {
#pragma unroll
        for (int i = 0; i < KQ_PT; ++i) (&kq[b][0][0][0])[threadIdx.x + i * NT] = st_kq[i];
#pragma unroll
        for (int i = 0; i < V_PT; ++i)
            if (threadIdx.x + i * NT < TB * COLS) (&vs[b][0][0])[threadIdx.x + i * NT] = st_v[i];
        if (threadIdx.x < 2 * TB) (&ac[b][0][0])[threadIdx.x] = st_ac;
    };
    const int nchunks = (n + TB - 1) / TB;
    fetch(0);
    publish(0);
    __syncthreads();
    for (int c = 0; c < nchunks; ++c) {
        const int b = c & 1;
        if (c + 1 < nchunks) fetch(c + 1);
        const int nt = min(TB, n - c * TB);
        for (int tt = 0; tt < nt; ++tt) {
            const int row = row0 + c * TB + tt;
            const float a = ac[b][tt][0], cf = ac[b][tt][1];
            const float vv = live ? vs[b][tt][cl] : 0.f;
            const float* kb = &kq[b][tt][0][part * NPL];
            const float* qb = &kq[b][tt][1][part * NPL];
            float u;
            if constexpr (DELTA) {
                float d0 = 0.f, d1 = 0.f;  // two chains instead of one of NPL dependent adds
                const float* ab = &kq[b][tt][NW - 1][part * NPL];  // (the channel decays; q's row when there are none)
#pragma unroll
                for (int j = 0; j < NPL; j += 2) {
                    S[j] *= CHD ? ab[j] : a;
                    S[j + 1] *= CHD ? ab[j + 1] : a;
                    d0 += S[j] * kb[j];
                    d1 += S[j + 1] * kb[j + 1];
                }
                u = cf * (vv - lanes_sum<LPC>(d0 + d1));
            } else if constexpr (CHD) {
                const float* ab = &kq[b][tt][NW - 1][part * NPL];
#pragma unroll
                for (int j = 0; j < NPL; ++j) S[j] *= ab[j];
                u = cf * vv;
            } else {
#pragma unroll
                for (int j = 0; j < NPL; ++j) S[j] *= a;
                u = cf * vv;
            }
            float o0 = 0.f, o1 = 0.f;
#pragma unroll
            for (int j = 0; j < NPL; j += 2) {
                S[j] += kb[j] * u;
                S[j + 1] += kb[j + 1] * u;
                o0 += S[j] * qb[j];
                o1 += S[j + 1] * qb[j + 1];
            }
            const float o = lanes_sum<LPC>(o0 + o1);
            if (live && part == 0) out[(long)row * ldo + (long)h * P + col] = o + sk * vv;
        }
        // the other buffer was last read while chunk c - 1 was worked on, before the barrier that ended that round
        if (c + 1 < nchunks) publish(b ^ 1);
        __syncthreads();
    }
    if (slot >= 0 && live) {
        if (whole) {
            float4* s4 = (float4*)(sp + part * NPL);
#pragma unroll
            for (int j = 0; j < NPL / 4; ++j) s4[j] = make_float4(S[4 * j], S[4 * j + 1], S[4 * j + 2], S[4 * j + 3]);
        } else {
#pragma unroll
            for (int j = 0; j < NPL; ++j)
                if (part * NPL + j < N) sp[part * NPL + j] = S[j];
        }
    }
}

}  // namespace

#define MXH_CHECK(cond) \
    if (!(cond)) return (int)hipErrorInvalidValue

extern "C" int mxh_state_scan(const float* k, int ldk, const float* q, int ldq, const float* v, int ldv,
                              const float* decay, int decay_rows, const float* coef, int ldc, int coef_sigmoid,
                              const float* skip, float* state, const int* seq_state, const int* positions, int n_dec,
                              const int* pf_cu, int n_pf, float* out, int ldo, int H, int G, int N, int P, int delta,
                              int channel, float q_scale, hipStream_t st) {
    const int n_seqs = n_dec + n_pf;
    if (n_seqs <= 0) return 0;
    MXH_CHECK(k && q && v && decay && state && seq_state && positions && out && (n_pf == 0 || pf_cu));
    MXH_CHECK((decay_rows || !channel) && (!coef || ldc >= H));  // decay_rows 0: one constant per head, [H]
    const int ldd = decay_rows ? H : 0;
    MXH_CHECK(H > 0 && G > 0 && H % G == 0 && N > 0 && N <= 256 && P > 0 && H <= 65535 && n_seqs <= 65535);
    MXH_CHECK(ldk >= G * N && ldq >= G * N && ldv >= H * P && ldo >= H * P);
    const int lpc = N <= 32 ? 4 : 16;
    const int threads = 256;
    const int cols = threads / lpc;
    const dim3 grid((P + cols - 1) / cols, H, n_seqs);
#define GO2(NPL, LPC, D_, C_)                                                                                      \
    state_scan_kernel<NPL, LPC, D_, C_><<<grid, threads, 0, st>>>(k, ldk, q, ldq, v, ldv, decay, ldd, coef, ldc,      \
                                                                  coef_sigmoid, skip, state, seq_state, positions,    \
                                                                  n_dec, pf_cu, out, ldo, H, G, N, P, q_scale)
#define GO(NPL, LPC)                              \
    do {                                          \
        if (delta && channel) GO2(NPL, LPC, true, true); \
        else if (delta) GO2(NPL, LPC, true, false);   \
        else if (channel) GO2(NPL, LPC, false, true); \
        else GO2(NPL, LPC, false, false);         \
    } while (0)
    if (N <= 16) GO(4, 4);
    else if (N <= 32) GO(8, 4);
    else if (N <= 64) GO(4, 16);
    else if (N <= 128) GO(8, 16);
    else GO(16, 16);
#undef GO
#undef GO2
    return (int)hipGetLastError();
}
