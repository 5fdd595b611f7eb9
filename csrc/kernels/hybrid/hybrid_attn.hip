// hybrid_attn.hip: causal softmax attention over paged key / value pools with a visible range that starts at a chunk
// border, a window's edge or position 0, and an optional sink term in the denominator (ops/hybrid.py
// masked_attention). Pools are token-major: keys [blocks, bs, G * dk], values [blocks, bs, G * dv], fp32 or bf16.
// The value pool may hold fewer heads than the key pool (gv of them, a divisor of G): key head g then reads value head
// g % gv, several attention maps over the same values. Every kernel also takes an AttnExtra: a learned sink score per
// head instead of 0, an additive bias looked up by the distance between query and key (table [H, distances], the last
// entry serving every larger distance), and a gate per row and head whose sigmoid multiplies the head's output.
//
// attn_rows_kernel: one wave per (query row, query head). Keys are taken 64 at a time, one per lane: the lane forms
// its key's whole score against the query (held in LDS as fp32, pre-multiplied by the scale), the wave updates the
// running maximum and sum (fp32), and the lanes then share out the value columns, each accumulating
// sum_j p_j v_j[c] for its columns over the tile's keys. Scores, softmax and accumulators are fp32 for both pool
// formats. The sink is a virtual key of score 0 and value 0: the running maximum starts at 0 and the sum at 1.
// With parts > 1 (decode rows of long contexts) grid.z splits a row's visible keys into partitions whose
// (max, sum, unnormalised output) go to a workspace; attn_merge_kernel combines them in a fixed order and adds the sink.
//
// bf16 pools with head sizes of 64 / 128 run on the matrix cores instead: attn_chunk_mfma_kernel for prompt chunks,
// attn_decode_mfma_kernel for single new tokens (both further down, with their fragment layouts).
//
// Other long prompt chunks take another route (ops/hybrid.py): kv_gather_kernel copies the chunk's visible keys and values
// from the pages into head-major matrices, head_transpose_kernel does the same for the queries, the library computes
// the score and value products, and masked_softmax_kernel turns raw scores into masked, sink-normalised weights.
#include "../mx_common.h"

namespace {

constexpr int DVU_MAX = 8;  // value columns per lane: heads of up to 512 numbers

struct AttnExtra {
    const float* sink_v;  // [H] sink scores (null: 0 where a sink is asked for)
    const float* bias;    // [H, nb] bias by distance (null: none)
    int nb;
    const float* gate;    // pre-sigmoid gate of row r and head h at gate[r * ldg + h] (null: none)
    int ldg;
    int gv;               // value heads in the pool: key head g reads value head g % gv
};
MX_DEV float sink_score(const AttnExtra& ex, int h) { return ex.sink_v ? ex.sink_v[h] : 0.f; }
MX_DEV float dist_bias(const AttnExtra& ex, int dist, int H, int h) {
    return ex.bias[(long)h * ex.nb + min(max(dist, 0), ex.nb - 1)];
}
MX_DEV float gate_factor(const AttnExtra& ex, long row, int h) {
    return ex.gate ? 1.f / (1.f + expf(-ex.gate[row * ex.ldg + h])) : 1.f;
}

template <bool B16>
MX_DEV float ld1(const void* p, long i) {
    if constexpr (B16) return bf16_to_f32(((const bf16_t*)p)[i]);
    else return ((const float*)p)[i];
}

MX_DEV float dot8(const uint4 w, const float* qq) {
    return __uint_as_float(w.x << 16) * qq[0] + __uint_as_float(w.x & 0xffff0000u) * qq[1] +
           __uint_as_float(w.y << 16) * qq[2] + __uint_as_float(w.y & 0xffff0000u) * qq[3] +
           __uint_as_float(w.z << 16) * qq[4] + __uint_as_float(w.z & 0xffff0000u) * qq[5] +
           __uint_as_float(w.w << 16) * qq[6] + __uint_as_float(w.w & 0xffff0000u) * qq[7];
}
MX_DEV float dot4(const float4 w, const float* qq) { return w.x * qq[0] + w.y * qq[1] + w.z * qq[2] + w.w * qq[3]; }

// dots of one pool row with REP fp32 queries in LDS (q + r * n; n numbers, row and queries 16-byte aligned when
// n % 8 == 0). Eight (fp32: four) 16-byte pieces of the row are requested before the first is used: a lane's loads
// are one dependent chain otherwise. The row is read once for all REP queries.
template <bool B16, int REP>
MX_DEV void dot_row(const void* base, long off, const float* q, int n, float (&acc)[REP]) {
#pragma unroll
    for (int r = 0; r < REP; ++r) acc[r] = 0.f;
    if ((n & 7) == 0) {
        if constexpr (B16) {
            const uint4* p = (const uint4*)((const bf16_t*)base + off);
            const int m = n / 8;
            int i = 0;
            for (; i + 8 <= m; i += 8) {
                uint4 w[8];  // (a struct type: kept in registers here only because every index is a constant after unrolling)
#pragma unroll
                for (int e = 0; e < 8; ++e) w[e] = p[i + e];
#pragma unroll
                for (int r = 0; r < REP; ++r) {
                    const float* qq = q + r * n + i * 8;
                    acc[r] += ((dot8(w[0], qq) + dot8(w[1], qq + 8)) + (dot8(w[2], qq + 16) + dot8(w[3], qq + 24))) +
                              ((dot8(w[4], qq + 32) + dot8(w[5], qq + 40)) + (dot8(w[6], qq + 48) + dot8(w[7], qq + 56)));
                }
            }
            for (; i + 4 <= m; i += 4) {
                const uint4 w0 = p[i], w1 = p[i + 1], w2 = p[i + 2], w3 = p[i + 3];
#pragma unroll
                for (int r = 0; r < REP; ++r) {
                    const float* qq = q + r * n + i * 8;
                    acc[r] += (dot8(w0, qq) + dot8(w1, qq + 8)) + (dot8(w2, qq + 16) + dot8(w3, qq + 24));
                }
            }
            for (; i < m; ++i) {
                const uint4 w0 = p[i];
#pragma unroll
                for (int r = 0; r < REP; ++r) acc[r] += dot8(w0, q + r * n + i * 8);
            }
        } else {
            const float4* p = (const float4*)((const float*)base + off);
            const int m = n / 4;
            int i = 0;
            for (; i + 4 <= m; i += 4) {
                const float4 w0 = p[i], w1 = p[i + 1], w2 = p[i + 2], w3 = p[i + 3];
#pragma unroll
                for (int r = 0; r < REP; ++r) {
                    const float* qq = q + r * n + i * 4;
                    acc[r] += (dot4(w0, qq) + dot4(w1, qq + 4)) + (dot4(w2, qq + 8) + dot4(w3, qq + 12));
                }
            }
            for (; i < m; ++i) {
                const float4 w0 = p[i];
#pragma unroll
                for (int r = 0; r < REP; ++r) acc[r] += dot4(w0, q + r * n + i * 4);
            }
        }
        return;
    }
    for (int i = 0; i < n; ++i) {
        const float w = ld1<B16>(base, off + i);
#pragma unroll
        for (int r = 0; r < REP; ++r) acc[r] += w * q[r * n + i];
    }
}

// grid (rows, H / REP, parts): a wave serves the REP query heads h0 .. h0 + REP - 1 of one row, which share a
// key / value head (REP divides H / G), so keys and values are read once for all of them. cu_q == nullptr: row r is
// sequence r's single new token at position ctx[r] - 1; otherwise rows are chunks laid end to end, sequence s owning
// rows [cu_q[s], cu_q[s + 1]) that end at position ctx[s] - 1.
template <bool B16, bool O16, int REP, int DVU>
__global__ __launch_bounds__(64) void attn_rows_kernel(const void* q, int ldq, const void* kc, const void* vc, int bs,
                                                       const int* bt, int bt_stride, const int* cu_q, const int* ctx,
                                                       int n_seqs, int row_base, void* out, int ldo, int H, int G,
                                                       int dk, int dv, float scale, int chunk, int window, int sink,
                                                       float out_scale, int row_off, int parts, int part_len,
                                                       float* part_ml, float* part_o, AttnExtra ex) {
    extern __shared__ float lds[];  // [REP][dk] queries, [REP][64] weights, [64] row offsets
    float* qs = lds;
    float* ps = lds + REP * dk;
    long* rowoff = (long*)(ps + REP * 64 + ((REP * dk) & 1));
    const int r = blockIdx.x + row_off, h0 = blockIdx.y * REP, lane = threadIdx.x, z = blockIdx.z;
    int s, pos;
    if (!cu_q) {
        s = r;
        pos = ctx[s] - 1;
    } else {
        int lo_ = 0, hi_ = n_seqs - 1;  // last s with cu_q[s] <= r
        while (lo_ < hi_) {
            const int mid = (lo_ + hi_ + 1) >> 1;
            if (cu_q[mid] <= r) lo_ = mid;
            else hi_ = mid - 1;
        }
        s = lo_;
        const int n = cu_q[s + 1] - cu_q[s];
        pos = ctx[s] - n + (r - cu_q[s]);
    }
    const int g = h0 / (H / G);
    const long qrow = (long)(row_base + r) * ldq + (long)h0 * dk;
    for (int e = lane; e < REP * dk; e += 64) qs[e] = ld1<B16>(q, qrow + e) * scale;
    int lo = chunk > 0 ? (pos / chunk) * chunk : window > 0 ? max(0, pos - window + 1) : 0;
    const int qpos = pos;
    if (parts > 1) {  // this partition's keys; the sink joins in the merge
        lo += z * part_len;
        pos = min(pos, lo + part_len - 1);
        sink = 0;
    }
    const int* table = bt + (long)s * bt_stride;
    float m[REP], l[REP], acc[REP][DVU];
#pragma unroll
    for (int i = 0; i < REP; ++i) {
        m[i] = sink ? sink_score(ex, h0 + i) : -INFINITY;
        l[i] = sink ? 1.f : 0.f;
#pragma unroll
        for (int u = 0; u < DVU; ++u) acc[i][u] = 0.f;
    }
    __syncthreads();
    for (int j0 = lo; j0 <= pos; j0 += 64) {
        const int j = j0 + lane;
        const bool ok = j <= pos;
        float sc[REP];
        long tok = 0;
        if (ok) {
            tok = (long)table[j / bs] * bs + (j % bs);
            dot_row<B16, REP>(kc, (tok * G + g) * dk, qs, dk, sc);
            if (ex.bias) {
#pragma unroll
                for (int i = 0; i < REP; ++i) sc[i] += dist_bias(ex, qpos - j, H, h0 + i);
            }
        }
        float alpha[REP], p[REP];
#pragma unroll
        for (int i = 0; i < REP; ++i) {
            const float si = ok ? sc[i] : -INFINITY;
            const float mn = fmaxf(m[i], wave_max(si));
            p[i] = ok ? expf(si - mn) : 0.f;
            alpha[i] = expf(m[i] - mn);  // 0 on the first tile without a sink (m = -inf, mn finite: the tile has key lo)
            l[i] = l[i] * alpha[i] + wave_sum(p[i]);
            m[i] = mn;
        }
        __syncthreads();  // the previous tile's weights and offsets have been read
#pragma unroll
        for (int i = 0; i < REP; ++i) ps[i * 64 + lane] = p[i];
        rowoff[lane] = (tok * ex.gv + g % ex.gv) * dv;
        __syncthreads();
        const int nk = min(64, pos - j0 + 1);
        // VB keys' values for all of the lane's columns are requested together (clamped columns: no branch between
        // the loads), then multiplied in
        constexpr int VB = DVU <= 2 ? 16 : 4;
#pragma unroll
        for (int i = 0; i < REP; ++i)
#pragma unroll
            for (int u = 0; u < DVU; ++u) acc[i][u] *= alpha[i];
        int jj = 0;
        for (; jj + VB <= nk; jj += VB) {
            float vv[DVU][VB];
#pragma unroll
            for (int u = 0; u < DVU; ++u)
#pragma unroll
                for (int e = 0; e < VB; ++e) vv[u][e] = ld1<B16>(vc, rowoff[jj + e] + min(lane + u * 64, dv - 1));
#pragma unroll
            for (int i = 0; i < REP; ++i)
#pragma unroll
                for (int u = 0; u < DVU; ++u)
#pragma unroll
                    for (int e = 0; e < VB; ++e) acc[i][u] += ps[i * 64 + jj + e] * vv[u][e];
        }
        for (; jj < nk; ++jj) {
#pragma unroll
            for (int u = 0; u < DVU; ++u) {
                const float vv = ld1<B16>(vc, rowoff[jj] + min(lane + u * 64, dv - 1));
#pragma unroll
                for (int i = 0; i < REP; ++i) acc[i][u] += ps[i * 64 + jj] * vv;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < REP; ++i) {
        const int h = h0 + i;
        if (parts > 1) {
            const long pr = ((long)r * H + h) * parts + z;
            if (lane == 0) {
                part_ml[pr * 2] = m[i];
                part_ml[pr * 2 + 1] = l[i];
            }
#pragma unroll
            for (int u = 0; u < DVU; ++u) {
                const int c = lane + u * 64;
                if (c < dv) part_o[pr * dv + c] = acc[i][u];
            }
            continue;
        }
        const float inv = out_scale / l[i] * gate_factor(ex, row_base + r, h);
        const long orow = (long)(row_base + r) * ldo + (long)h * dv;
#pragma unroll
        for (int u = 0; u < DVU; ++u) {
            const int c = lane + u * 64;
            if (c < dv) {
                if constexpr (O16) ((bf16_t*)out)[orow + c] = f32_to_bf16(acc[i][u] * inv);
                else ((float*)out)[orow + c] = acc[i][u] * inv;
            }
        }
    }
}

// Staging of a key tile [KT][DK] and a value tile [KT][DV] (both row-major, padded rows) by NTH threads: 16-byte pieces wait in
// registers (tile_load) until the previous tile has been worked on, then go to LDS (tile_store). Plain functions over
// array references: the pieces stay in registers.
template <int DK, int DV, int KT, int NTH>
MX_DEV void tile_load(u32x4 (&kr)[KT * DK / 8 / NTH], u32x4 (&vr)[KT * DV / 8 / NTH], const bf16_t* __restrict__ kc,
                      const bf16_t* __restrict__ vc, const int* __restrict__ table, int bs, int G, int kvh, int Gv,
                      int kt0, int kv_end, int tid) {
    const int vh = kvh % Gv;
#pragma unroll
    for (int j = 0; j < KT * DK / 8 / NTH; ++j) {
        const int id = tid + j * NTH;
        const int p = id / (DK / 8), c = id % (DK / 8);
        const int pos = min(kt0 + p, kv_end - 1);  // clamped: keys past the end are masked by the caller
        const size_t tok = (size_t)table[pos / bs] * bs + (pos % bs);
        kr[j] = *(const u32x4*)(kc + (tok * G + kvh) * DK + c * 8);
    }
#pragma unroll
    for (int j = 0; j < KT * DV / 8 / NTH; ++j) {
        const int id = tid + j * NTH;
        const int p = id / (DV / 8), c = id % (DV / 8);
        const int pos = min(kt0 + p, kv_end - 1);
        const size_t tok = (size_t)table[pos / bs] * bs + (pos % bs);
        vr[j] = *(const u32x4*)(vc + (tok * Gv + vh) * DV + c * 8);
    }
}
template <int DK, int DV, int KT, int NTH, int KSTR, int VSTR>
MX_DEV void tile_store(const u32x4 (&kr)[KT * DK / 8 / NTH], const u32x4 (&vr)[KT * DV / 8 / NTH], char* k_lds,
                       char* v_lds, int tid) {
#pragma unroll
    for (int j = 0; j < KT * DK / 8 / NTH; ++j) {
        const int id = tid + j * NTH;
        const int p = id / (DK / 8), c = id % (DK / 8);
        *(u32x4*)(k_lds + p * KSTR + c * 16) = kr[j];
    }
#pragma unroll
    for (int j = 0; j < KT * DV / 8 / NTH; ++j) {
        const int id = tid + j * NTH;
        const int p = id / (DV / 8), c = id % (DV / 8);
        *(u32x4*)(v_lds + p * VSTR + c * 16) = vr[j];
    }
}

// B fragment of O += P V from a row-major value tile in LDS (row = key, VSTR bytes apart): the values of keys
// r0 .. r0 + 7 at dim 16 nt + col, through the transposing LDS read (each lane of a 16-lane group hands in 4 dims of one
// key and receives one dim of 4 keys). The result is reinterpreted as a whole vector.
template <int VSTR>
MX_DEV bf16x8 v_fragment(const char* v_lds, int r0, int nt, int col) {
    const int q4 = col >> 2, p4 = col & 3;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MX_LDS s16x4*)(v_lds + (r0 + q4) * VSTR + 32 * nt + 8 * p4));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MX_LDS s16x4*)(v_lds + (r0 + 4 + q4) * VSTR + 32 * nt + 8 * p4));
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    const u32x4 w4 = {l2[0], l2[1], h2[0], h2[1]};
    return __builtin_bit_cast(bf16x8, w4);
}

// attn_chunk_mfma_kernel: a prompt chunk of one sequence on the matrix cores (bf16 pools, head sizes that are
// multiples of 32 / 16). A workgroup of 4 waves owns RT 16-row query tiles of GW query heads that share a key / value
// head (GW * RT = 4); a wave owns one tile of one head, its query fragments in registers. Keys are taken 64 at a time:
// the workgroup stages the key tile [64][DK] and the value tile [64][DV] in LDS (the next tile's numbers are
// requested from memory before the current tile is worked on and wait in registers), each wave forms S = Q K^T with
// MFMA 16x16x32, masks (causal, chunk or window start) and updates its rows' running maximum and sum in fp32 (the sink
// starts them at 0 and 1), writes the weights as bf16 to its own LDS patch and accumulates O += P V, the value
// fragments coming out of LDS through the transposing read.
// Fragment layout of v_mfma_f32_16x16x32_bf16 (g = lane / 16, col = lane % 16): A holds row col, k = 8g .. 8g + 7;
// B holds column col, k = 8g .. 8g + 7; the result holds rows 4g .. 4g + 3 of column col.
// P2: every softmax weight enters the value product as two bf16 numbers (its rounding, and the rounding of what that
// lost) in two products that share the value fragment, so the weights count to 16 bits of mantissa.
template <int DK, int DV, bool O16, bool P2>
__global__ __launch_bounds__(256) void attn_chunk_mfma_kernel(const bf16_t* __restrict__ q, int ldq,
                                                              const bf16_t* __restrict__ kc,
                                                              const bf16_t* __restrict__ vc, int bs,
                                                              const int* __restrict__ table, int p0, int n, void* out,
                                                              int ldo, int H, int G, int GW, float scale, int chunk,
                                                              int window, int sink, float out_scale, AttnExtra ex) {
    constexpr int KT = 64;
    constexpr int KSTR = (DK + 8) * 2;  // bytes per key row in LDS (padded)
    constexpr int VSTR = (DV + 8) * 2;  // bytes per value row in LDS (padded)
    constexpr int PSTR = (KT + 8) * 2;  // bytes per weight row
    constexpr float LOG2E_ = 1.4426950408889634f;
    __shared__ __attribute__((aligned(16))) char k_lds[KT * KSTR];
    __shared__ __attribute__((aligned(16))) char v_lds[KT * VSTR];
    __shared__ __attribute__((aligned(16))) char p_lds[(P2 ? 2 : 1) * 4 * 16 * PSTR];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int g = lane >> 4, col = lane & 15;
    const int RT = 4 / GW;
    const int hq = blockIdx.y * GW + (wave % GW);
    const int kvh = (blockIdx.y * GW) / (H / G);
    // the chunk's last rows see the most keys: their workgroups are scheduled first
    const int q0 = (gridDim.x - 1 - blockIdx.x) * RT * 16;  // first query row of the workgroup
    const int row_q0 = q0 + (wave / GW) * 16;     // first query row of this wave
    const int a_pos = p0 + q0;                    // position of the workgroup's first row
    const int kv_end = p0 + min(n, q0 + RT * 16);  // one past the last visible key
    const int kt_begin = chunk > 0 ? (a_pos / chunk) * chunk : window > 0 ? max(0, a_pos - window + 1) : 0;
    const float qs = scale * LOG2E_;

    bf16x8 qf[DK / 32];
    {
        const int qi = row_q0 + col;
#pragma unroll
        for (int ks = 0; ks < DK / 32; ++ks) {
            if (qi < n) qf[ks] = *(const bf16x8*)(q + (size_t)qi * ldq + (size_t)hq * DK + 32 * ks + 8 * g);
            else qf[ks] = (bf16x8){};
        }
    }
    f32x4 oacc[DV / 16];
#pragma unroll
    for (int i = 0; i < DV / 16; ++i) oacc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float mrow[4], lrow[4];
    int lo_row[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        mrow[i] = sink ? sink_score(ex, hq) * LOG2E_ : -INFINITY;
        lrow[i] = sink ? 1.f : 0.f;
        const int qpos = p0 + row_q0 + 4 * g + i;
        lo_row[i] = chunk > 0 ? (qpos / chunk) * chunk : window > 0 ? max(0, qpos - window + 1) : 0;
    }
    char* pw = p_lds + wave * 16 * PSTR;
    char* pw2 = pw + (P2 ? 4 * 16 * PSTR : 0);  // the weights' second halves

    constexpr int KCH = KT * DK / 8 / 256, VCH = KT * DV / 8 / 256;  // 16-byte pieces per thread
    u32x4 kr[KCH], vr[VCH];
#define LOAD_TILE(kt0_) tile_load<DK, DV, KT, 256>(kr, vr, kc, vc, table, bs, G, kvh, ex.gv, kt0_, kv_end, threadIdx.x)
#define STORE_TILE() tile_store<DK, DV, KT, 256, KSTR, VSTR>(kr, vr, k_lds, v_lds, threadIdx.x)
    if (kt_begin < kv_end) LOAD_TILE(kt_begin);
    for (int kt0 = kt_begin; kt0 < kv_end; kt0 += KT) {
        STORE_TILE();
        if (kt0 + KT < kv_end) LOAD_TILE(kt0 + KT);
        __syncthreads();
        // ---- S = Q K^T : 16 rows x 64 keys ----
        f32x4 sacc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            sacc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < DK / 32; ++ks) {
                const bf16x8 kf = *(const bf16x8*)(k_lds + (16 * t + col) * KSTR + (32 * ks + 8 * g) * 2);
                sacc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], kf, sacc[t], 0, 0, 0);
            }
        }
        // ---- bias by distance: row 4g + i against key 16t + col lies d0 + i - 16t keys back. When every distance
        // of the wave's 16 rows against the tile's 64 keys lies inside the table (a wave-uniform test) the 16 entries
        // are read at constant offsets from one address; the diagonal tile and tiles beyond the table clamp ----
        if (ex.bias) {
            const float* bp = ex.bias + (size_t)hq * ex.nb;
            const int d0 = p0 + row_q0 + 4 * g - kt0 - col;
            const int dmin = p0 + row_q0 - (kt0 + KT - 1), dmax = p0 + row_q0 + 15 - kt0;
            if (dmin >= 0 && dmax < ex.nb) {
                const float* pp = bp + d0;
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) sacc[t][i] = sacc[t][i] * qs + pp[i - 16 * t] * LOG2E_;
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        sacc[t][i] = sacc[t][i] * qs + bp[min(max(d0 + i - 16 * t, 0), ex.nb - 1)] * LOG2E_;
            }
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) sacc[t][i] *= qs;
        }
        // ---- mask + online softmax in base 2 (rows 4g + i, keys 16t + col) ----
        float alpha[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int qi = row_q0 + 4 * g + i;
            const int qpos = p0 + qi;
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int kp = kt0 + 16 * t + col;
                float v = sacc[t][i];
                if (kp > qpos || kp < lo_row[i] || qi >= n) v = -INFINITY;
                sacc[t][i] = v;
                mx = fmaxf(mx, v);
            }
            const float mn = fmaxf(mrow[i], group_max<16>(mx));
            alpha[i] = mn == -INFINITY ? 1.f : exp2f(mrow[i] - mn);
            float rs = 0.f;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const float pv = mn == -INFINITY ? 0.f : exp2f(sacc[t][i] - mn);
                sacc[t][i] = pv;
                rs += pv;
            }
            lrow[i] = lrow[i] * alpha[i] + group_sum<16>(rs);
            mrow[i] = mn;
        }
#pragma unroll
        for (int nt = 0; nt < DV / 16; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) oacc[nt][i] *= alpha[i];
        // ---- P -> LDS (bf16), read back as the next A fragments by the same wave ----
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bf16_t hi = f32_to_bf16(sacc[t][i]);
                *(bf16_t*)(pw + (4 * g + i) * PSTR + (16 * t + col) * 2) = hi;
                if constexpr (P2)
                    *(bf16_t*)(pw2 + (4 * g + i) * PSTR + (16 * t + col) * 2) = f32_to_bf16(sacc[t][i] - bf16_to_f32(hi));
            }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's own LDS writes have landed
        __builtin_amdgcn_wave_barrier();
        // ---- O += P V ----
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const bf16x8 pa = *(const bf16x8*)(pw + col * PSTR + (32 * ks + 8 * g) * 2);
            const bf16x8 pb = *(const bf16x8*)(pw2 + col * PSTR + (32 * ks + 8 * g) * 2);
#pragma unroll
            for (int nt = 0; nt < DV / 16; ++nt) {
                const auto vf = v_fragment<VSTR>(v_lds, 32 * ks + 8 * g, nt, col);
                oacc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, vf, oacc[nt], 0, 0, 0);
                if constexpr (P2) oacc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pb, vf, oacc[nt], 0, 0, 0);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int qi = row_q0 + 4 * g + i;
        if (qi >= n) continue;
        const float inv = lrow[i] > 0.f ? out_scale / lrow[i] * gate_factor(ex, qi, hq) : 0.f;
#pragma unroll
        for (int nt = 0; nt < DV / 16; ++nt) {
            const size_t o = (size_t)qi * ldo + (size_t)hq * DV + 16 * nt + col;
            if constexpr (O16) ((bf16_t*)out)[o] = f32_to_bf16(oacc[nt][i] * inv);
            else ((float*)out)[o] = oacc[nt][i] * inv;
        }
    }
}

// attn_decode_mfma_kernel: single new tokens on the matrix cores (bf16 pools, head sizes 64 / 128, up to 16 query heads
// per key / value head). grid (sequences, G, partitions), one wave per workgroup: the 16 rows of its tile are the
// query heads that share key / value head blockIdx.y (rows beyond H / G are zero), all at the sequence's newest
// position, so a key and value tile is read once for all of them. The wave walks its partition's keys
// as attn_chunk_mfma_kernel does, 32 at a time (key fragments straight from the pages, values staged in LDS by the
// wave itself, the next tile requested ahead). With one
// partition it writes the result, otherwise (max, sum, unnormalised output) for attn_merge_kernel; the running maximum
// is kept in base 2 and handed over in base e.
template <int DK, int DV, bool O16, bool P2>
__global__ __launch_bounds__(64) void attn_decode_mfma_kernel(const bf16_t* __restrict__ q, int ldq,
                                                              const bf16_t* __restrict__ kc,
                                                              const bf16_t* __restrict__ vc, int bs,
                                                              const int* __restrict__ bt, int bt_stride,
                                                              const int* __restrict__ ctx, void* out, int ldo, int H,
                                                              int G, float scale, int chunk, int window, int sink,
                                                              float out_scale, int parts, int part_len,
                                                              float* __restrict__ part_ml, float* __restrict__ part_o,
                                                              AttnExtra ex) {
    constexpr int KT = 32;  // keys per tile: the wave stages its tiles alone, 64 keys would not fit its registers
    constexpr int VSTR = (DV + 8) * 2, PSTR = (KT + 8) * 2;
    constexpr float LOG2E_ = 1.4426950408889634f, LN2_ = 0.6931471805599453f;
    __shared__ __attribute__((aligned(16))) char v_lds[KT * VSTR];
    __shared__ __attribute__((aligned(16))) char pw[(P2 ? 2 : 1) * 16 * PSTR];
    char* pw2 = pw + (P2 ? 16 * PSTR : 0);  // the weights' second halves (P2 as in attn_chunk_mfma_kernel)
    const int lane = threadIdx.x, g = lane >> 4, col = lane & 15;
    const int s = blockIdx.x, kvh = blockIdx.y, z = blockIdx.z;
    const int rep = H / G;
    const int qpos = ctx[s] - 1;
    int lo = chunk > 0 ? (qpos / chunk) * chunk : window > 0 ? max(0, qpos - window + 1) : 0;
    int kv_end = qpos + 1;
    if (parts > 1) {
        lo += z * part_len;
        kv_end = min(kv_end, lo + part_len);
        sink = 0;  // joins in the merge
    }
    int hrow[4];  // query head of each of the lane's result rows (rows beyond the group repeat its last head)
#pragma unroll
    for (int i = 0; i < 4; ++i) hrow[i] = kvh * (H / G) + min(4 * g + i, H / G - 1);
    const int* table = bt + (size_t)s * bt_stride;
    const float qs = scale * LOG2E_;
    bf16x8 qf[DK / 32];
    {
        const bf16_t* qp = q + (size_t)s * ldq + (size_t)(kvh * rep + min(col, rep - 1)) * DK + 8 * g;
#pragma unroll
        for (int ks = 0; ks < DK / 32; ++ks) {
            const uint4 w = *(const uint4*)(qp + 32 * ks);
            const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
            qf[ks] = __builtin_bit_cast(bf16x8, col < rep ? w : zero);
        }
    }
    f32x4 oacc[DV / 16];
#pragma unroll
    for (int i = 0; i < DV / 16; ++i) oacc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float mrow[4], lrow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        mrow[i] = sink ? sink_score(ex, hrow[i]) * LOG2E_ : -INFINITY;
        lrow[i] = sink ? 1.f : 0.f;
    }
    // key fragments come straight from the pages (lane (g, col) of tile t: key 16 t + col, dims 32 ks + 8 g .. + 7 are 16
    // contiguous bytes); values are staged row-major in LDS. Both are requested one tile ahead.
    constexpr int VCH = KT * DV / 8 / 64;  // 16-byte value pieces per lane
    u32x4 kf[KT / 16][DK / 32], vr[VCH];
    auto load_tile = [&](int kt0) {
#pragma unroll
        for (int t = 0; t < KT / 16; ++t) {
            const int pos = min(kt0 + 16 * t + col, kv_end - 1);  // clamped: keys past the end are masked below
            const bf16_t* kp = kc + (((size_t)table[pos / bs] * bs + (pos % bs)) * G + kvh) * DK + 8 * g;
#pragma unroll
            for (int ks = 0; ks < DK / 32; ++ks) kf[t][ks] = *(const u32x4*)(kp + 32 * ks);
        }
#pragma unroll
        for (int j = 0; j < VCH; ++j) {
            const int id = lane + j * 64;
            const int p = id / (DV / 8), c = id % (DV / 8);
            const int pos = min(kt0 + p, kv_end - 1);
            vr[j] = *(const u32x4*)(vc + (((size_t)table[pos / bs] * bs + (pos % bs)) * ex.gv + kvh % ex.gv) * DV + c * 8);
        }
    };
    if (lo < kv_end) load_tile(lo);
    for (int kt0 = lo; kt0 < kv_end; kt0 += KT) {
        __syncthreads();  // (one wave: orders the previous tile's LDS reads before these writes)
#pragma unroll
        for (int j = 0; j < VCH; ++j) {
            const int id = lane + j * 64;
            *(u32x4*)(v_lds + (id / (DV / 8)) * VSTR + (id % (DV / 8)) * 16) = vr[j];
        }
        f32x4 sacc[KT / 16];
#pragma unroll
        for (int t = 0; t < KT / 16; ++t) {
            sacc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < DK / 32; ++ks)
                sacc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], __builtin_bit_cast(bf16x8, kf[t][ks]), sacc[t],
                                                                  0, 0, 0);
        }
        if (kt0 + KT < kv_end) load_tile(kt0 + KT);
        // bias by distance: every row (query head) of the tile is at the same position, key 16t + col lies
        // qpos - kt0 - col - 16t keys back; each head has its own table row
        if (ex.bias) {
            const int d0 = qpos - kt0 - col;
            const bool inside = qpos - (kt0 + KT - 1) >= 0 && qpos - kt0 < ex.nb;  // wave-uniform: no clamps needed
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float* bp = ex.bias + (size_t)hrow[i] * ex.nb;
#pragma unroll
                for (int t = 0; t < KT / 16; ++t) {
                    const int d = inside ? d0 - 16 * t : min(max(d0 - 16 * t, 0), ex.nb - 1);
                    sacc[t][i] = sacc[t][i] * qs + bp[d] * LOG2E_;
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int t = 0; t < KT / 16; ++t) sacc[t][i] *= qs;
        }
        float alpha[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < KT / 16; ++t) {
                const int kp = kt0 + 16 * t + col;
                float v = sacc[t][i];
                if (kp >= kv_end) v = -INFINITY;
                sacc[t][i] = v;
                mx = fmaxf(mx, v);
            }
            const float mn = fmaxf(mrow[i], group_max<16>(mx));
            alpha[i] = mn == -INFINITY ? 1.f : exp2f(mrow[i] - mn);
            float rs = 0.f;
#pragma unroll
            for (int t = 0; t < KT / 16; ++t) {
                const float pv = mn == -INFINITY ? 0.f : exp2f(sacc[t][i] - mn);
                sacc[t][i] = pv;
                rs += pv;
            }
            lrow[i] = lrow[i] * alpha[i] + group_sum<16>(rs);
            mrow[i] = mn;
        }
#pragma unroll
        for (int nt = 0; nt < DV / 16; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) oacc[nt][i] *= alpha[i];
#pragma unroll
        for (int t = 0; t < KT / 16; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bf16_t hi = f32_to_bf16(sacc[t][i]);
                *(bf16_t*)(pw + (4 * g + i) * PSTR + (16 * t + col) * 2) = hi;
                if constexpr (P2)
                    *(bf16_t*)(pw2 + (4 * g + i) * PSTR + (16 * t + col) * 2) = f32_to_bf16(sacc[t][i] - bf16_to_f32(hi));
            }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < KT / 32; ++ks) {
            const bf16x8 pa = *(const bf16x8*)(pw + col * PSTR + (32 * ks + 8 * g) * 2);
            const bf16x8 pb = *(const bf16x8*)(pw2 + col * PSTR + (32 * ks + 8 * g) * 2);
#pragma unroll
            for (int nt = 0; nt < DV / 16; ++nt) {
                const auto vf = v_fragment<VSTR>(v_lds, 32 * ks + 8 * g, nt, col);
                oacc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, vf, oacc[nt], 0, 0, 0);
                if constexpr (P2) oacc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pb, vf, oacc[nt], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = 4 * g + i;
        if (r >= rep) continue;
        const int h = kvh * rep + r;
        if (parts > 1) {
            const size_t pr = ((size_t)s * H + h) * parts + z;
            if (col == 0) {
                part_ml[pr * 2] = mrow[i] * LN2_;
                part_ml[pr * 2 + 1] = lrow[i];
            }
#pragma unroll
            for (int nt = 0; nt < DV / 16; ++nt) part_o[pr * DV + 16 * nt + col] = oacc[nt][i];
            continue;
        }
        const float inv = lrow[i] > 0.f ? out_scale / lrow[i] * gate_factor(ex, s, h) : 0.f;
#pragma unroll
        for (int nt = 0; nt < DV / 16; ++nt) {
            const size_t o = (size_t)s * ldo + (size_t)h * DV + 16 * nt + col;
            if constexpr (O16) ((bf16_t*)out)[o] = f32_to_bf16(oacc[nt][i] * inv);
            else ((float*)out)[o] = oacc[nt][i] * inv;
        }
    }
}

#undef LOAD_TILE
#undef STORE_TILE

// grid (rows, H): combines the partitions of a row (at most 64: lane z holds partition z's maximum and sum) in a fixed
// order; an empty partition has sum 0
template <bool O16>
__global__ __launch_bounds__(64) void attn_merge_kernel(const float* part_ml, const float* part_o, int parts, int H,
                                                        int dv, int sink, float out_scale, int row_base, void* out,
                                                        int ldo, AttnExtra ex) {
    constexpr int DVU = DVU_MAX;
    const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const long p0 = ((long)r * H + h) * parts;
    const int zc = min(lane, parts - 1);
    const float mz = part_ml[(p0 + zc) * 2], lz = lane < parts ? part_ml[(p0 + zc) * 2 + 1] : 0.f;
    float M = wave_max(lz > 0.f ? mz : -INFINITY);
    const float s0 = sink_score(ex, h);
    if (sink) M = fmaxf(M, s0);
    const float w = lz > 0.f ? expf(mz - M) : 0.f;
    const float L = wave_sum(lz * w) + (sink ? expf(s0 - M) : 0.f);
    const float inv = out_scale / L * gate_factor(ex, row_base + r, h);
    const long orow = (long)(row_base + r) * ldo + (long)h * dv;
#pragma unroll
    for (int u = 0; u < DVU; ++u) {
        const int c = lane + u * 64;
        if (u * 64 < dv) {
            const int cc = min(c, dv - 1);
            float a = 0.f;
            for (int z0 = 0; z0 < parts; z0 += 8) {  // eight partitions' numbers requested together
                float x[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = part_o[(p0 + min(z0 + e, parts - 1)) * dv + cc];
#pragma unroll
                for (int e = 0; e < 8; ++e) a += x[e] * __shfl(w, min(z0 + e, 63), 64) * (z0 + e < parts ? 1.f : 0.f);
            }
            if (c < dv) {
                if constexpr (O16) ((bf16_t*)out)[orow + c] = f32_to_bf16(a * inv);
                else ((float*)out)[orow + c] = a * inv;
            }
        }
    }
}

// grid (keys, G): key jj of the range is the token at position lo + jj of the sequence whose block table is `table`;
// its group's key and value rows go to kh [G][n][dk] and vh [G][n][dv] (the value row of head g % Gv)
template <typename E>
__global__ __launch_bounds__(64) void kv_gather_kernel(const E* kc, const E* vc, int bs, const int* table, int lo, int n,
                                                       int G, int dk, int dv, E* kh, E* vh, int Gv) {
    const int jj = blockIdx.x, g = blockIdx.y;
    const int j = lo + jj;
    const long tok = (long)table[j / bs] * bs + (j % bs);
    const E* ks = kc + (tok * G + g) * dk;
    const E* vs = vc + (tok * Gv + g % Gv) * dv;
    E* kd = kh + ((long)g * n + jj) * dk;
    E* vd = vh + ((long)g * n + jj) * dv;
    for (int e = threadIdx.x; e < dk; e += 64) kd[e] = ks[e];
    for (int e = threadIdx.x; e < dv; e += 64) vd[e] = vs[e];
}

// grid (n, H): dst[i * d_si + h * d_sh + e] = scale * src[i * s_si + h * s_sh + e], e < d
template <bool S16, bool D16>
__global__ __launch_bounds__(64) void head_transpose_kernel(const void* src, long s_si, long s_sh, void* dst, long d_si,
                                                            long d_sh, int d, float scale, const float* gate, int ldg) {
    const long so = blockIdx.x * s_si + blockIdx.y * s_sh, dof = blockIdx.x * d_si + blockIdx.y * d_sh;
    if (gate) scale /= 1.f + expf(-gate[(long)blockIdx.x * ldg + blockIdx.y]);  // sigmoid gate of (row, head)
    for (int e = threadIdx.x; e < d; e += 64) {
        const float v = ld1<S16>(src, so + e) * scale;
        if constexpr (D16) ((bf16_t*)dst)[dof + e] = f32_to_bf16(v);
        else ((float*)dst)[dof + e] = v;
    }
}

// grid (H * n): row (h, i) holds the raw scores of the query at position p0 + i against the keys at positions
// key0 .. key0 + nk - 1. Writes the masked, sink-normalised softmax weights (zeros outside the visible range). With
// `two` (bf16 weights) a row of the output holds 2 nk numbers: every weight's bf16 rounding, then the bf16 roundings
// of what the first rounding lost, so that a product with the values stacked twice sees 16 bits of each weight.
template <bool P16>
__global__ __launch_bounds__(256) void masked_softmax_kernel(const float* sc, void* pw, int n, int nk, int p0, int key0,
                                                             float scale, int chunk, int window, int sink,
                                                             const float* sink_v, const float* bias, int nb, int H,
                                                             int two) {
    __shared__ float red[4];
    const long row = blockIdx.x;
    const int i = (int)(row % n), h = (int)(row / n);
    const int pos = p0 + i;
    const int lo = chunk > 0 ? (pos / chunk) * chunk : window > 0 ? max(0, pos - window + 1) : 0;
    const int a = max(lo, key0) - key0, b = min(pos - key0, nk - 1);  // visible local range [a, b]
    const float* s = sc + row * nk;
    const float s0 = sink_v ? sink_v[h] : 0.f;
    const int d0 = pos - key0;  // distance of local key j: d0 - j
    auto score = [&](int j) { return s[j] * scale + (bias ? bias[(long)h * nb + min(d0 - j, nb - 1)] : 0.f); };
    float m = sink ? s0 : -INFINITY;
    for (int j = a + threadIdx.x; j <= b; j += 256) m = fmaxf(m, score(j));
    m = block_max<256>(m, red);
    float l = 0.f;
    for (int j = a + threadIdx.x; j <= b; j += 256) l += expf(score(j) - m);
    l = block_sum<256>(l, red) + (sink ? expf(s0 - m) : 0.f);
    const float inv = 1.f / l;
    for (int j = threadIdx.x; j < nk; j += 256) {
        const float p = (j >= a && j <= b) ? expf(score(j) - m) * inv : 0.f;
        if constexpr (P16) {
            const bf16_t hi = f32_to_bf16(p);
            if (two) {
                ((bf16_t*)pw)[row * 2 * nk + j] = hi;
                ((bf16_t*)pw)[row * 2 * nk + nk + j] = f32_to_bf16(p - bf16_to_f32(hi));
            } else {
                ((bf16_t*)pw)[row * nk + j] = hi;
            }
        } else {
            ((float*)pw)[row * nk + j] = p;
        }
    }
}

}  // namespace

#define MXH_CHECK(cond) \
    if (!(cond)) return (int)hipErrorInvalidValue

extern "C" int mxh_attention(const void* q, int ldq, int q16, const void* kc, const void* vc, int bs, const int* bt,
                             int bt_stride, const int* cu_q, const int* ctx, int n_seqs, int n_rows, int row_base,
                             void* out, int ldo, int o16, int H, int G, int dk, int dv, float scale, int chunk,
                             int window, int sink, float out_scale, int row_off, int parts, int part_len,
                             float* part_ml, float* part_o, const float* sink_v, const float* bias, int nb,
                             const float* gate, int ldg, int gv, hipStream_t st) {
    if (n_rows <= 0 || n_seqs <= 0) return 0;
    MXH_CHECK((!bias || nb > 0) && (!gate || ldg >= H) && (!sink_v || sink) && gv > 0 && G % gv == 0);
    const AttnExtra ex = {sink_v, bias, nb, gate, ldg, gv};
    MXH_CHECK(q && kc && vc && bt && ctx && out && bs > 0 && bt_stride > 0);
    MXH_CHECK(H > 0 && G > 0 && H % G == 0 && dk > 0 && dv > 0 && dv <= 64 * DVU_MAX && dk <= 4096);
    MXH_CHECK(ldq >= H * dk && ldo >= H * dv && chunk >= 0 && window >= 0 && H <= 65535 && row_off >= 0);
    MXH_CHECK(cu_q || (row_off == 0 && n_rows == n_seqs));
    MXH_CHECK(parts >= 1 && parts <= 64 && (parts == 1 || (!cu_q && part_len > 0 && part_ml && part_o)));
    // REP query heads that share a key / value head could go to one wave (the kernel takes REP as a parameter), but a
    // wave that serves four heads measured 3.7x slower than four waves that serve one each: the row kernel is bound by
    // its dependent chains, not by the loads it would save. One head per wave.
    constexpr int REP = 1;
    const dim3 grid(n_rows, H / REP, parts);
    const size_t sh = (size_t)(REP * dk + REP * 64 + 2) * sizeof(float) + 64 * sizeof(long);
#define GO3(B, O, R, D)                                                                                               \
    attn_rows_kernel<B, O, R, D><<<grid, 64, sh, st>>>(q, ldq, kc, vc, bs, bt, bt_stride, cu_q, ctx, n_seqs, row_base, \
                                                       out, ldo, H, G, dk, dv, scale, chunk, window, sink, out_scale, \
                                                       row_off, parts, part_len, part_ml, part_o, ex)
#define GO(B, O)                                  \
    do {                                          \
        if (dv <= 128) GO3(B, O, REP, 2);         \
        else GO3(B, O, REP, DVU_MAX);             \
    } while (0)
    if (q16 && o16) GO(true, true);
    else if (q16) GO(true, false);
    else if (o16) GO(false, true);
    else GO(false, false);
#undef GO
#undef GO3
    if (parts > 1) {
        const dim3 g2(n_rows, H);
        if (o16) attn_merge_kernel<true><<<g2, 64, 0, st>>>(part_ml, part_o, parts, H, dv, sink, out_scale, row_base, out, ldo, ex);
        else attn_merge_kernel<false><<<g2, 64, 0, st>>>(part_ml, part_o, parts, H, dv, sink, out_scale, row_base, out, ldo, ex);
    }
    return (int)hipGetLastError();
}

extern "C" int mxh_kv_gather(const void* kc, const void* vc, int is16, int bs, const int* table, int lo, int n, int G,
                             int dk, int dv, void* kh, void* vh, int Gv, hipStream_t st) {
    if (n <= 0) return 0;
    MXH_CHECK(kc && vc && table && kh && vh && bs > 0 && lo >= 0 && G > 0 && G <= 65535 && dk > 0 && dv > 0);
    MXH_CHECK(Gv > 0 && G % Gv == 0);
    const dim3 grid(n, G);
    if (is16) kv_gather_kernel<bf16_t><<<grid, 64, 0, st>>>((const bf16_t*)kc, (const bf16_t*)vc, bs, table, lo, n, G, dk,
                                                           dv, (bf16_t*)kh, (bf16_t*)vh, Gv);
    else kv_gather_kernel<float><<<grid, 64, 0, st>>>((const float*)kc, (const float*)vc, bs, table, lo, n, G, dk, dv,
                                                      (float*)kh, (float*)vh, Gv);
    return (int)hipGetLastError();
}

extern "C" int mxh_head_transpose(const void* src, int s16, long s_si, long s_sh, void* dst, int d16, long d_si,
                                  long d_sh, int n, int H, int d, float scale, const float* gate, int ldg,
                                  hipStream_t st) {
    if (n <= 0) return 0;
    MXH_CHECK(src && dst && H > 0 && H <= 65535 && d > 0 && (!gate || ldg >= H));
    const dim3 grid(n, H);
#define GO(S, D) head_transpose_kernel<S, D><<<grid, 64, 0, st>>>(src, s_si, s_sh, dst, d_si, d_sh, d, scale, gate, ldg)
    if (s16 && d16) GO(true, true);
    else if (s16) GO(true, false);
    else if (d16) GO(false, true);
    else GO(false, false);
#undef GO
    return (int)hipGetLastError();
}

extern "C" int mxh_masked_softmax(const float* sc, void* pw, int p16, long rows, int n, int nk, int p0, int key0,
                                  float scale, int chunk, int window, int sink, const float* sink_v,
                                  const float* bias, int nb, int H, int two, hipStream_t st) {
    if (rows <= 0) return 0;
    MXH_CHECK(!two || p16);
    MXH_CHECK(sc && pw && n > 0 && nk > 0 && rows % n == 0 && rows < (1L << 31) && key0 >= 0 && p0 >= key0);
    MXH_CHECK((!bias || nb > 0) && (!(bias || sink_v) || rows == (long)H * n));
    if (p16)
        masked_softmax_kernel<true><<<(unsigned)rows, 256, 0, st>>>(sc, pw, n, nk, p0, key0, scale, chunk, window, sink,
                                                                    sink_v, bias, nb, H, two);
    else
        masked_softmax_kernel<false><<<(unsigned)rows, 256, 0, st>>>(sc, pw, n, nk, p0, key0, scale, chunk, window, sink,
                                                                     sink_v, bias, nb, H, 0);
    return (int)hipGetLastError();
}

// A prompt chunk of n rows of one sequence (q and out point at its first row) at positions p0 .., bf16 pools.
// Returns hipErrorInvalidValue for head sizes without an instantiation: the caller asks mxh_attention_mfma_ok first.
extern "C" int mxh_attention_mfma_ok(int dk, int dv) { return (dk == 64 || dk == 128) && (dv == 64 || dv == 128); }

extern "C" int mxh_attention_mfma(const void* q, int ldq, const void* kc, const void* vc, int bs, const int* table,
                                  int p0, int n, void* out, int ldo, int o16, int H, int G, int dk, int dv,
                                  float scale, int chunk, int window, int sink, float out_scale, const float* sink_v,
                                  const float* bias, int nb, const float* gate, int ldg, int gv, int p2,
                                  hipStream_t st) {
    if (n <= 0) return 0;
    MXH_CHECK((!bias || nb > 0) && (!gate || ldg >= H) && (!sink_v || sink) && gv > 0 && G % gv == 0);
    const AttnExtra ex = {sink_v, bias, nb, gate, ldg, gv};
    MXH_CHECK(q && kc && vc && table && out && bs > 0 && p0 >= 0 && H > 0 && G > 0 && H % G == 0);
    MXH_CHECK(mxh_attention_mfma_ok(dk, dv) && ldq >= H * dk && ldq % 8 == 0 && ldo >= H * dv && chunk >= 0 && window >= 0);
    const int rep = H / G;
    const int GW = rep % 4 == 0 ? 4 : rep % 2 == 0 ? 2 : 1;
    const int RT = 4 / GW;
    MXH_CHECK(H / GW <= 65535);
    const dim3 grid((n + RT * 16 - 1) / (RT * 16), H / GW);
#define GO3(K_, V_, O_, P_)                                                                                       \
    attn_chunk_mfma_kernel<K_, V_, O_, P_><<<grid, 256, 0, st>>>((const bf16_t*)q, ldq, (const bf16_t*)kc,             \
                                                                 (const bf16_t*)vc, bs, table, p0, n, out, ldo, H, G, \
                                                                 GW, scale, chunk, window, sink, out_scale, ex)
#define GO(K_, V_)                                 \
    do {                                           \
        if (o16 && p2) GO3(K_, V_, true, true);    \
        else if (o16) GO3(K_, V_, true, false);    \
        else if (p2) GO3(K_, V_, false, true);     \
        else GO3(K_, V_, false, false);            \
    } while (0)
    if (dk == 64 && dv == 64) GO(64, 64);
    else if (dk == 64 && dv == 128) GO(64, 128);
    else if (dk == 128 && dv == 64) GO(128, 64);
    else GO(128, 128);
#undef GO
#undef GO3
    return (int)hipGetLastError();
}

// Decode rows (row r = sequence r's new token) on the matrix cores; same conditions as mxh_attention_mfma plus at most
// 16 query heads per key / value head. Partitions as in mxh_attention.
extern "C" int mxh_attention_decode_mfma(const void* q, int ldq, const void* kc, const void* vc, int bs, const int* bt,
                                         int bt_stride, const int* ctx, int n_seqs, void* out, int ldo, int o16, int H,
                                         int G, int dk, int dv, float scale, int chunk, int window, int sink,
                                         float out_scale, int parts, int part_len, float* part_ml, float* part_o,
                                         const float* sink_v, const float* bias, int nb, const float* gate, int ldg,
                                         int gv, int p2, hipStream_t st) {
    if (n_seqs <= 0) return 0;
    MXH_CHECK((!bias || nb > 0) && (!gate || ldg >= H) && (!sink_v || sink) && gv > 0 && G % gv == 0);
    const AttnExtra ex = {sink_v, bias, nb, gate, ldg, gv};
    MXH_CHECK(q && kc && vc && bt && ctx && out && bs > 0 && bt_stride > 0 && H > 0 && G > 0 && H % G == 0);
    MXH_CHECK(H / G <= 16 && G <= 65535 && mxh_attention_mfma_ok(dk, dv) && ldq >= H * dk && ldq % 8 == 0 && ldo >= H * dv);
    MXH_CHECK(parts >= 1 && parts <= 64 && (parts == 1 || (part_len > 0 && part_ml && part_o)) && chunk >= 0 && window >= 0);
    const dim3 grid(n_seqs, G, parts);
#define GO3(K_, V_, O_, P_)                                                                                             \
    attn_decode_mfma_kernel<K_, V_, O_, P_><<<grid, 64, 0, st>>>(                                                           \
        (const bf16_t*)q, ldq, (const bf16_t*)kc, (const bf16_t*)vc, bs, bt, bt_stride, ctx, out, ldo, H, G, scale, chunk, \
        window, sink, out_scale, parts, part_len, part_ml, part_o, ex)
#define GO(K_, V_)                                 \
    do {                                           \
        if (o16 && p2) GO3(K_, V_, true, true);    \
        else if (o16) GO3(K_, V_, true, false);    \
        else if (p2) GO3(K_, V_, false, true);     \
        else GO3(K_, V_, false, false);            \
    } while (0)
    if (dk == 64 && dv == 64) GO(64, 64);
    else if (dk == 64 && dv == 128) GO(64, 128);
    else if (dk == 128 && dv == 64) GO(128, 64);
    else GO(128, 128);
#undef GO
#undef GO3
    if (parts > 1) {
        const dim3 g2(n_seqs, H);
        if (o16) attn_merge_kernel<true><<<g2, 64, 0, st>>>(part_ml, part_o, parts, H, dv, sink, out_scale, 0, out, ldo, ex);
        else attn_merge_kernel<false><<<g2, 64, 0, st>>>(part_ml, part_o, parts, H, dv, sink, out_scale, 0, out, ldo, ex);
    }
    return (int)hipGetLastError();
}
