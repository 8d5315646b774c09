// Decode-step buffer pass + log-sum-exp merge + in-place cache append (gfx950).
//
// One wavefront per (trajectory, head).  The buffer K/V rows of that pair are
// streamed once with 16-byte loads (HBM-bound: 2 flop per byte), each group of
// DH/8 lanes owning one key row at a time and keeping a private online-softmax
// state per query.  The partial results of the split context pass enter the same
// states as extra "keys" whose weight is their log-sum-exp, and one butterfly
// reduction across the lane groups (a wavefront-wide log-sum-exp merge in
// float32) produces the final output.  The new buffer row is read from the
// projection and written to its cache slot by the same wavefront: no torch.cat,
// no second pass.
#pragma once

#include "common.h"

namespace artab {

struct DecodeParams {
    View q, kb, vb, knew, vnew, out;
    const float *part_o;    // [n_split][B*H*Lq][DH] normalised context partials
    const float *part_lse;  // [n_split][B*H*Lq] natural-log LSE of each partial
    float *lse;             // optional final LSE [B,H,Lq]
    int B, H;
    int n_split;
    int n_buf;    // committed buffer rows
    const int *n_buf_dev;  // when set, the committed length is read from here at run time
    int has_new;  // 1: row n_buf comes from knew/vnew, is attended and appended
    float qscale; // scale * log2(e)
};

constexpr int kDecodeWaves = 4;
constexpr int kDecodeUnroll = 4;

template <typename T>
__device__ __forceinline__ void unpack8(const u32x4 &raw, float (&f)[8]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        f[2 * e] = unpack_lo<T>(raw[e]);
        f[2 * e + 1] = unpack_hi<T>(raw[e]);
    }
}

template <typename T, int DH, int LQ>
__global__ __launch_bounds__(kDecodeWaves * 64) void decode_buffer_kernel(DecodeParams P) {
    constexpr int LPR = DH / 8;    // lanes per key row
    constexpr int RPW = 64 / LPR;  // key rows per wavefront load
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const long pair = static_cast<long>(blockIdx.x) * kDecodeWaves + wave;  // b*H + h
    if (pair >= static_cast<long>(P.B) * P.H) return;
    const long b = pair / P.H;
    const int h = static_cast<int>(pair % P.H);
    const int grp = lane / LPR;  // which row of a load this lane works on
    const int sub = lane % LPR;  // which 8-element slice of the head dimension
    const long total_rows = static_cast<long>(P.B) * P.H * LQ;

    float qf[LQ][8];
#pragma unroll
    for (int i = 0; i < LQ; ++i) {
        u32x4 raw = *reinterpret_cast<const u32x4 *>(view_row<T>(P.q, b, h, i) + 8 * sub);
        unpack8<T>(raw, qf[i]);
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[i][e] *= P.qscale;
    }

    float m[LQ], l[LQ], acc[LQ][8];
#pragma unroll
    for (int i = 0; i < LQ; ++i) {
        m[i] = -INFINITY;
        l[i] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[i][e] = 0.f;
    }

    const int n_buf = P.n_buf_dev ? *P.n_buf_dev : P.n_buf;
    const int n_total = n_buf + (P.has_new ? 1 : 0);
    const T *knew_row = P.has_new ? view_row<T>(P.knew, b, h, 0) : nullptr;
    const T *vnew_row = P.has_new ? view_row<T>(P.vnew, b, h, 0) : nullptr;

    for (int kv0 = 0; kv0 < n_total; kv0 += RPW * kDecodeUnroll) {
        u32x4 kraw[kDecodeUnroll], vraw[kDecodeUnroll];
        bool ok[kDecodeUnroll];
#pragma unroll
        for (int u = 0; u < kDecodeUnroll; ++u) {
            int kv = kv0 + u * RPW + grp;
            ok[u] = kv < n_total;
            kraw[u] = u32x4{0u, 0u, 0u, 0u};
            vraw[u] = u32x4{0u, 0u, 0u, 0u};
            if (ok[u]) {
                const bool is_new = P.has_new && kv == n_buf;
                const T *kr = is_new ? knew_row : view_row<T>(P.kb, b, h, kv);
                const T *vr = is_new ? vnew_row : view_row<T>(P.vb, b, h, kv);
                kraw[u] = *reinterpret_cast<const u32x4 *>(kr + 8 * sub);
                vraw[u] = *reinterpret_cast<const u32x4 *>(vr + 8 * sub);
            }
        }
        float s[LQ][kDecodeUnroll];
#pragma unroll
        for (int u = 0; u < kDecodeUnroll; ++u) {
            float kf[8];
            unpack8<T>(kraw[u], kf);
#pragma unroll
            for (int i = 0; i < LQ; ++i) {
                float d = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) d = fmaf(qf[i][e], kf[e], d);
#pragma unroll
                for (int o = 1; o < LPR; o <<= 1) d += __shfl_xor(d, o, 64);
                s[i][u] = ok[u] ? d : -INFINITY;
            }
        }
#pragma unroll
        for (int i = 0; i < LQ; ++i) {
            float cm = s[i][0];
#pragma unroll
            for (int u = 1; u < kDecodeUnroll; ++u) cm = fmaxf(cm, s[i][u]);
            const float m_new = fmaxf(m[i], cm);
            if (m_new == -INFINITY) continue;  // this lane group had no row in the chunk yet
            const float alpha = fast_exp2(m[i] - m_new);
            m[i] = m_new;
            l[i] *= alpha;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[i][e] *= alpha;
        }
#pragma unroll
        for (int u = 0; u < kDecodeUnroll; ++u) {
            float vf[8];
            unpack8<T>(vraw[u], vf);
#pragma unroll
            for (int i = 0; i < LQ; ++i) {
                const float p = ok[u] ? fast_exp2(s[i][u] - m[i]) : 0.f;
                l[i] += p;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[i][e] = fmaf(p, vf[e], acc[i][e]);
            }
        }
    }

    // Context partials: split s is folded in by lane group s mod RPW.  A partial
    // (o, lse) is a key with score lse (log2 domain) and value o.
    for (int sp = grp; sp < P.n_split; sp += RPW) {
#pragma unroll
        for (int i = 0; i < LQ; ++i) {
            const long row = pair * LQ + i;
            const float sc = P.part_lse[static_cast<long>(sp) * total_rows + row] * kLog2e;
            const float *po = P.part_o + (static_cast<long>(sp) * total_rows + row) * DH + 8 * sub;
            f32x4 o0 = *reinterpret_cast<const f32x4 *>(po);
            f32x4 o1 = *reinterpret_cast<const f32x4 *>(po + 4);
            const float m_new = fmaxf(m[i], sc);
            if (m_new == -INFINITY) continue;
            const float alpha = fast_exp2(m[i] - m_new);
            const float p = fast_exp2(sc - m_new);
            m[i] = m_new;
            l[i] = l[i] * alpha + p;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc[i][e] = fmaf(p, o0[e], acc[i][e] * alpha);
                acc[i][4 + e] = fmaf(p, o1[e], acc[i][4 + e] * alpha);
            }
        }
    }

    // Butterfly merge of the RPW lane-group states (same slice `sub` across groups).
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) {
#pragma unroll
        for (int i = 0; i < LQ; ++i) {
            const float m_o = __shfl_xor(m[i], off, 64);
            const float l_o = __shfl_xor(l[i], off, 64);
            const float m_new = fmaxf(m[i], m_o);
            const float a_s = m[i] == -INFINITY ? 0.f : fast_exp2(m[i] - m_new);
            const float a_o = m_o == -INFINITY ? 0.f : fast_exp2(m_o - m_new);
            l[i] = l[i] * a_s + l_o * a_o;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float acc_o = __shfl_xor(acc[i][e], off, 64);
                acc[i][e] = acc[i][e] * a_s + acc_o * a_o;
            }
            m[i] = m_new;
        }
    }

    if (grp == 0) {
#pragma unroll
        for (int i = 0; i < LQ; ++i) {
            const float inv = l[i] > 0.f ? 1.f / l[i] : 0.f;
            u32x4 val;
#pragma unroll
            for (int e = 0; e < 4; ++e) val[e] = pack2<T>(acc[i][2 * e] * inv, acc[i][2 * e + 1] * inv);
            *reinterpret_cast<u32x4 *>(view_row<T>(P.out, b, h, i) + 8 * sub) = val;
            if (P.lse && sub == 0)
                P.lse[pair * LQ + i] = l[i] > 0.f ? (m[i] + fast_log2(l[i])) * kLn2 : -INFINITY;
        }
    } else if (grp == 1 && P.has_new) {
        // In-place append: slot n_buf of the cache receives the new row.
        *reinterpret_cast<u32x4 *>(view_row<T>(P.kb, b, h, n_buf) + 8 * sub) =
            *reinterpret_cast<const u32x4 *>(knew_row + 8 * sub);
        *reinterpret_cast<u32x4 *>(view_row<T>(P.vb, b, h, n_buf) + 8 * sub) =
            *reinterpret_cast<const u32x4 *>(vnew_row + 8 * sub);
    }
}

}  // namespace artab
