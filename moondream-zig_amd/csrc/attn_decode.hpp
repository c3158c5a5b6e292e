// Device-side building blocks of single-token attention, shared by the stand-alone decode-attention kernels
// and the persistent decode kernel.  Written for 256-thread workgroups (4 wavefronts).
#pragma once
#include "epilogue.hpp"

constexpr int DEC_SPLITS = 8;
constexpr int DEC_MAX_KEYS = (2048 + DEC_SPLITS - 2) / (DEC_SPLITS - 1); // per split at the reference's kv limit (attention.zig:252)

// The key range [j0, j1) of split `split`.  Plain mode: the kv_len keys of the cache in DEC_SPLITS even parts.  Fused mode
// (the new token's k and v come from the qkv vector): the pos_real cached keys in DEC_SPLITS - 1 even parts, and the new
// token's own key alone in the last split.  The cached keys need nothing of the new token but q, so only that last split
// has to wait for its k and v, and it has next to nothing to do once they are there.
__device__ __forceinline__ void decode_attn_range(int pos_real, bool fused, int split, int &j0, int &j1) {
    if (!fused) {
        const int kv_len = pos_real + 1, per = (kv_len + DEC_SPLITS - 1) / DEC_SPLITS;
        j0 = split * per;
        j1 = min(kv_len, j0 + per);
    } else if (split == DEC_SPLITS - 1) {
        j0 = pos_real;
        j1 = pos_real + 1;
    } else {
        const int per = (pos_real + DEC_SPLITS - 2) / (DEC_SPLITS - 1);
        j0 = split * per;
        j1 = min(pos_real, j0 + per);
    }
}
constexpr int DEC_PREFETCH = 4;                 // keys per lane group whose K and V rows are loaded up front (the default of the PF parameters below)

// Merge the DEC_SPLITS partials of one head in a fixed order; returns output element d of that head.
template <int D, bool COH = false>
__device__ __forceinline__ half_t decode_attn_merge(const float *__restrict__ p /* partials of this head */, int d) {
    // everything is requested before anything is used: one round trip (device-coherent loads are issued where the source
    // has them, so loads that followed the maximum would be a second one)
    float ms_[DEC_SPLITS], ls_[DEC_SPLITS], os_[DEC_SPLITS];
#pragma unroll
    for (int s = 0; s < DEC_SPLITS; s++) {
        ms_[s] = ld_f<COH>(p + s * (D + 2) + D);
        ls_[s] = ld_f<COH>(p + s * (D + 2) + D + 1);
        os_[s] = ld_f<COH>(p + s * (D + 2) + d);
    }
    float m = -INFINITY;
#pragma unroll
    for (int s = 0; s < DEC_SPLITS; s++) m = fmaxf(m, ms_[s]);
    float l = 0.0f, o = 0.0f;
#pragma unroll
    for (int s = 0; s < DEC_SPLITS; s++) {
        const float ms = ms_[s];
        const float w = (ms == -INFINITY) ? 0.0f : __expf(ms - m);
        l = fmaf(ls_[s], w, l);
        o = fmaf(os_[s], w, o);
    }
    return (half_t)f32_round(o * (1.0f / l)); // attention.zig:612-615 multiplies by the reciprocal of the sum
}

// K and V rows of the first PF keys of every lane group of a (head, split) task (32 keys of the split per step: 8 lane groups in
// each of 4 wavefronts).  They depend only on the position, not on the new token, so a caller may request them long before it
// runs the task.  Keys past 32 * PF of a split are loaded inside the task, one dependent round trip per 32: a caller that
// knows the position picks PF to cover the split (results do not depend on PF).
template <int PF = DEC_PREFETCH>
struct DecodeAttnPrefetch {
    uint4 k[PF], v[PF];
};
template <int D, int PF = DEC_PREFETCH>
__device__ __forceinline__ void decode_attn_prefetch(DecodeAttnPrefetch<PF> &pf, const half_t *__restrict__ ck, const half_t *__restrict__ cv,
                                                     int max_seq, int pos_real, bool fused, int h, int split) {
    const int pos = fused ? pos_real : -1;
    int j0, j1;
    decode_attn_range(pos_real, fused, split, j0, j1);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 3, e = lane & 7;
    const half_t *kbase = ck + size_t(h) * max_seq * D;
    const half_t *vbase = cv + size_t(h) * max_seq * D;
    const int jfirst = j0 + wave * 8 + g;
#pragma unroll
    for (int i = 0; i < PF; i++) {
        const int j = jfirst + 32 * i;
        pf.k[i] = make_uint4(0, 0, 0, 0);
        pf.v[i] = make_uint4(0, 0, 0, 0);
        if (j < j1 && j != pos) {
            pf.k[i] = *reinterpret_cast<const uint4 *>(kbase + size_t(j) * D + 8 * e);
            pf.v[i] = *reinterpret_cast<const uint4 *>(vbase + size_t(j) * D + 8 * e);
        }
    }
}

// One (head, split) task: un-normalised partial (o[D], m, l) of softmax(q.K^T/sqrt(D)).V over the split's keys.
// FUSED: q | k | v of the new token come from qkv[3*H*D], are rotated here (rope.zig:223-224), and the split that
//        owns position pos appends k', v to the cache (text_model.zig:483-491).
// !FUSED: qkv is an already rotated q[H,D] and all pos+1 keys are in ck/cv (head stride max_seq*D).
// COH: (persistent kernel) qkv reads, the cache append and the partial stores use device-coherent accesses, and
//      the task that completes a head last (head_count[h] reaches count_target) merges the head's partials into
//      (the stand-alone path merges in a second kernel instead)
//      merged_out[h*D ..] and then counts the head in at done_count.
// pf holds the rows requested by decode_attn_prefetch for the same (h, split, pos).  Workgroup synchronisation is LDS-only.
// Every thread of the workgroup must call it.
template <int D, bool FUSED, bool COH = false, int PF = DEC_PREFETCH>
__device__ __forceinline__ void decode_attn_task(const half_t *__restrict__ qkv, half_t *__restrict__ ck,
                                                 half_t *__restrict__ cv, const float *__restrict__ table,
                                                 float *__restrict__ partial, int H, int rot_dim, int max_seq, int pos_real,
                                                 int h, int split, const DecodeAttnPrefetch<PF> &pf, uint32_t *head_count = nullptr,
                                                 uint32_t count_target = 0, half_t *merged_out = nullptr, uint32_t *done_count = nullptr,
                                                 int done_copies = 1, int done_stride = 0, int head_stride = 1) {
    static_assert(D == 64, "one 16-byte granule per lane, 8 lanes per key");
    __shared__ float sq[D];
    __shared__ __attribute__((aligned(16))) half_t sk_new[D];
    __shared__ __attribute__((aligned(16))) half_t sv_new[D];
    __shared__ float sscore[DEC_MAX_KEYS];
    __shared__ float sred[4][D];
    __shared__ float sstat[8];
    __shared__ int s_last;

    const int pos = FUSED ? pos_real : -1; // in plain mode no key is special
    int j0, j1;
    decode_attn_range(pos_real, FUSED, split, j0, j1);
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int hd = H * D, half = rot_dim >> 1;
    const int g = lane >> 3, e = lane & 7; // key within a group of 8, granule within the key
    const half_t *kbase = ck + size_t(h) * max_seq * D;
    const half_t *vbase = cv + size_t(h) * max_seq * D;
    const int jfirst = j0 + wave * 8 + g; // this lane group's keys: jfirst, jfirst + 32, ...

    lds_barrier(); // the shared arrays may still be in use by a previous task of this workgroup
    if (!FUSED) {
        if (t < D) sq[t] = (float)ld_h<COH>(qkv + h * D + t);
    } else if (t < D) {
#pragma clang fp contract(off)
        // q stays f16-rounded like the reference's qr tensor; multiplies and adds are separate as in rope.zig
        const int d = t;
        const half_t *q = qkv + h * D, *k = qkv + hd + h * D, *v = qkv + 2 * hd + h * D;
        // k and v of the new token are read by the split that holds its key alone (a caller may run the other splits
        // before those rows exist)
        const bool own = split == DEC_SPLITS - 1;
        sv_new[d] = own ? ld_h<COH>(v + d) : (half_t)0.0f;
        if (d >= rot_dim) {
            sq[d] = (float)ld_h<COH>(q + d);
            sk_new[d] = own ? ld_h<COH>(k + d) : (half_t)0.0f;
        } else {
            const int f = d < half ? d : d - half;
            const float c = table[(size_t(pos) * half + f) * 2], sn = table[(size_t(pos) * half + f) * 2 + 1];
            const float qr = (float)ld_h<COH>(q + f), qi = (float)ld_h<COH>(q + f + half);
            const float kr = own ? (float)ld_h<COH>(k + f) : 0.0f, ki = own ? (float)ld_h<COH>(k + f + half) : 0.0f;
            if (d < half) {
                sq[d] = (float)(half_t)(qr * c - qi * sn);
                sk_new[d] = (half_t)(kr * c - ki * sn);
            } else {
                sq[d] = (float)(half_t)(qr * sn + qi * c);
                sk_new[d] = (half_t)(kr * sn + ki * c);
            }
        }
    }
    lds_barrier();
    if (FUSED && pos >= j0 && pos < j1 && t < D) {
        st_h<COH>(ck + (size_t(h) * max_seq + pos) * D + t, sk_new[t]);
        st_h<COH>(cv + (size_t(h) * max_seq + pos) * D + t, sv_new[t]);
    }

    float qf[8];
#pragma unroll
    for (int i = 0; i < 8; i++) qf[i] = sq[8 * e + i];
    const float scale = 0.125f; // 1/sqrt(64), attention.zig:569

    // scores; the 8 lanes of a key group share j, so they stay converged through the shuffles
    auto score = [&](int j, const uint4 &kv) {
        const half_t *kh = reinterpret_cast<const half_t *>(&kv);
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) s = fmaf(qf[i], (float)kh[i], s);
        // the 8 lanes' sum on the DPP path (swap within pairs, swap pairs, mirror the 8): the same additions as an xor butterfly
        // over 1, 2, 4 (each level adds the same two values, in either order), without three trips through the LDS crossbar
        s += dpp_move<DPP_QUAD_XOR1>(s);
        s += dpp_move<DPP_QUAD_XOR2>(s);
        s += dpp_move<DPP_ROW_HALF_MIRROR>(s);
        if (e == 0) sscore[j - j0] = s * scale;
    };
#pragma unroll
    for (int i = 0; i < PF; i++) {
        const int j = jfirst + 32 * i;
        if (j < j1) score(j, j == pos ? *reinterpret_cast<const uint4 *>(&sk_new[8 * e]) : pf.k[i]);
    }
    for (int j = jfirst + 32 * PF; j < j1; j += 32)
        score(j, j == pos ? *reinterpret_cast<const uint4 *>(&sk_new[8 * e]) : *reinterpret_cast<const uint4 *>(kbase + size_t(j) * D + 8 * e));
    lds_barrier();

    // softmax statistics of this split
    const int nkeys = max(j1 - j0, 0);
    float m = -INFINITY;
    for (int i = t; i < nkeys; i += 256) m = fmaxf(m, sscore[i]);
    m = wave_max(m);
    if (lane == 0) sstat[wave] = m;
    lds_barrier();
    m = fmaxf(fmaxf(sstat[0], sstat[1]), fmaxf(sstat[2], sstat[3]));
    float l = 0.0f;
    for (int i = t; i < nkeys; i += 256) {
        const float p = __expf(sscore[i] - m);
        sscore[i] = p;
        l += p;
    }
    l = wave_sum(l);
    if (lane == 0) sstat[4 + wave] = l;
    lds_barrier();
    l = (sstat[4] + sstat[5]) + (sstat[6] + sstat[7]);

    // o = sum_j p_j v_j
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.0f;
    auto accumulate = [&](int j, const uint4 &vv) {
        const half_t *vh = reinterpret_cast<const half_t *>(&vv);
        const float p = sscore[j - j0];
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = fmaf(p, (float)vh[i], acc[i]);
    };
#pragma unroll
    for (int i = 0; i < PF; i++) {
        const int j = jfirst + 32 * i;
        if (j < j1) accumulate(j, j == pos ? *reinterpret_cast<const uint4 *>(&sv_new[8 * e]) : pf.v[i]);
    }
    for (int j = jfirst + 32 * PF; j < j1; j += 32)
        accumulate(j, j == pos ? *reinterpret_cast<const uint4 *>(&sv_new[8 * e]) : *reinterpret_cast<const uint4 *>(vbase + size_t(j) * D + 8 * e));
#pragma unroll
    for (int i = 0; i < 8; i++) {
        acc[i] += __shfl_xor(acc[i], 8, 64);
        acc[i] += __shfl_xor(acc[i], 16, 64);
        acc[i] += __shfl_xor(acc[i], 32, 64);
    }
    if (g == 0) {
#pragma unroll
        for (int i = 0; i < 8; i++) sred[wave][8 * e + i] = acc[i];
    }
    lds_barrier();
    float *dst = partial + (size_t(h) * DEC_SPLITS + split) * (D + 2);
    if (t < D) st_f<COH>(dst + t, (sred[0][t] + sred[1][t]) + (sred[2][t] + sred[3][t]));
    if (t == 0) {
        st_f<COH>(dst + D, m);
        st_f<COH>(dst + D + 1, l);
    }
    if (COH && head_count) {
        // the partial is stored by wavefront 0 only (t < 64): once its stores are acknowledged, thread 0 counts this
        // task in; whoever brings the head's count to the target sees all DEC_SPLITS partials and merges them
        if (wave == 0) {
            __builtin_amdgcn_s_waitcnt(0); // vmcnt(0): the partial has reached memory
            if (t == 0) {
                const uint32_t old = __hip_atomic_fetch_add(head_count + size_t(h) * head_stride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                s_last = (old + 1 == count_target) ? 1 : 0;
            }
        }
        lds_barrier();
        if (s_last && wave == 0) { // t < D: the merged head, then (once acknowledged) the head is counted as done
            st_h<true>(merged_out + h * D + t, decode_attn_merge<D, true>(partial + size_t(h) * DEC_SPLITS * (D + 2), t));
            __builtin_amdgcn_s_waitcnt(0);
            // (done_copies copies of the counter, done_stride words apart: a lane each)
            if (t < done_copies && done_count) __hip_atomic_fetch_add(done_count + t * done_stride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}
