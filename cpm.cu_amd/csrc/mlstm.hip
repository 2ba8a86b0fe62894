// The matrix-memory recurrence of the mLSTM kind, per head with key size d and value size dv:
//
//   a_t = cap tanh((i_t + bi) / cap)                     log input gate
//   b_t = logsigmoid(cap tanh((f_t + bf) / cap))         log forget gate
//   m_t = max(b_t + m_(t-1), a_t)                        running maximum, 0 before the first token
//   S_t = exp(b_t + m_(t-1) - m_t) S_(t-1) + exp(a_t - m_t) k_t v_t^T          S: [d, dv], zero at the start
//   n_t = exp(b_t + m_(t-1) - m_t) n_(t-1) + exp(a_t - m_t) k_t
//   y_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
//
// q, k, v and the raw gates i, f are columns of one projection (q is multiplied by `q_scale` as it is read);
// gates, decays, the state and the output are float.  S, n and m live per cache slot and are carried from step to
// step, so a step of any number of tokens continues where the last one ended.
#include "common.h"

#define ML_PB 32        // value columns a workgroup
#define ML_L 8          // lanes a column: key index c = l + 8 i

__device__ inline float log_sigmoid_f(float v) { return fminf(v, 0.f) - log1pf(expf(-fabsf(v))); }

// grid (sequences, heads, ceil(dv / 32)), 256 threads.  proj: [n, ld]; q at column q_off + h * d, k at k_off + h * d,
// v at v_off + h * dv, raw gates at i_off + h and f_off + h.  S: [slots][heads][dv][d], nst: [slots][heads][d],
// mst: [slots][heads]; y: float [n, heads * dv].
template <int NR, int ML_TT, typename T>   // ML_TT: tokens a tile in LDS
__global__ __launch_bounds__(256) void mlstm_scan_kernel(const T* __restrict__ proj, long ld, long q_off, long k_off,
                                                         long v_off, long i_off, long f_off,
                                                         const float* __restrict__ i_bias,
                                                         const float* __restrict__ f_bias, float cap, float q_scale,
                                                         float* __restrict__ S_state, float* __restrict__ n_state,
                                                         float* __restrict__ m_state, float* __restrict__ y,
                                                         const int* __restrict__ cu_q, const int* __restrict__ seq_slot,
                                                         int heads, int d, int dv, int write_state) {
    constexpr int NS = NR * ML_L;                   // key features, padded
    constexpr int QK = ML_TT * NS / 256;            // q (and k) values a thread brings a tile
    constexpr int XV = ML_TT * ML_PB / 256;         // v values a thread brings a tile
    __shared__ float qs[ML_TT][NS];
    __shared__ float ks[ML_TT][NS];
    __shared__ float vs[ML_TT][ML_PB];
    __shared__ float as_[ML_TT], bs_[ML_TT];
    const int b = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * ML_PB;
    const int start = cu_q[b], q = cu_q[b + 1] - start;
    const int slot = seq_slot[b];
    const int pl = threadIdx.x / ML_L, l = threadIdx.x % ML_L;
    const int p = p0 + pl;
    const bool p_ok = p < dv;
    float S[NR], nv[NR];
    float* sp = S_state + (((long)slot * heads + h) * dv + (p_ok ? p : 0)) * d;
    float* np = n_state + ((long)slot * heads + h) * d;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const int c = l + ML_L * i;
        S[i] = (p_ok && c < d) ? sp[c] : 0.f;
        nv[i] = c < d ? np[c] : 0.f;
    }
    float m = m_state[(long)slot * heads + h];
    const float bi = i_bias[h], bf = f_bias[h], inv_cap = 1.0f / cap;
    float rq[QK], rk[QK], rx[XV], ri = 0.f, rf = 0.f;
    auto fetch = [&](int t0) {
        const int tn = min(ML_TT, q - t0);
#pragma unroll
        for (int e2 = 0; e2 < QK; ++e2) {
            const int e = threadIdx.x + e2 * 256;
            const int tt = e / NS, c = e % NS;
            const bool ok = tt < tn && c < d;
            const T* row = proj + (long)(start + t0 + min(tt, tn - 1)) * ld + (long)h * d + min(c, d - 1);
            rq[e2] = ok ? to_f32(row[q_off]) * q_scale : 0.f;
            rk[e2] = ok ? to_f32(row[k_off]) : 0.f;
        }
#pragma unroll
        for (int e2 = 0; e2 < XV; ++e2) {
            const int e = threadIdx.x + e2 * 256;
            const int tt = e / ML_PB, pp = e % ML_PB;
            rx[e2] = (tt < tn && p0 + pp < dv) ? to_f32(proj[(long)(start + t0 + tt) * ld + v_off + (long)h * dv + p0 + pp]) : 0.f;
        }
        if ((int)threadIdx.x < tn) {
            const T* row = proj + (long)(start + t0 + threadIdx.x) * ld + h;
            ri = to_f32(row[i_off]);
            rf = to_f32(row[f_off]);
        }
    };
    fetch(0);
    for (int t0 = 0; t0 < q; t0 += ML_TT) {
        const int tn = min(ML_TT, q - t0);
        __syncthreads();
#pragma unroll
        for (int e2 = 0; e2 < QK; ++e2) {
            const int e = threadIdx.x + e2 * 256;
            qs[e / NS][e % NS] = rq[e2];
            ks[e / NS][e % NS] = rk[e2];
        }
#pragma unroll
        for (int e2 = 0; e2 < XV; ++e2) {
            const int e = threadIdx.x + e2 * 256;
            vs[e / ML_PB][e % ML_PB] = rx[e2];
        }
        if ((int)threadIdx.x < tn) {
            as_[threadIdx.x] = cap * tanhf((ri + bi) * inv_cap);
            bs_[threadIdx.x] = log_sigmoid_f(cap * tanhf((rf + bf) * inv_cap));
        }
        __syncthreads();
        if (t0 + ML_TT < q) fetch(t0 + ML_TT);
        for (int tt = 0; tt < tn; ++tt) {
            const float a = as_[tt], bb = bs_[tt];
            const float m_new = fmaxf(bb + m, a);
            const float keep = expf(bb + m - m_new), take = expf(a - m_new);
            m = m_new;
            const float tv = take * vs[tt][pl];
            float num = 0.f, dot = 0.f;
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const int c = l + ML_L * i;
                const float kk = ks[tt][c], qq = qs[tt][c];
                S[i] = keep * S[i] + tv * kk;
                nv[i] = keep * nv[i] + take * kk;
                num += S[i] * qq;
                dot += nv[i] * qq;
            }
            // the column's 8 lanes are neighbours: sums inside the vector unit
            num += CPMCU_DPP(num, 0xB1);
            num += CPMCU_DPP(num, 0x4E);
            num += CPMCU_DPP(num, 0x141);
            dot += CPMCU_DPP(dot, 0xB1);
            dot += CPMCU_DPP(dot, 0x4E);
            dot += CPMCU_DPP(dot, 0x141);
            if (l == 0 && p_ok) {
                const float den = fmaxf(fabsf(dot), expf(-m)) + 1e-6f;
                y[(long)(start + t0 + tt) * heads * dv + (long)h * dv + p] = num / den;
            }
        }
    }
    if (write_state) {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int c = l + ML_L * i;
            if (p_ok && c < d) sp[c] = S[i];
            // every workgroup of a head walks the same n and m; the first one writes them
            if (blockIdx.z == 0 && pl == 0 && c < d) np[c] = nv[i];
        }
        if (blockIdx.z == 0 && threadIdx.x == 0) m_state[(long)slot * heads + h] = m;
    }
}

extern "C" const char* cpmcu_mlstm_scan(const void* proj, long ld, int dtype, long q_off, long k_off, long v_off,
                                        long i_off, long f_off, const float* i_bias, const float* f_bias, float cap,
                                        float q_scale, float* S_state, float* n_state, float* m_state, float* y,
                                        const int* cu_q, const int* seq_slot, int n_seqs, int heads, int d, int dv,
                                        int write_state, hipStream_t stream) {
    CPMCU_REQUIRE(n_seqs > 0 && heads > 0 && d > 0 && dv > 0, "mlstm_scan: empty shape");
    CPMCU_REQUIRE(d <= 256, "mlstm_scan: a key size of %d is not supported (at most 256)", d);
    CPMCU_REQUIRE(cap > 0.f, "mlstm_scan: gate cap %g", cap);
    CPMCU_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && i_off >= 0 && f_off >= 0 && q_off + (long)heads * d <= ld &&
                  k_off + (long)heads * d <= ld && v_off + (long)heads * dv <= ld && i_off + heads <= ld && f_off + heads <= ld,
                  "mlstm_scan: columns beyond rows of %ld", ld);
    const int pb = (dv + ML_PB - 1) / ML_PB;
    CPMCU_REQUIRE(heads <= 65535 && pb <= 65535, "mlstm_scan: shape exceeds the launch grid");
    dim3 grid(n_seqs, heads, pb);
    const int need = (d + ML_L - 1) / ML_L;
#define LAUNCH(NRv, TTv, Tv)                                                                                             \
    mlstm_scan_kernel<NRv, TTv, Tv><<<grid, 256, 0, stream>>>((const Tv*)proj, ld, q_off, k_off, v_off, i_off, f_off, i_bias, \
                                                         f_bias, cap, q_scale, S_state, n_state, m_state, y, cu_q,  \
                                                         seq_slot, heads, d, dv, write_state)
#define BY_NR(Tv)                            \
    do {                                     \
        if (need <= 2) LAUNCH(2, 32, Tv);        \
        else if (need <= 4) LAUNCH(4, 32, Tv);   \
        else if (need <= 8) LAUNCH(8, 32, Tv);   \
        else if (need <= 16) LAUNCH(16, 32, Tv); \
        else LAUNCH(32, 16, Tv);                 \
    } while (0)
    if (dtype == CPMCU_F32) BY_NR(float);
    else if (dtype == CPMCU_BF16) BY_NR(bf16_t);
    else CPMCU_FAIL("mlstm_scan: unknown dtype %d", dtype);
#undef BY_NR
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("mlstm_scan");
    return nullptr;
}
