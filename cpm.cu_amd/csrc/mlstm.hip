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
// gates, decays, the state and the output are float.  The kernel leaves S_t^T q_t and the denominator side by side;
// the head norm that follows divides.  S, n and m live per cache slot and are carried from step to
// step, so a step of any number of tokens continues where the last one ended.
#include "common.h"

// A workgroup of 256 threads walks ML_PB = 256 / ML_L columns; a column's d state values lie over ML_L neighbouring
// lanes (8 or 32: key index c = l + ML_L i), which sum their shares inside the vector unit.  Keys beyond 128
// features take 32 lanes a column: four times the workgroups (several a CU, whose walks hide each other's waits)
// and a quarter of the chain of dependent steps a token.

__device__ inline float log_sigmoid_f(float v) { return fminf(v, 0.f) - log1pf(expf(-fabsf(v))); }

// grid (sequences, heads, ceil((dv + 1) / ML_PB)), 256 threads.  proj: [n, ld]; q at column q_off + h * d, k at
// k_off + h * d, v at v_off + h * dv, raw gates at i_off + h and f_off + h.  S: [slots][heads][dv][d],
// nst: [slots][heads][d], mst: [slots][heads].
//
// The normaliser n obeys the recurrence of a column of S whose value is always 1, so it is walked as column dv:
// columns 0 .. dv - 1 give the unnormalised y = S^T q (float [n, heads * dv]) and column dv gives n . q, from which
// den[t, h] = max(|n . q|, exp(-m)) + 1e-6 (float [n, heads]); whoever reads y divides by den (the head norm does).
// Tiles of ML_TT tokens pass through LDS; the running maximum of a tile is walked by one thread first (additions and
// maxima only), then the tile's exponentials are formed side by side, so the walk over the state itself holds
// nothing but multiply-adds.
template <int NR, int ML_L, int ML_TT, typename T>
__global__ __launch_bounds__(256) void mlstm_scan_kernel(const T* __restrict__ proj, long ld, long q_off, long k_off,
                                                         long v_off, long i_off, long f_off,
                                                         const float* __restrict__ i_bias,
                                                         const float* __restrict__ f_bias, float cap, float q_scale,
                                                         float* __restrict__ S_state, float* __restrict__ n_state,
                                                         float* __restrict__ m_state, float* __restrict__ y,
                                                         float* __restrict__ den, const int* __restrict__ cu_q,
                                                         const int* __restrict__ seq_slot, int heads, int d, int dv,
                                                         int write_state) {
    constexpr int ML_PB = 256 / ML_L;               // columns a workgroup
    constexpr int NS = NR * ML_L;                   // key features, padded
    constexpr int QK = ML_TT * NS / 256;            // q (and k) values a thread brings a tile
    constexpr int XV = (ML_TT * ML_PB + 255) / 256;   // v values a thread brings a tile
    __shared__ float qs[ML_TT][NS];
    __shared__ float ks[ML_TT][NS];
    __shared__ float vs[ML_TT][ML_PB];
    __shared__ float keep_s[ML_TT], take_s[ML_TT], em_s[ML_TT];
    __shared__ float m_carry;
    const int b = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * ML_PB;
    const int start = cu_q[b], q = cu_q[b + 1] - start;
    const int slot = seq_slot[b];
    const int pl = threadIdx.x / ML_L, l = threadIdx.x % ML_L;
    const int p = p0 + pl;
    const bool p_ok = p <= dv, is_n = p == dv;
    float S[NR];
    float* sp = is_n ? n_state + ((long)slot * heads + h) * d
                     : S_state + (((long)slot * heads + h) * dv + (p_ok ? p : 0)) * d;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const int c = l + ML_L * i;
        S[i] = (p_ok && c < d) ? sp[c] : 0.f;
    }
    if (threadIdx.x == 0) m_carry = m_state[(long)slot * heads + h];
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
            const int tt = e / ML_PB, pp = p0 + e % ML_PB;
            const long at = (long)(start + t0 + min(tt, tn - 1)) * ld + v_off + (long)h * dv + min(pp, dv - 1);
            const float v = to_f32(proj[at]);
            rx[e2] = tt < tn ? (pp < dv ? v : (pp == dv ? 1.0f : 0.f)) : 0.f;
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
            if (e < ML_TT * ML_PB) vs[e / ML_PB][e % ML_PB] = rx[e2];
        }
        if ((int)threadIdx.x < tn) {                 // log gates, parked where their exponentials will stand
            take_s[threadIdx.x] = cap * tanhf((ri + bi) * inv_cap);
            keep_s[threadIdx.x] = log_sigmoid_f(cap * tanhf((rf + bf) * inv_cap));
        }
        __syncthreads();
        if (threadIdx.x == 0) {                      // the running maximum through the tile, in registers
            float av[ML_TT], bv[ML_TT];
#pragma unroll
            for (int tt = 0; tt < ML_TT; ++tt) {
                av[tt] = take_s[tt];
                bv[tt] = keep_s[tt];
            }
            float m = m_carry;
#pragma unroll
            for (int tt = 0; tt < ML_TT; ++tt) {
                const float m_new = tt < tn ? fmaxf(bv[tt] + m, av[tt]) : m;
                bv[tt] = bv[tt] + m - m_new;
                av[tt] = av[tt] - m_new;
                m = m_new;
                keep_s[tt] = bv[tt];
                take_s[tt] = av[tt];
                em_s[tt] = -m_new;
            }
            m_carry = m;
        }
        __syncthreads();
        if ((int)threadIdx.x < tn) {
            keep_s[threadIdx.x] = expf(keep_s[threadIdx.x]);
            take_s[threadIdx.x] = expf(take_s[threadIdx.x]);
            em_s[threadIdx.x] = expf(em_s[threadIdx.x]);
        }
        __syncthreads();
        if (t0 + ML_TT < q) fetch(t0 + ML_TT);
        // a token's keys and queries are asked of LDS while the token before it is worked on
        float kc[NR], qc[NR], keep_c, tv_c, em_c;
        auto ask = [&](int tt, float* kk, float* qq, float& keep, float& tv, float& em) {
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                kk[i] = ks[tt][l + ML_L * i];
                qq[i] = qs[tt][l + ML_L * i];
            }
            keep = keep_s[tt];
            tv = take_s[tt] * vs[tt][pl];
            em = em_s[tt];
        };
        ask(0, kc, qc, keep_c, tv_c, em_c);
        float* yp = y + (long)(start + t0) * heads * dv + (long)h * dv + p;
        float* dp = den + (long)(start + t0) * heads + h;
#pragma unroll 2
        for (int tt = 0; tt < tn; ++tt) {
            float kn[NR], qn[NR], keep_n, tv_n, em_n;
            ask(min(tt + 1, tn - 1), kn, qn, keep_n, tv_n, em_n);
            float part[4] = {0.f, 0.f, 0.f, 0.f};       // four chains of additions side by side
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                S[i] = keep_c * S[i] + tv_c * kc[i];
                part[i & 3] += S[i] * qc[i];
            }
            float num = (part[0] + part[1]) + (part[2] + part[3]);
            // the column's lanes are neighbours: the sum inside the vector unit
            num += CPMCU_DPP(num, 0xB1);
            num += CPMCU_DPP(num, 0x4E);
            num += CPMCU_DPP(num, 0x141);
            if (ML_L >= 16) num += CPMCU_DPP(num, 0x140);
            if (ML_L == 32) {                            // the two rows of 16 lanes that share a column
                cpmcu_u32x2_t sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(num), __float_as_uint(num), false, false);
                num = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
            }
            if (l == 0 && p_ok) {
                if (is_n) *dp = fmaxf(fabsf(num), em_c) + 1e-6f;
                else *yp = num;
            }
            yp += (long)heads * dv;
            dp += heads;
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                kc[i] = kn[i];
                qc[i] = qn[i];
            }
            keep_c = keep_n;
            tv_c = tv_n;
            em_c = em_n;
        }
    }
    __syncthreads();
    if (write_state) {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int c = l + ML_L * i;
            if (p_ok && c < d) sp[c] = S[i];
        }
        if (blockIdx.z == 0 && threadIdx.x == 0) m_state[(long)slot * heads + h] = m_carry;
    }
}

extern "C" const char* cpmcu_mlstm_scan(const void* proj, long ld, int dtype, long q_off, long k_off, long v_off,
                                        long i_off, long f_off, const float* i_bias, const float* f_bias, float cap,
                                        float q_scale, float* S_state, float* n_state, float* m_state, float* y,
                                        float* den, const int* cu_q, const int* seq_slot, int n_seqs, int heads, int d, int dv,
                                        int write_state, hipStream_t stream) {
    CPMCU_REQUIRE(n_seqs > 0 && heads > 0 && d > 0 && dv > 0, "mlstm_scan: empty shape");
    CPMCU_REQUIRE(d <= 1024, "mlstm_scan: a key size of %d is not supported (at most 1024)", d);
    CPMCU_REQUIRE(cap > 0.f, "mlstm_scan: gate cap %g", cap);
    CPMCU_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && i_off >= 0 && f_off >= 0 && q_off + (long)heads * d <= ld &&
                  k_off + (long)heads * d <= ld && v_off + (long)heads * dv <= ld && i_off + heads <= ld && f_off + heads <= ld,
                  "mlstm_scan: columns beyond rows of %ld", ld);
    const int lanes = d > 128 ? 32 : 8, cols = 256 / lanes;
    const int pb = (dv + 1 + cols - 1) / cols;       // the normaliser is walked as column dv
    CPMCU_REQUIRE(heads <= 65535 && pb <= 65535, "mlstm_scan: shape exceeds the launch grid");
    dim3 grid(n_seqs, heads, pb);
    const int need = (d + lanes - 1) / lanes;
#define LAUNCH(NRv, Lv, TTv, Tv)                                                                                     \
    mlstm_scan_kernel<NRv, Lv, TTv, Tv><<<grid, 256, 0, stream>>>((const Tv*)proj, ld, q_off, k_off, v_off, i_off,   \
                                                                  f_off, i_bias, f_bias, cap, q_scale, S_state,      \
                                                                  n_state, m_state, y, den, cu_q, seq_slot, heads,   \
                                                                  d, dv, write_state)
#define BY_NR(Tv)                                  \
    do {                                           \
        if (lanes == 32 && need <= 8) LAUNCH(8, 32, 16, Tv);        \
        else if (lanes == 32 && need <= 16) LAUNCH(16, 32, 8, Tv);  \
        else if (lanes == 32) LAUNCH(32, 32, 4, Tv);                \
        else if (need <= 2) LAUNCH(2, 8, 32, Tv);  \
        else if (need <= 4) LAUNCH(4, 8, 32, Tv);  \
        else if (need <= 8) LAUNCH(8, 8, 32, Tv);  \
        else LAUNCH(16, 8, 32, Tv);                \
    } while (0)
    if (dtype == CPMCU_F32) BY_NR(float);
    else if (dtype == CPMCU_BF16) BY_NR(bf16_t);
    else CPMCU_FAIL("mlstm_scan: unknown dtype %d", dtype);
#undef BY_NR
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("mlstm_scan");
    return nullptr;
}
