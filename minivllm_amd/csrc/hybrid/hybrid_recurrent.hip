// Gated outer-product recurrences with a fp32 matrix state S [D, E] per (sequence, head), for
// prefill portions and single decode tokens alike.  One kernel template, three rules:
//
//   GLA     S <- diag(alpha) S + k v^T;  o = S^T q          alpha = sigmoid(z + b)^(1/tau) per key channel
//   CDELTA  S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q     g per key channel
//   MLSTM   m' = max(f + m, i);  S <- e^(f+m-m') S + e^(i-m') k v^T;  n likewise with k alone;
//           o = S^T q / (max(|n . q|, e^(-m')) + 1e-6)       i, f soft-capped log gates
//
// A state column S[:, e] evolves independently of the others, so a column is owned by 4
// neighbouring lanes, lane r holding d in [r*NR, (r+1)*NR) in registers (D <= 4*NR, missing d
// padded with zeros); sums over d close with two exchanges inside the quad.  Workgroup = 64
// columns of one (sequence, head).  The tokens' operands are staged through LDS in chunks of CT
// tokens, double-buffered: k, q (and the decay vector) of the head as padded [token][quad lane]
// slices read with 16-byte LDS loads, v of the 64 columns, and the per-token scalars.  GLA and
// MLSTM read the raw projections (bfloat16 or float rows of a wider projection output) and do
// the gates' fp32 arithmetic while staging; CDELTA reads the fp32 outputs of delta_prepare.
// MLSTM's running maximum is a sequential max-plus chain over tokens: wave 0 walks it once per
// chunk (two dependent operations per token) and leaves the three factors of every token in LDS;
// the normaliser n is kept by every quad (its d-slice), since every column divides by n . q.
//
// Sequence layout: `cu_q` [B+1] rows of each sequence (null: row b is sequence b), `positions`
// (a sequence's first row holds the position its portion starts at; 0 = start from zeros),
// `slots` [B] state slot per sequence (< 0: unused row of a padded batch).
#include "hybrid_common.h"

using namespace hyb;

enum ScanRule { GLA = 0, CDELTA = 1, MLSTM = 2 };

struct ScanArgs {
    const void *q, *k, *v;          // rows of [*, D] / [*, E] heads; element strides per token below
    long q_row, k_row, v_row;
    const void* a;                  // GLA: raw decay pre-activation [T, H*D]; CDELTA: decay fp32 [T, H*D]
    long a_row;
    const float* a_bias;            // GLA [H*D]
    float tau_inv;
    const void *gi, *gf;            // MLSTM: raw gate pre-activations [T, H]
    long g_row;
    const float *bi, *bf;           // MLSTM [H]
    float cap;
    const float* beta;              // CDELTA [T, H]
    float *state, *nstate, *mstate; // [slots,H,D,E], MLSTM: [slots,H,D], [slots,H]
    const int *cu_q, *positions, *slots;
    float* o;                       // [T, H, E]
    int H, G, D, E;
    float qscale;
};

__device__ __forceinline__ float logsigmoidf_(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename TI, int NR, int MODE>
__global__ void __launch_bounds__(256) gated_scan_kernel(const ScanArgs a) {
    constexpr int CT = NR >= 64 ? 8 : 16;
    constexpr int RS = NR + 4;                  // padded slice: the 4 lanes of a quad hit 4 bank groups
    constexpr int IMG = CT * 4 * RS;            // floats of one [token][quad lane][slice] image
    constexpr int NIMG = MODE == MLSTM ? 2 : 3; // k, q (, decay)
    constexpr int NSC = MODE == MLSTM ? 3 : (MODE == CDELTA ? 1 : 0);    // LDS scalars per token
    constexpr int NSC_IN = MODE == MLSTM ? 2 : NSC;                      // staged scalars per token
    constexpr int BUF = NIMG * IMG + CT * 64 + NSC * CT;
    constexpr int IMG_ITEMS = CT * 4 * NR;
    constexpr int NITEM = NIMG * IMG_ITEMS + CT * 64 + NSC_IN * CT;
    constexpr int NLD = (NITEM + 255) / 256;
    extern __shared__ float sm[];
    const int b = blockIdx.x, h = blockIdx.y;
    const int H = a.H, G = a.G, D = a.D, E = a.E;
    const int slot = a.slots[b];
    if (slot < 0) return;
    const long first = a.cu_q ? a.cu_q[b] : b;
    const int n = a.cu_q ? a.cu_q[b + 1] - a.cu_q[b] : 1;
    if (n <= 0) return;
    const int tid = threadIdx.x, r = tid & 3, c = tid >> 2;
    const int e0 = blockIdx.z * 64, e = e0 + c;
    const bool col = e < E;
    const int g = h / (H / G);
    const int d0 = r * NR;
    const bool has_past = a.positions[first] > 0;
    float S[NR], N[MODE == MLSTM ? NR : 1];
    float* sp = a.state + (((long)slot * H + h) * D) * E + (col ? e : 0);
#pragma unroll
    for (int i = 0; i < NR; ++i)
        S[i] = (has_past && col && d0 + i < D) ? sp[(long)(d0 + i) * E] : 0.f;
    float m_run = 0.f;
    if constexpr (MODE == MLSTM) {
        const float* np = a.nstate + ((long)slot * H + h) * D;
#pragma unroll
        for (int i = 0; i < NR; ++i) N[i] = (has_past && d0 + i < D) ? np[d0 + i] : 0.f;
        if (has_past) m_run = a.mstate[(long)slot * H + h];
    }
    const TI* qp = (const TI*)a.q;
    const TI* kp = (const TI*)a.k;
    const TI* vp = (const TI*)a.v;

    // staging: item j of a chunk = one float of an image (padded to 4*NR per token), of v, or a scalar
    auto fetch = [&](int chunk, float* reg) {
        const long t0 = first + (long)chunk * CT;
        const int nt = min(CT, n - chunk * CT);
#pragma unroll
        for (int x = 0; x < NLD; ++x) {
            const int j = tid + x * 256;
            float v = 0.f;
            if (j < NIMG * IMG_ITEMS) {
                const int which = j / IMG_ITEMS, jj = j - which * IMG_ITEMS;
                const int tok = jj / (4 * NR), d = jj - tok * (4 * NR);
                if (tok < nt && d < D) {
                    const long t = t0 + tok;
                    if (which == 0) v = ld(kp + t * a.k_row + (long)g * D + d);
                    else if (which == 1) v = ld(qp + t * a.q_row + (long)g * D + d) * a.qscale;
                    else if constexpr (MODE == GLA) {
                        const float z = ld((const TI*)a.a + t * a.a_row + (long)h * D + d) + a.a_bias[h * D + d];
                        v = expf(logsigmoidf_(z) * a.tau_inv);
                    } else if constexpr (MODE == CDELTA) {
                        v = ((const float*)a.a)[t * a.a_row + (long)h * D + d];
                    }
                }
            } else if (j < NIMG * IMG_ITEMS + CT * 64) {
                const int jj = j - NIMG * IMG_ITEMS, tok = jj >> 6, cc = jj & 63;
                if (tok < nt && e0 + cc < E) v = ld(vp + (t0 + tok) * a.v_row + (long)h * E + e0 + cc);
            } else if (j < NITEM) {
                const int jj = j - NIMG * IMG_ITEMS - CT * 64, which = jj / CT, tok = jj - which * CT;
                if (tok < nt) {
                    const long t = t0 + tok;
                    if constexpr (MODE == CDELTA) v = a.beta[t * H + h];
                    if constexpr (MODE == MLSTM) {
                        if (which == 0)
                            v = a.cap * tanhf((ld((const TI*)a.gi + t * a.g_row + h) + a.bi[h]) / a.cap);
                        else
                            v = logsigmoidf_(a.cap * tanhf((ld((const TI*)a.gf + t * a.g_row + h) + a.bf[h]) / a.cap));
                    }
                }
            }
            reg[x] = v;
        }
    };
    auto stash = [&](const float* reg, float* buf) {
#pragma unroll
        for (int x = 0; x < NLD; ++x) {
            const int j = tid + x * 256;
            if (j < NIMG * IMG_ITEMS) {
                const int which = j / IMG_ITEMS, jj = j - which * IMG_ITEMS;
                const int tok = jj / (4 * NR), d = jj - tok * (4 * NR);
                buf[which * IMG + (tok * 4 + d / NR) * RS + d % NR] = reg[x];
            } else if (j < NITEM) {
                buf[NIMG * IMG + j - NIMG * IMG_ITEMS] = reg[x];
            }
        }
    };
    // MLSTM: the chunk's raw log gates (i at [0, CT), f at [CT, 2 CT) of the scalar area) become the
    // factors e^(f+m-m'), e^(i-m'), e^(-m') of every token; wave 0 only, m_run is its running maximum
    auto gates = [&](float* buf, int nt) {
        if constexpr (MODE == MLSTM) {
            if (tid < kWave) {
                float* sc = buf + NIMG * IMG + CT * 64;
                const float gi = tid < CT ? sc[tid] : 0.f, gf = tid < CT ? sc[CT + tid] : 0.f;
                float mp = 0.f, mn = 0.f, m = m_run;
#pragma unroll
                for (int s = 0; s < CT; ++s) {
                    const float fs = __shfl(gf, s, kWave), is = __shfl(gi, s, kWave);
                    const float m2 = s < nt ? fmaxf(fs + m, is) : m;
                    if (tid == s) { mp = m; mn = m2; }
                    m = m2;
                }
                m_run = m;
                if (tid < CT) {
                    sc[tid] = expf(gf + mp - mn);
                    sc[CT + tid] = expf(gi - mn);
                    sc[2 * CT + tid] = expf(-mn);
                }
            }
            __syncthreads();
        }
    };
    float reg[NLD];
    fetch(0, reg);
    stash(reg, sm);
    __syncthreads();
    const int nchunks = (n + CT - 1) / CT;
    for (int ch = 0; ch < nchunks; ++ch) {
        float* buf = sm + (ch & 1) * BUF;
        const int nt = min(CT, n - ch * CT);
        gates(buf, nt);
        if (ch + 1 < nchunks) fetch(ch + 1, reg);
        const float* sc = buf + NIMG * IMG + CT * 64;
#pragma unroll 2
        for (int tok = 0; tok < nt; ++tok) {
            const float4* k4p = reinterpret_cast<const float4*>(buf + (tok * 4 + r) * RS);
            const float4* q4p = reinterpret_cast<const float4*>(buf + IMG + (tok * 4 + r) * RS);
            const float ve = buf[NIMG * IMG + tok * 64 + c];
            float kk[NR], qq[NR];
#pragma unroll
            for (int i = 0; i < NR / 4; ++i) {
                const float4 k4 = k4p[i], q4 = q4p[i];
                kk[4 * i] = k4.x; kk[4 * i + 1] = k4.y; kk[4 * i + 2] = k4.z; kk[4 * i + 3] = k4.w;
                qq[4 * i] = q4.x; qq[4 * i + 1] = q4.y; qq[4 * i + 2] = q4.z; qq[4 * i + 3] = q4.w;
            }
            float o4[4] = {0.f, 0.f, 0.f, 0.f};       // four partial sums: no chain of NR dependent FMAs
            float out;
            if constexpr (MODE == MLSTM) {
                const float fs = sc[tok], is = sc[CT + tok], em = sc[2 * CT + tok];
                const float kv = is * ve;
                float n4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < NR; ++i) {
                    S[i] = fs * S[i] + kk[i] * kv;
                    o4[i & 3] += S[i] * qq[i];
                    N[i] = fs * N[i] + is * kk[i];
                    n4[i & 3] += N[i] * qq[i];
                }
                float num = (o4[0] + o4[1]) + (o4[2] + o4[3]), nq = (n4[0] + n4[1]) + (n4[2] + n4[3]);
                num += __shfl_xor(num, 1, kWave); nq += __shfl_xor(nq, 1, kWave);
                num += __shfl_xor(num, 2, kWave); nq += __shfl_xor(nq, 2, kWave);
                out = num / (fmaxf(fabsf(nq), em) + 1e-6f);
            } else {
                const float4* g4p = reinterpret_cast<const float4*>(buf + 2 * IMG + (tok * 4 + r) * RS);
                float gg[NR];
#pragma unroll
                for (int i = 0; i < NR / 4; ++i) {
                    const float4 g4 = g4p[i];
                    gg[4 * i] = g4.x; gg[4 * i + 1] = g4.y; gg[4 * i + 2] = g4.z; gg[4 * i + 3] = g4.w;
                }
                float u = ve;
                if constexpr (MODE == CDELTA) {
                    float d4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int i = 0; i < NR; ++i) {
                        S[i] *= gg[i];
                        d4[i & 3] += S[i] * kk[i];
                    }
                    float dot = (d4[0] + d4[1]) + (d4[2] + d4[3]);
                    dot += __shfl_xor(dot, 1, kWave);
                    dot += __shfl_xor(dot, 2, kWave);
                    u = sc[tok] * (ve - dot);
#pragma unroll
                    for (int i = 0; i < NR; ++i) {
                        S[i] += kk[i] * u;
                        o4[i & 3] += S[i] * qq[i];
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < NR; ++i) {
                        S[i] = gg[i] * S[i] + kk[i] * u;
                        o4[i & 3] += S[i] * qq[i];
                    }
                }
                out = (o4[0] + o4[1]) + (o4[2] + o4[3]);
                out += __shfl_xor(out, 1, kWave);
                out += __shfl_xor(out, 2, kWave);
            }
            if (col && r == 0) a.o[((first + ch * CT + tok) * H + h) * (long)E + e] = out;
        }
        if (ch + 1 < nchunks) stash(reg, sm + ((ch + 1) & 1) * BUF);
        __syncthreads();
    }
    if (col) {
#pragma unroll
        for (int i = 0; i < NR; ++i)
            if (d0 + i < D) sp[(long)(d0 + i) * E] = S[i];
    }
    if constexpr (MODE == MLSTM) {
        if (blockIdx.z == 0 && c == 0) {
            float* np = a.nstate + ((long)slot * H + h) * D;
#pragma unroll
            for (int i = 0; i < NR; ++i)
                if (d0 + i < D) np[d0 + i] = N[i];
            if (tid == 0) a.mstate[(long)slot * H + h] = m_run;
        }
    }
}

template <typename TI, int NR, int MODE>
static void launch_scan(const ScanArgs& a, int B, hipStream_t s) {
    constexpr int CT = NR >= 64 ? 8 : 16;
    constexpr int NIMG = MODE == MLSTM ? 2 : 3;
    constexpr int NSC = MODE == MLSTM ? 3 : (MODE == CDELTA ? 1 : 0);
    constexpr int BUF = NIMG * CT * 4 * (NR + 4) + CT * 64 + NSC * CT;
    hipLaunchKernelGGL((gated_scan_kernel<TI, NR, MODE>), dim3(B, a.H, (a.E + 63) / 64), dim3(256),
                       2 * BUF * sizeof(float), s, a);
}

template <typename TI, int MODE>
static int scan_by_size(const ScanArgs& a, int B, hipStream_t s) {
    if (B <= 0) return 0;
    if (a.G <= 0 || a.H % a.G || a.D > 256 || a.D <= 0 || a.E <= 0) return 1;
    if (a.D <= 32) launch_scan<TI, 8, MODE>(a, B, s);
    else if (a.D <= 64) launch_scan<TI, 16, MODE>(a, B, s);
    else if (a.D <= 128) launch_scan<TI, 32, MODE>(a, B, s);
    else launch_scan<TI, 64, MODE>(a, B, s);
    return HYB_LAUNCH_OK();
}

extern "C" {

// q, k [T, H, D], v [T, H, E], a_raw [T, H*D]: rows of the activation type with element strides
// q_row .. a_row; state [slots, H, D, E]; o [T, H, E] fp32.
int hyb_gla_scan(const void* q, const void* k, const void* v, long q_row, long k_row, long v_row,
                 const void* a_raw, long a_row, const void* a_bias, float tau, void* state,
                 const void* cu_q, const void* positions, const void* slots, void* o, int B, int H,
                 int D, int E, int dt, hipStream_t s) {
    ScanArgs a{};
    a.q = q; a.k = k; a.v = v; a.q_row = q_row; a.k_row = k_row; a.v_row = v_row;
    a.a = a_raw; a.a_row = a_row; a.a_bias = (const float*)a_bias; a.tau_inv = 1.f / tau;
    a.state = (float*)state; a.cu_q = (const int*)cu_q; a.positions = (const int*)positions;
    a.slots = (const int*)slots; a.o = (float*)o; a.H = H; a.G = H; a.D = D; a.E = E;
    a.qscale = 1.f / sqrtf((float)D);
    HYB_DISPATCH(dt, return (scan_by_size<T, GLA>(a, B, s)));
    return 1;
}

// gi, gf [T, H] raw gate projections (activation type, element stride g_row); nstate [slots, H, D],
// mstate [slots, H].
int hyb_mlstm_scan(const void* q, const void* k, const void* v, long q_row, long k_row, long v_row,
                   const void* gi, const void* gf, long g_row, const void* bi, const void* bf,
                   float cap, void* state, void* nstate, void* mstate, const void* cu_q,
                   const void* positions, const void* slots, void* o, int B, int H, int D, int E,
                   int dt, hipStream_t s) {
    ScanArgs a{};
    a.q = q; a.k = k; a.v = v; a.q_row = q_row; a.k_row = k_row; a.v_row = v_row;
    a.gi = gi; a.gf = gf; a.g_row = g_row; a.bi = (const float*)bi; a.bf = (const float*)bf;
    a.cap = cap; a.state = (float*)state; a.nstate = (float*)nstate; a.mstate = (float*)mstate;
    a.cu_q = (const int*)cu_q; a.positions = (const int*)positions; a.slots = (const int*)slots;
    a.o = (float*)o; a.H = H; a.G = H; a.D = D; a.E = E; a.qscale = 1.f / sqrtf((float)D);
    HYB_DISPATCH(dt, return (scan_by_size<T, MLSTM>(a, B, s)));
    return 1;
}

// fp32 outputs of delta_prepare: qn, kn [T, G, D], vv [T, H, E], beta [T, H], decay [T, H, D].
int hyb_channel_delta_scan(const void* qn, const void* kn, const void* vv, const void* beta,
                           const void* decay, void* state, const void* cu_q, const void* positions,
                           const void* slots, void* o, int B, int H, int G, int D, int E,
                           hipStream_t s) {
    ScanArgs a{};
    a.q = qn; a.k = kn; a.v = vv; a.q_row = (long)G * D; a.k_row = (long)G * D; a.v_row = (long)H * E;
    a.a = decay; a.a_row = (long)H * D; a.beta = (const float*)beta; a.state = (float*)state;
    a.cu_q = (const int*)cu_q; a.positions = (const int*)positions; a.slots = (const int*)slots;
    a.o = (float*)o; a.H = H; a.G = G; a.D = D; a.E = E; a.qscale = 1.f;
    return scan_by_size<float, CDELTA>(a, B, s);
}

}  // extern "C"
