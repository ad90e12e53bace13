// Gated outer-product recurrences with a fp32 matrix state S [D, E] per (sequence, head), for
// prefill portions and single decode tokens alike.  One kernel template, three rules:
//
//   GLA     S <- diag(alpha) S + k v^T;  o = S^T q          alpha = sigmoid(z + b)^(1/tau) per key channel
//   CDELTA  S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q     g per key channel
//   MLSTM   m' = max(f + m, i);  S <- e^(f+m-m') S + e^(i-m') k v^T;  n likewise with k alone;
//           o = S^T q / (max(|n . q|, e^(-m')) + 1e-6)       i, f soft-capped log gates
//
// A state column S[:, e] evolves independently of the others, so a column is owned by LPC
// neighbouring lanes (4, 8 or 16), lane r holding d in [r*NR, (r+1)*NR) in registers
// (D <= LPC*NR, missing d padded with zeros); sums over d close with log2(LPC) exchanges inside
// the group.  Workgroup = 256 / LPC columns of one (sequence, head).  LPC is chosen per launch: 4
// when that already gives every SIMD of the chip two waves (decode batches), more lanes per
// column - shorter dependent chains per token, more waves to hide their latency - when the step
// has few (sequence, head) pairs (prompt portions).  The tokens' operands are staged through LDS
// in chunks of CT tokens, double-buffered: k, q (and the decay vector) of the head as padded
// [token][group lane] slices read with 16-byte LDS loads, v of the workgroup's columns, and the
// per-token scalars.  GLA and
// MLSTM read the raw projections (bfloat16 or float rows of a wider projection output) and do
// the gates' fp32 arithmetic while staging; CDELTA reads the fp32 outputs of delta_prepare.
// MLSTM's running maximum is a sequential max-plus chain over tokens: wave 0 walks it once per
// chunk (two dependent operations per token) and leaves the three factors of every token in LDS;
// the normaliser n is kept by every lane group (its d-slice), since every column divides by n . q.
//
// Sequence layout: `cu_q` [B+1] rows of each sequence (null: row b is sequence b), `positions`
// (a sequence's first row holds the position its portion starts at; 0 = start from zeros),
// `slots` [B] state slot per sequence (< 0: unused row of a padded batch).
#include "hybrid_common.h"
#include <stdlib.h>

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
    float *state, *nstate, *mstate; // [slots,H,D,E]; MLSTM: [slots,H,ZG,D], [slots,H,ZG], ZG = ceil(E/16)
    const int *cu_q, *positions, *slots;
    float* o;                       // [T, H, E]
    int H, G, D, E;
    float qscale;
};

__device__ __forceinline__ float logsigmoidf_(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename TI, int NR, int LPC, int MODE>
__global__ void __launch_bounds__(256) gated_scan_kernel(const ScanArgs a) {
    constexpr int CT = NR >= 64 ? 8 : 16;
    constexpr int COLS = 256 / LPC;             // state columns per workgroup
    constexpr int RS = NR + 4;                  // padded slice: neighbouring lanes hit different bank groups
    constexpr int IMG = CT * LPC * RS;          // floats of one [token][group lane][slice] image
    constexpr int NIMG = MODE == MLSTM ? 2 : 3; // k, q (, decay)
    constexpr int NSC = MODE == MLSTM ? 3 : (MODE == CDELTA ? 1 : 0);    // LDS scalars per token
    constexpr int NSC_IN = MODE == MLSTM ? 2 : NSC;                      // staged scalars per token
    constexpr int BUF = NIMG * IMG + CT * COLS + NSC * CT;
    constexpr int IMG_ITEMS = CT * LPC * NR;
    constexpr int NITEM = NIMG * IMG_ITEMS + CT * COLS + NSC_IN * CT;
    constexpr int NLD = (NITEM + 255) / 256;
    extern __shared__ float sm[];
    const int b = blockIdx.x, h = blockIdx.y;
    const int H = a.H, G = a.G, D = a.D, E = a.E;
    const int slot = a.slots[b];
    if (slot < 0) return;
    const long first = a.cu_q ? a.cu_q[b] : b;
    const int n = a.cu_q ? a.cu_q[b + 1] - a.cu_q[b] : 1;
    if (n <= 0) return;
    const int tid = threadIdx.x, r = tid % LPC, c = tid / LPC;
    const int e0 = blockIdx.z * COLS, e = e0 + c;
    const bool col = e < E;
    const int g = h / (H / G);
    const int d0 = r * NR;
    const bool has_past = a.positions[first] > 0;
    // MLSTM's normaliser n and running maximum m are the same for every column, but the workgroups
    // of one (sequence, head) - one per block of columns - each read them when they start and would
    // overwrite them when they end: so the slot keeps one copy per 16 columns (the smallest block),
    // and a workgroup reads the copy of its first 16 columns and writes those of all it covers
    const int ZG = (E + 15) / 16, zg0 = e0 / 16;
    constexpr int NZG = COLS / 16;
    float S[NR], N[MODE == MLSTM ? NR : 1];
    float* sp = a.state + (((long)slot * H + h) * D) * E + (col ? e : 0);
#pragma unroll
    for (int i = 0; i < NR; ++i)
        S[i] = (has_past && col && d0 + i < D) ? sp[(long)(d0 + i) * E] : 0.f;
    float m_run = 0.f;
    if constexpr (MODE == MLSTM) {
        const float* np = a.nstate + (((long)slot * H + h) * ZG + zg0) * D;
#pragma unroll
        for (int i = 0; i < NR; ++i) N[i] = (has_past && d0 + i < D) ? np[d0 + i] : 0.f;
        if (has_past) m_run = a.mstate[((long)slot * H + h) * ZG + zg0];
    }
    const TI* qp = (const TI*)a.q;
    const TI* kp = (const TI*)a.k;
    const TI* vp = (const TI*)a.v;

    if (n == 1) {
        // A single token (decode rows, one-token portions): k, q and the decay vector of the head
        // (and MLSTM's three factors) are worked out once per workgroup into LDS, every lane then
        // takes its slice and its column's v, updates, reduces.  No chunk machinery.
        const long t = first;
        constexpr int DP = LPC * NR;
        for (int i = tid; i < NIMG * DP; i += 256) {
            const int which = i / DP, d = i - which * DP;
            float v = 0.f;
            if (d < D) {
                if (which == 0) v = ld(kp + t * a.k_row + (long)g * D + d);
                else if (which == 1) v = ld(qp + t * a.q_row + (long)g * D + d) * a.qscale;
                else if constexpr (MODE == GLA)
                    v = expf(logsigmoidf_(ld((const TI*)a.a + t * a.a_row + (long)h * D + d) +
                                          a.a_bias[h * D + d]) * a.tau_inv);
                else if constexpr (MODE == CDELTA) v = ((const float*)a.a)[t * a.a_row + (long)h * D + d];
            }
            sm[i] = v;
        }
        if constexpr (MODE == MLSTM) {
            if (tid == 0) {
                const float gi = a.cap * tanhf((ld((const TI*)a.gi + t * a.g_row + h) + a.bi[h]) / a.cap);
                const float gf = logsigmoidf_(a.cap * tanhf((ld((const TI*)a.gf + t * a.g_row + h) + a.bf[h]) / a.cap));
                const float m2 = fmaxf(gf + m_run, gi);
                sm[NIMG * DP] = expf(gf + m_run - m2);
                sm[NIMG * DP + 1] = expf(gi - m2);
                sm[NIMG * DP + 2] = expf(-m2);
                sm[NIMG * DP + 3] = m2;
            }
        }
        __syncthreads();
        float kk[NR], qq[NR], gg[MODE == MLSTM ? 1 : NR];
#pragma unroll
        for (int i = 0; i < NR / 4; ++i) {
            const float4 k4 = reinterpret_cast<const float4*>(sm + d0)[i];
            const float4 q4 = reinterpret_cast<const float4*>(sm + DP + d0)[i];
            kk[4 * i] = k4.x; kk[4 * i + 1] = k4.y; kk[4 * i + 2] = k4.z; kk[4 * i + 3] = k4.w;
            qq[4 * i] = q4.x; qq[4 * i + 1] = q4.y; qq[4 * i + 2] = q4.z; qq[4 * i + 3] = q4.w;
            if constexpr (MODE != MLSTM) {
                const float4 g4 = reinterpret_cast<const float4*>(sm + 2 * DP + d0)[i];
                gg[4 * i] = g4.x; gg[4 * i + 1] = g4.y; gg[4 * i + 2] = g4.z; gg[4 * i + 3] = g4.w;
            }
        }
        const float ve = col ? ld(vp + t * a.v_row + (long)h * E + e) : 0.f;
        float po = 0.f, pn = 0.f, em = 0.f;
        if constexpr (MODE == MLSTM) {
            const float fs = sm[NIMG * DP], is = sm[NIMG * DP + 1];
            em = sm[NIMG * DP + 2];
            m_run = sm[NIMG * DP + 3];
            const float kv = is * ve;
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                S[i] = fs * S[i] + kk[i] * kv;
                po += S[i] * qq[i];
                N[i] = fs * N[i] + is * kk[i];
                pn += N[i] * qq[i];
            }
        } else if constexpr (MODE == CDELTA) {
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                S[i] *= gg[i];
                dot += S[i] * kk[i];
            }
#pragma unroll
            for (int x = 1; x < LPC; x <<= 1) dot += __shfl_xor(dot, x, kWave);
            const float u = a.beta[t * H + h] * (ve - dot);
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                S[i] += kk[i] * u;
                po += S[i] * qq[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                S[i] = gg[i] * S[i] + kk[i] * ve;
                po += S[i] * qq[i];
            }
        }
#pragma unroll
        for (int x = 1; x < LPC; x <<= 1) {
            po += __shfl_xor(po, x, kWave);
            if constexpr (MODE == MLSTM) pn += __shfl_xor(pn, x, kWave);
        }
        if (col) {
            if (r == 0) {
                if constexpr (MODE == MLSTM) po /= fmaxf(fabsf(pn), em) + 1e-6f;
                a.o[(t * H + h) * (long)E + e] = po;
            }
#pragma unroll
            for (int i = 0; i < NR; ++i)
                if (d0 + i < D) sp[(long)(d0 + i) * E] = S[i];
        }
        if constexpr (MODE == MLSTM) {
            if (c < NZG && zg0 + c < ZG) {              // (these lanes sit in wave 0, which owns m_run)
                float* np = a.nstate + (((long)slot * H + h) * ZG + zg0 + c) * D;
#pragma unroll
                for (int i = 0; i < NR; ++i)
                    if (d0 + i < D) np[d0 + i] = N[i];
                if (r == 0) a.mstate[((long)slot * H + h) * ZG + zg0 + c] = m_run;
            }
        }
        return;
    }

    // Staging.  Item j = tid + 256 x of a chunk is one element of an image (padded to LPC*NR per
    // token), of v, or a scalar; which tensor, token-in-chunk and channel an item is does not
    // change from chunk to chunk (and, the regions being multiples of 256 items, which REGION an x
    // belongs to is known at compile time), so its global offset, LDS offset and bias are worked
    // out once.  fetch() only issues the loads (raw values, nothing waits for them before the
    // chunk's token loop); stash() converts, applies the gate arithmetic and writes LDS.
    constexpr int X_IMG = NIMG * IMG_ITEMS / 256, X_V = CT * COLS / 256;
    static_assert(IMG_ITEMS % 256 == 0 && (CT * COLS) % 256 == 0, "staging regions are whole rounds");
    constexpr bool HAS_AUX = MODE != CDELTA;
    int goff[NLD];                  // element offset from the chunk's first row (< 0: the item is 0)
    int ldso[NLD];                  // where it goes in the LDS buffer (< 0: nowhere)
    float aux[HAS_AUX ? NLD : 1];   // GLA: the decay channel's bias; MLSTM: the gate's bias
    auto item_tok = [&](int x) {    // token-in-chunk of item x (shifts: every size is a power of two)
        const int j = tid + x * 256;
        if (x < X_IMG) return (j % IMG_ITEMS) / (LPC * NR);
        if (x < X_IMG + X_V) return (j - NIMG * IMG_ITEMS) / COLS;
        return (j - NIMG * IMG_ITEMS - CT * COLS) % CT;
    };
#pragma unroll
    for (int x = 0; x < NLD; ++x) {
        const int j = tid + x * 256, tok = item_tok(x);
        goff[x] = -1; ldso[x] = -1;
        if constexpr (HAS_AUX) aux[x] = 0.f;
        if (x < X_IMG) {
            const int which = (x * 256) / IMG_ITEMS, d = (j % IMG_ITEMS) % (LPC * NR);
            ldso[x] = which * IMG + (tok * LPC + d / NR) * RS + d % NR;
            if (d < D) {
                if (which == 0) goff[x] = tok * (int)a.k_row + g * D + d;
                else if (which == 1) goff[x] = tok * (int)a.q_row + g * D + d;
                else {
                    goff[x] = tok * (int)a.a_row + h * D + d;
                    if constexpr (MODE == GLA) aux[x] = a.a_bias[h * D + d];
                }
            }
        } else if (x < X_IMG + X_V) {
            const int jj = j - NIMG * IMG_ITEMS, cc = jj % COLS;
            ldso[x] = NIMG * IMG + jj;
            if (e0 + cc < E) goff[x] = tok * (int)a.v_row + h * E + e0 + cc;
        } else if (j < NITEM) {
            const int jj = j - NIMG * IMG_ITEMS - CT * COLS, which = jj / CT;
            ldso[x] = NIMG * IMG + CT * COLS + jj;
            if constexpr (MODE == CDELTA) goff[x] = tok * H + h;
            if constexpr (MODE == MLSTM) {
                goff[x] = tok * (int)a.g_row + h;
                aux[x] = which == 0 ? a.bi[h] : a.bf[h];
            }
        }
    }
    auto fetch = [&](int chunk, TI* raw) {
        const int nt = min(CT, n - chunk * CT);
        const long t0 = first + (long)chunk * CT;
        const TI* kc = kp + t0 * a.k_row;
        const TI* qc = qp + t0 * a.q_row;
        const TI* vc = vp + t0 * a.v_row;
        const TI* ac = MODE == MLSTM ? nullptr : (const TI*)a.a + t0 * a.a_row;
        const TI* bc = MODE == CDELTA ? (const TI*)a.beta + t0 * H : nullptr;
        const TI* gic = MODE == MLSTM ? (const TI*)a.gi + t0 * a.g_row : nullptr;
        const TI* gfc = MODE == MLSTM ? (const TI*)a.gf + t0 * a.g_row : nullptr;
#pragma unroll
        for (int x = 0; x < NLD; ++x) {
            raw[x] = TI{};
            if (goff[x] < 0 || item_tok(x) >= nt) continue;
            if (x < X_IMG) {
                const int which = (x * 256) / IMG_ITEMS;
                raw[x] = (which == 0 ? kc : which == 1 ? qc : ac)[goff[x]];
            } else if (x < X_IMG + X_V) {
                raw[x] = vc[goff[x]];
            } else {
                if constexpr (MODE == CDELTA) raw[x] = bc[goff[x]];
                if constexpr (MODE == MLSTM)
                    raw[x] = ((tid + x * 256 - NIMG * IMG_ITEMS - CT * COLS) / CT ? gfc : gic)[goff[x]];
            }
        }
    };
    auto stash = [&](int chunk, const TI* raw, float* buf) {
        const int nt = min(CT, n - chunk * CT);
#pragma unroll
        for (int x = 0; x < NLD; ++x) {
            if (ldso[x] < 0) continue;
            float v = 0.f;
            if (goff[x] >= 0 && item_tok(x) < nt) {
                v = ld(raw + x);
                if (x < X_IMG) {
                    const int which = (x * 256) / IMG_ITEMS;
                    if (which == 1) v *= a.qscale;
                    if constexpr (MODE == GLA)
                        if (which == 2) v = expf(logsigmoidf_(v + aux[x]) * a.tau_inv);
                } else if (x >= X_IMG + X_V) {
                    if constexpr (MODE == MLSTM) {
                        v = a.cap * tanhf((v + aux[x]) / a.cap);
                        if ((tid + x * 256 - NIMG * IMG_ITEMS - CT * COLS) / CT) v = logsigmoidf_(v);
                    }
                }
            }
            buf[ldso[x]] = v;
        }
    };
    // MLSTM: the chunk's raw log gates (i at [0, CT), f at [CT, 2 CT) of the scalar area) become the
    // factors e^(f+m-m'), e^(i-m'), e^(-m') of every token; wave 0 only, m_run is its running maximum
    auto gates = [&](float* buf, int nt) {
        if constexpr (MODE == MLSTM) {
            if (tid < kWave) {
                float* sc = buf + NIMG * IMG + CT * COLS;
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
    TI reg[NLD];
    fetch(0, reg);
    stash(0, reg, sm);
    __syncthreads();
    const int nchunks = (n + CT - 1) / CT;
    for (int ch = 0; ch < nchunks; ++ch) {
        float* buf = sm + (ch & 1) * BUF;
        const int nt = min(CT, n - ch * CT);
        gates(buf, nt);
        if (ch + 1 < nchunks) fetch(ch + 1, reg);
        const float* sc = buf + NIMG * IMG + CT * COLS;
        // TB tokens back to back, then their sums over d together: only the state update is a chain
        // from token to token, so the exchanges (and the stores behind them) of one token do not
        // hold up the next one's loads and FMAs
        constexpr int TB = 4;
        for (int tb = 0; tb < nt; tb += TB) {
            float po[TB], pn[MODE == MLSTM ? TB : 1];
#pragma unroll
            for (int j = 0; j < TB; ++j) {
                const int tok = tb + j;
                po[j] = 0.f;
                if constexpr (MODE == MLSTM) pn[j] = 0.f;
                if (tok >= nt) continue;
                const float4* k4p = reinterpret_cast<const float4*>(buf + (tok * LPC + r) * RS);
                const float4* q4p = reinterpret_cast<const float4*>(buf + IMG + (tok * LPC + r) * RS);
                const float ve = buf[NIMG * IMG + tok * COLS + c];
                float kk[NR], qq[NR];
#pragma unroll
                for (int i = 0; i < NR / 4; ++i) {
                    const float4 k4 = k4p[i], q4 = q4p[i];
                    kk[4 * i] = k4.x; kk[4 * i + 1] = k4.y; kk[4 * i + 2] = k4.z; kk[4 * i + 3] = k4.w;
                    qq[4 * i] = q4.x; qq[4 * i + 1] = q4.y; qq[4 * i + 2] = q4.z; qq[4 * i + 3] = q4.w;
                }
                float o4[4] = {0.f, 0.f, 0.f, 0.f};   // four partial sums: no chain of NR dependent FMAs
                if constexpr (MODE == MLSTM) {
                    const float fs = sc[tok], is = sc[CT + tok];
                    const float kv = is * ve;
                    float n4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int i = 0; i < NR; ++i) {
                        S[i] = fs * S[i] + kk[i] * kv;
                        o4[i & 3] += S[i] * qq[i];
                        N[i] = fs * N[i] + is * kk[i];
                        n4[i & 3] += N[i] * qq[i];
                    }
                    pn[j] = (n4[0] + n4[1]) + (n4[2] + n4[3]);
                } else {
                    const float4* g4p = reinterpret_cast<const float4*>(buf + 2 * IMG + (tok * LPC + r) * RS);
                    float gg[NR];
#pragma unroll
                    for (int i = 0; i < NR / 4; ++i) {
                        const float4 g4 = g4p[i];
                        gg[4 * i] = g4.x; gg[4 * i + 1] = g4.y; gg[4 * i + 2] = g4.z; gg[4 * i + 3] = g4.w;
                    }
                    if constexpr (MODE == CDELTA) {
                        float d4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int i = 0; i < NR; ++i) {
                            S[i] *= gg[i];
                            d4[i & 3] += S[i] * kk[i];
                        }
                        float dot = (d4[0] + d4[1]) + (d4[2] + d4[3]);
#pragma unroll
                        for (int x = 1; x < LPC; x <<= 1) dot += __shfl_xor(dot, x, kWave);
                        const float u = sc[tok] * (ve - dot);
#pragma unroll
                        for (int i = 0; i < NR; ++i) {
                            S[i] += kk[i] * u;
                            o4[i & 3] += S[i] * qq[i];
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < NR; ++i) {
                            S[i] = gg[i] * S[i] + kk[i] * ve;
                            o4[i & 3] += S[i] * qq[i];
                        }
                    }
                }
                po[j] = (o4[0] + o4[1]) + (o4[2] + o4[3]);
            }
#pragma unroll
            for (int x = 1; x < LPC; x <<= 1) {
#pragma unroll
                for (int j = 0; j < TB; ++j) {
                    po[j] += __shfl_xor(po[j], x, kWave);
                    if constexpr (MODE == MLSTM) pn[j] += __shfl_xor(pn[j], x, kWave);
                }
            }
            // every lane of a group holds the sums now: lane j writes token j's
#pragma unroll
            for (int j = 0; j < TB; ++j) {
                const int tok = tb + j;
                if (tok < nt && col && r == j) {
                    float out = po[j];
                    if constexpr (MODE == MLSTM) out /= fmaxf(fabsf(pn[j]), sc[2 * CT + tok]) + 1e-6f;
                    a.o[((first + ch * CT + tok) * H + h) * (long)E + e] = out;
                }
            }
        }
        if (ch + 1 < nchunks) stash(ch + 1, reg, sm + ((ch + 1) & 1) * BUF);
        __syncthreads();
    }
    if (col) {
#pragma unroll
        for (int i = 0; i < NR; ++i)
            if (d0 + i < D) sp[(long)(d0 + i) * E] = S[i];
    }
    if constexpr (MODE == MLSTM) {
        if (c < NZG && zg0 + c < ZG) {              // (these lanes sit in wave 0, which owns m_run)
            float* np = a.nstate + (((long)slot * H + h) * ZG + zg0 + c) * D;
#pragma unroll
            for (int i = 0; i < NR; ++i)
                if (d0 + i < D) np[d0 + i] = N[i];
            if (r == 0) a.mstate[((long)slot * H + h) * ZG + zg0 + c] = m_run;
        }
    }
}

template <typename TI, int NR, int LPC, int MODE>
static void launch_scan(const ScanArgs& a, int B, hipStream_t s) {
    constexpr int CT = NR >= 64 ? 8 : 16;
    constexpr int COLS = 256 / LPC;
    constexpr int NIMG = MODE == MLSTM ? 2 : 3;
    constexpr int NSC = MODE == MLSTM ? 3 : (MODE == CDELTA ? 1 : 0);
    constexpr int BUF = NIMG * CT * LPC * (NR + 4) + CT * COLS + NSC * CT;
    hipLaunchKernelGGL((gated_scan_kernel<TI, NR, LPC, MODE>), dim3(B, a.H, (a.E + COLS - 1) / COLS),
                       dim3(256), 2 * BUF * sizeof(float), s, a);
}

// Lanes per state column: the fewest of 4 / 8 / 16 that give every CU a workgroup
// (B * H * ceil(E * LPC / 256) workgroups of 4 waves; measured on 8 x 1024-token portions: 8 lanes
// beat 4 by 1.3x for the rules without a dependency inside a token, while the delta rule, whose
// update waits for a sum over d, is fastest with 4 whenever that fills half the chip);
// MINIVLLM_SCAN_LPC in the environment overrides (read at every launch: tests switch it).
template <int MODE>
static int pick_lpc(const ScanArgs& a, int B) {
    const char* env = getenv("MINIVLLM_SCAN_LPC");
    const int forced = env ? atoi(env) : 0;
    if (forced == 4 || forced == 8 || forced == 16) return forced;
    const long want = MODE == CDELTA ? 128 : 256;
    for (int lpc = 4; lpc < 16; lpc *= 2)
        if ((long)B * a.H * ((a.E * lpc + 255) / 256) >= want) return lpc;
    return 16;
}

template <typename TI, int MODE>
static int scan_by_size(const ScanArgs& a, int B, hipStream_t s) {
    if (B <= 0) return 0;
    if (a.G <= 0 || a.H % a.G || a.D > 256 || a.D <= 0 || a.E <= 0) return 1;
    const int lpc = pick_lpc<MODE>(a, B);
#define SCAN3(N4, N8, N16)                                                   \
    do {                                                                     \
        if (lpc == 4) launch_scan<TI, N4, 4, MODE>(a, B, s);                 \
        else if (lpc == 8) launch_scan<TI, N8, 8, MODE>(a, B, s);            \
        else launch_scan<TI, N16, 16, MODE>(a, B, s);                        \
    } while (0)
    if (a.D <= 32) {
        if (lpc == 4) launch_scan<TI, 8, 4, MODE>(a, B, s);
        else launch_scan<TI, 4, 8, MODE>(a, B, s);
    } else if (a.D <= 64) SCAN3(16, 8, 4);
    else if (a.D <= 128) SCAN3(32, 16, 8);
    else SCAN3(64, 32, 16);
#undef SCAN3
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

// gi, gf [T, H] raw gate projections (activation type, element stride g_row); nstate
// [slots, H, ZG, D], mstate [slots, H, ZG] with ZG = ceil(E / 16) identical copies.
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
