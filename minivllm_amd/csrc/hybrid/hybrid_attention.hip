// Causal attention over a paged cache with a sink term in the softmax denominator, separate key
// and value head sizes, grouped query heads and an optional sigmoid gate per head.  fp32 scores,
// weights and accumulation for bfloat16 and float caches alike.
//
// One workgroup (256 threads) per (query row, group of up to RC query heads that share a KV
// head).  The keys of the row's context are walked in tiles of 256: a thread scores one key of
// the tile against the RC heads (key read once), the tile's maximum and sum update the running
// softmax, then the threads switch roles and each owns output columns (head, e) whose weighted
// value sum it extends over the tile's keys (value rows read coalesced).  The running maximum
// starts at the sink and the running sum at 1 = exp(sink - sink): the sink is a key without a
// value.  Rows: a decode batch (row b = sequence b, context_lens[b] keys) or the rows of a
// prefill-form step (row_seq gives the sequence, positions[t] + 1 keys).
#include "hybrid_common.h"

using namespace hyb;

constexpr int TILE = 256;
constexpr int RC = 4;       // query heads per workgroup
constexpr int NACC = 4;     // output columns per thread: RC * E <= NACC * 256

template <typename T> struct Vec4;
template <> struct Vec4<float> {
    static __device__ __forceinline__ void load(const float* p, float* o) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
};
template <> struct Vec4<bf16_t> {
    static __device__ __forceinline__ void load(const bf16_t* p, float* o) {
        const uint2 v = *reinterpret_cast<const uint2*>(p);
        o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
        o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
    }
};

template <typename T>
__global__ void __launch_bounds__(TILE)
sink_attention_rows_kernel(const T* __restrict__ q, long q_row, long q_head,
                           const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                           const int* __restrict__ block_tables, int max_blocks, int block_size,
                           const int* __restrict__ row_seq, const int* __restrict__ lens,
                           int len_add, const float* __restrict__ sink,
                           const T* __restrict__ gate, long gate_row, T* __restrict__ out,
                           float scale, int H, int G, int D, int E, int vec_ok) {
    extern __shared__ float sm[];
    const int R = H / G;
    const int chunks = (R + RC - 1) / RC;
    const long t = blockIdx.x;
    const int g = blockIdx.y / chunks, h0 = g * R + (blockIdx.y % chunks) * RC;
    const int nr = min(RC, g * R + R - h0);
    const int b = row_seq ? row_seq[t] : (int)t;
    if (b < 0) return;
    const int ctx = lens[row_seq ? t : b] + len_add;
    if (ctx <= 0) return;
    const int* table = block_tables + (long)b * max_blocks;
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid & (kWave - 1);

    float* qs = sm;                           // [RC][D]
    float* ps = qs + RC * D;                  // [RC][TILE]
    float* wred = ps + RC * TILE;             // [4 waves][RC]
    float* stat = wred + 4 * RC;              // [RC] alpha, then [RC] running max, [RC] running sum
    long* rowbase = reinterpret_cast<long*>(stat + 3 * RC + 1 + ((3 * RC + 1) & 1));   // [TILE]

    for (int i = tid; i < nr * D; i += TILE) {
        const int r = i / D, d = i - r * D;
        qs[r * D + d] = ld(q + t * q_row + (long)(h0 + r) * q_head + d) * scale;
    }
    if (tid < RC) {
        stat[RC + tid] = tid < nr ? sink[h0 + tid] : 0.f;       // running max
        stat[2 * RC + tid] = 1.f;                               // running sum (the sink's term)
    }
    float acc[NACC];
#pragma unroll
    for (int a = 0; a < NACC; ++a) acc[a] = 0.f;
    __syncthreads();

    for (int j0 = 0; j0 < ctx; j0 += TILE) {
        const int j = j0 + tid;
        const bool live = j < ctx;
        float s[RC];
#pragma unroll
        for (int r = 0; r < RC; ++r) s[r] = -INFINITY;
        if (live) {
            const long slot = (long)table[j / block_size] * block_size + j % block_size;
            rowbase[tid] = slot;
            const T* kr = k_cache + (slot * G + g) * (long)D;
#pragma unroll
            for (int r = 0; r < RC; ++r) s[r] = 0.f;
            if (vec_ok) {
                for (int d = 0; d < D; d += 4) {
                    float kv[4];
                    Vec4<T>::load(kr + d, kv);
#pragma unroll
                    for (int r = 0; r < RC; ++r)
                        if (r < nr) {
                            const float* qq = qs + r * D + d;
                            s[r] += kv[0] * qq[0] + kv[1] * qq[1] + kv[2] * qq[2] + kv[3] * qq[3];
                        }
                }
            } else {
                for (int d = 0; d < D; ++d) {
                    const float kv = ld(kr + d);
#pragma unroll
                    for (int r = 0; r < RC; ++r) if (r < nr) s[r] += kv * qs[r * D + d];
                }
            }
        }
        // tile maximum per head
#pragma unroll
        for (int r = 0; r < RC; ++r) {
            const float m = wave_max(s[r]);
            if (lane == 0) wred[wave * RC + r] = m;
        }
        __syncthreads();
        float mnew[RC];
#pragma unroll
        for (int r = 0; r < RC; ++r) {
            float m = stat[RC + r];
            for (int w = 0; w < TILE / kWave; ++w) m = fmaxf(m, wred[w * RC + r]);
            mnew[r] = m;
        }
        float psum[RC];
#pragma unroll
        for (int r = 0; r < RC; ++r) {
            const float p = (live && r < nr) ? expf(s[r] - mnew[r]) : 0.f;
            ps[r * TILE + tid] = p;
            psum[r] = wave_sum(p);
        }
        __syncthreads();                       // every thread has read wred and stat
#pragma unroll
        for (int r = 0; r < RC; ++r) if (lane == 0) wred[wave * RC + r] = psum[r];
        __syncthreads();
        if (tid < RC) {
            const int r = tid;
            const float alpha = expf(stat[RC + r] - mnew[r]);
            float l = stat[2 * RC + r] * alpha;
            for (int w = 0; w < TILE / kWave; ++w) l += wred[w * RC + r];
            stat[r] = alpha;
            stat[RC + r] = mnew[r];
            stat[2 * RC + r] = l;
        }
        __syncthreads();
        // weighted value sums: thread owns columns c = tid + a * TILE of [nr][E]
        const int n = min(TILE, ctx - j0);
#pragma unroll
        for (int a = 0; a < NACC; ++a) {
            const int c = tid + a * TILE;
            if (c < nr * E) {
                const int r = c / E, e = c - r * E;
                float o = acc[a] * stat[r];
                const float* pr = ps + r * TILE;
                const T* vb = v_cache + (long)g * E + e;
                for (int jj = 0; jj < n; ++jj) o += pr[jj] * ld(vb + rowbase[jj] * (long)(G * E));
                acc[a] = o;
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int a = 0; a < NACC; ++a) {
        const int c = tid + a * TILE;
        if (c < nr * E) {
            const int r = c / E, e = c - r * E;
            float o = acc[a] / stat[2 * RC + r];
            if (gate) o *= sigmoidf_(ld(gate + t * gate_row + h0 + r));
            st(out + (t * H + h0 + r) * (long)E + e, o);
        }
    }
}

extern "C" {

// q: [rows, H, D] with strides (q_row, q_head, 1); caches contiguous [blocks, block, G, D|E];
// out contiguous [rows, H, E]; gate [rows, H] with row stride gate_row (or null).
int hyb_sink_attention_rows(const void* q, long q_row, long q_head, const void* k_cache,
                            const void* v_cache, const void* block_tables, int max_blocks,
                            int block_size, const void* row_seq, const void* lens, int len_add,
                            const void* sink, const void* gate, long gate_row, void* out,
                            float scale, long rows, int H, int G, int D, int E, int dt,
                            hipStream_t s) {
    if (rows <= 0) return 0;
    if (G <= 0 || H % G || RC * E > NACC * TILE || D > 1024) return 1;
    const int R = H / G, chunks = (R + RC - 1) / RC;
    const size_t lds = (RC * D + RC * TILE + 4 * RC + 3 * RC + 2) * sizeof(float) + TILE * sizeof(long);
    const int esize = dt == 0 ? 2 : 4;
    const int vec_ok = (D % 4 == 0) && (((size_t)k_cache) % 16 == 0) && ((D * esize) % (4 * esize) == 0);
    HYB_DISPATCH(dt, hipLaunchKernelGGL(sink_attention_rows_kernel<T>, dim3(rows, G * chunks),
                                        dim3(TILE), lds, s, (const T*)q, q_row, q_head,
                                        (const T*)k_cache, (const T*)v_cache,
                                        (const int*)block_tables, max_blocks, block_size,
                                        (const int*)row_seq, (const int*)lens, len_add,
                                        (const float*)sink, (const T*)gate, gate_row, (T*)out,
                                        scale, H, G, D, E, vec_ok));
    return HYB_LAUNCH_OK();
}

}  // extern "C"
