// Tail-biting Viterbi search of the trellis-3INST quantizer on the GPU
// (bitshift_codebook.viterbi / quantize, glq/trellis.py:253-296, 467-484;
// _viterbi_acs_step, glq/trellis_step_kernel.py:30-109).
//
// A tile is a sequence of T = 256 values; the trellis has 2^16 states, a step shifts K new
// bits in (state' = (state << K | b) & 0xFFFF) and costs (lut[state'] - x)^2.  With
// G = 2^(16-K), the predecessors of state' are the 2^K states k*G + (state' >> K), so only
//     best_i[g] = min_k ( err_{i-1}[k*G + g] + best_{i-1}[(k*G + g) >> K] ),  lowest k on ties,
// has to be carried from step to step (G floats, double-buffered in LDS); the arg-min k per
// (step, g) goes to a scratch slab in global memory for the backtrack.  The search runs twice
// (glq/trellis.py:479-482): on the sequence rolled by T/2 without constraints, then on the
// sequence itself with first and last state tied to the overlap the first pass found.
// All arithmetic is fp32 with separate subtract, multiply and add (no contraction), the
// input is rounded to fp16 first (glq/trellis.py:468), lut = decode_3inst computed on the fly.
//
// One workgroup (16 waves) per tile at a time; workgroups are persistent and walk the tiles
// with a fixed stride, each owning one scratch slab.  At K = 1 the two buffers of G = 32768
// floats do not fit the LDS together: the new costs of a step go through a slab of global
// scratch (each thread reads back what it wrote itself) into the one LDS buffer once every
// thread has finished reading the old ones.
#include "common.h"
#include "trellis_device.h"

#pragma clang fp contract(off)

namespace {

constexpr int VT_THREADS = 1024;
constexpr int VT_T = 256;

struct vt_best {
    float cost;
    int state;
};

// One pass.  x: T inputs in LDS; best: 2*G floats in LDS; from_k: T*G bytes of scratch;
// overlap < 0: unconstrained.  Returns, in `states` (LDS, T ints), the best state sequence.
template <int K>
__device__ __forceinline__ void viterbi_pass(const float *x, float *best, uint8_t *__restrict__ from_k,
                                             float *__restrict__ spill, int overlap, int *states,
                                             vt_best *red) {
    constexpr int G = 1 << (16 - K);
    constexpr int NK = 1 << K;
    constexpr int PER = G / VT_THREADS;                       // groups per thread
    const float inf = __builtin_inff();
    constexpr bool ONE_BUF = K == 1;
    float *cur = best, *nxt = ONE_BUF ? spill : best + G;
    for (int g = threadIdx.x; g < G; g += VT_THREADS) cur[g] = (overlap < 0 || g == overlap) ? 0.0f : inf;
    __syncthreads();
    for (int i = 1; i < VT_T; ++i) {
        const float xi = x[i - 1];
#pragma unroll 1
        for (int u = 0; u < PER; ++u) {
            const int g = threadIdx.x + u * VT_THREADS;
            float bc = 0.0f;
            int bk = 0;
#pragma unroll
            for (int k = 0; k < NK; ++k) {
                const int s = k * G + g;
                const float d = (float)tr_weight((uint32_t)s) - xi;
                const float e = d * d;
                const float c = e + cur[s >> K];
                if (k == 0 || c < bc) { bc = c; bk = k; }
            }
            nxt[g] = bc;
            from_k[(int64_t)i * G + g] = (uint8_t)bk;
        }
        __syncthreads();
        if constexpr (ONE_BUF) {
#pragma unroll 4
            for (int u = 0; u < PER; ++u) cur[threadIdx.x + u * VT_THREADS] = nxt[threadIdx.x + u * VT_THREADS];
            __syncthreads();
        } else {
            float *t = cur; cur = nxt; nxt = t;
        }
    }
    // final costs, with the tail-biting mask on the low 16-K bits; lowest state on ties
    {
        const float xi = x[VT_T - 1];
        float bc = inf;
        int bs = 0x7fffffff;
#pragma unroll 1
        for (int u = 0; u < PER; ++u) {
            const int g = threadIdx.x + u * VT_THREADS;
#pragma unroll
            for (int k = 0; k < NK; ++k) {
                const int s = k * G + g;
                const float d = (float)tr_weight((uint32_t)s) - xi;
                const float e = d * d;
                float c = e + cur[s >> K];
                if (overlap >= 0 && g != overlap) c = inf;
                if (c < bc || (c == bc && s < bs)) { bc = c; bs = s; }
            }
        }
        // wave, then workgroup reduction of (cost, state)
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float oc = __shfl_xor(bc, o, GLQH_WAVE);
            const int os = __shfl_xor(bs, o, GLQH_WAVE);
            if (oc < bc || (oc == bc && os < bs)) { bc = oc; bs = os; }
        }
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = vt_best{bc, bs};
        __syncthreads();
        if (threadIdx.x == 0) {
            vt_best b = red[0];
            for (int w = 1; w < VT_THREADS / 64; ++w)
                if (red[w].cost < b.cost || (red[w].cost == b.cost && red[w].state < b.state)) b = red[w];
            // every state is infinite only if the constraint is unsatisfiable, which the
            // first pass rules out; argmin of an all-inf row is state 0 in the reference
            int s = b.state == 0x7fffffff ? 0 : b.state;
            states[VT_T - 1] = s;
            for (int i = VT_T - 1; i > 0; --i) {              // backtrack
                const int g = s >> K;
                const uint8_t kk = __hip_atomic_load(from_k + (int64_t)i * G + g, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT);   // written by other waves
                s = g + ((int)kk << (16 - K));
                states[i - 1] = s;
            }
        }
        __syncthreads();
    }
}

template <int K>
__global__ void __launch_bounds__(VT_THREADS)
viterbi_kernel(const float *__restrict__ tiles, int64_t n_tiles, uint8_t *__restrict__ scratch,
               int32_t *__restrict__ states_out, float *__restrict__ hat_out) {
    constexpr int G = 1 << (16 - K);
    extern __shared__ float best[];                            // 2 * G floats (G at K = 1)
    __shared__ float x[VT_T], xr[VT_T];
    __shared__ int states[VT_T];
    __shared__ vt_best red[VT_THREADS / 64];
    uint8_t *from_k = scratch + (int64_t)blockIdx.x * VT_T * G;
    // K = 1: the spill slabs follow the back-pointer slabs of all workgroups
    float *spill = K == 1 ? (float *)(scratch + (int64_t)gridDim.x * VT_T * G) + (int64_t)blockIdx.x * G : nullptr;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        if (threadIdx.x < VT_T) {
            const float v = (float)(f16)tiles[tile * VT_T + threadIdx.x];
            x[threadIdx.x] = v;
            xr[(threadIdx.x + VT_T / 2) & (VT_T - 1)] = v;    // np.roll(x, T/2)
        }
        __syncthreads();
        viterbi_pass<K>(xr, best, from_k, spill, -1, states, red);
        const int overlap = states[VT_T / 2] >> K;
        __syncthreads();
        viterbi_pass<K>(x, best, from_k, spill, overlap, states, red);
        if (threadIdx.x < VT_T) {
            const int s = states[threadIdx.x];
            states_out[tile * VT_T + threadIdx.x] = s;
            hat_out[tile * VT_T + threadIdx.x] = (float)tr_weight((uint32_t)s);
        }
        __syncthreads();
    }
}

// states (tiles in row-major tile order, 256 steps each) -> packed kernel layout: the chunk of
// stream lane l is the top K bits of states 8l..8l+7, first state in the most significant
// position, stored little-endian (glq/trellis.py:486-523, 580-619).  One thread per chunk.
__global__ void __launch_bounds__(256)
pack_states_kernel(const int32_t *__restrict__ states, int m, int n, int K, uint8_t *__restrict__ packed) {
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t nblocks = (int64_t)(m >> 5) * (n >> 5);
    if (id >= nblocks * 128) return;
    const int c = (int)(id & 3), l = (int)((id >> 2) & 31);
    const int64_t blk = id >> 7;
    const int kpairs = n >> 5;
    const int mp = (int)(blk / kpairs), kp = (int)(blk % kpairs);
    const int tm = 2 * mp + (c & 1), tn = 2 * kp + (c >> 1);
    const int32_t *st = states + ((int64_t)tm * (n >> 4) + tn) * 256 + 8 * l;
    uint32_t chunk = 0;
    for (int j = 0; j < 8; ++j) chunk |= (((uint32_t)st[j] & 0xFFFFu) >> (16 - K)) << (K * (7 - j));
    uint8_t *dst = packed + (blk * 32 + l) * (4 * K) + c * K;
    for (int b = 0; b < K; ++b) dst[b] = (uint8_t)(chunk >> (8 * b));
}

// One add-compare-select step over cost rows that live in memory, for callers that drive the
// search step by step (bitshift_codebook.update, glq/trellis.py:230-251; its one-kernel form
// _viterbi_acs_step, glq/trellis_step_kernel.py:30-84).  V = 1, 2^16 states, NK = 2^K
// candidates: group j takes the minimum of cost[b, k*G + j] over ascending k (strict <, a NaN
// displaces a number and is never displaced), stores the predecessor j + (k << (16-K)) and
// the NK new costs (lut[s] - x[b])^2 + best of states s = j*NK .. j*NK + NK-1.  One thread per
// group: its loads are coalesced across the wave for every k, its stores are NK consecutive
// floats.  Streams 2 * B * 2^16 floats; bound by HBM.
template <int K>
__global__ void __launch_bounds__(256)
viterbi_acs_step_kernel(const float *__restrict__ cost, const f16 *__restrict__ x,
                        const float *__restrict__ lut, float *__restrict__ cost_out,
                        int32_t *__restrict__ prev) {
    constexpr int G = 1 << (16 - K);
    constexpr int NK = 1 << K;
    const int j = blockIdx.x * 256 + threadIdx.x;             // G is a multiple of 256
    const int b = blockIdx.y;
    const float *row = cost + (int64_t)b * 65536;
    float v[NK];
#pragma unroll
    for (int k = 0; k < NK; ++k) v[k] = row[k * G + j];
    float best = __builtin_inff();
    int bestk = 0;
#pragma unroll
    for (int k = 0; k < NK; ++k) {
        const bool take = (v[k] < best) || ((v[k] != v[k]) && (best == best));
        best = take ? v[k] : best;
        bestk = take ? k : bestk;
    }
    prev[(int64_t)b * G + j] = j + (bestk << (16 - K));
    const float xb = (float)x[b];
    float *o = cost_out + (int64_t)b * 65536 + (int64_t)j * NK;
    const float *l = lut + (int64_t)j * NK;
    if constexpr (NK >= 4) {
#pragma unroll
        for (int r = 0; r < NK; r += 4) {
            const f32x4 lv = *(const f32x4 *)(l + r);
            f32x4 e;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float d = lv[c] - xb;
                e[c] = d * d + best;                          // contraction is off in this file
            }
            *(f32x4 *)(o + r) = e;
        }
    } else {
        const f32x2 lv = *(const f32x2 *)l;
        f32x2 e;
        for (int c = 0; c < 2; ++c) {
            const float d = lv[c] - xb;
            e[c] = d * d + best;
        }
        *(f32x2 *)o = e;
    }
}

template <int K>
int acs_launch(const float *cost, const void *x, const float *lut, float *cost_out, int32_t *prev, int64_t B,
               hipStream_t stream) {
    hipLaunchKernelGGL(viterbi_acs_step_kernel<K>, dim3((1u << (16 - K)) / 256, (unsigned)B), dim3(256), 0, stream,
                       cost, (const f16 *)x, lut, cost_out, prev);
    GLQH_LAUNCH_CHECK("viterbi step launch");
    return 0;
}

template <int K>
int vt_launch(const float *tiles, int64_t n_tiles, uint8_t *scratch, int grid, int32_t *states, float *hat,
              hipStream_t stream) {
    constexpr size_t lds = (K == 1 ? 1 : 2) * sizeof(float) * ((size_t)1 << (16 - K));
    hipLaunchKernelGGL(viterbi_kernel<K>, dim3((unsigned)grid), dim3(VT_THREADS), lds, stream, tiles, n_tiles,
                       scratch, states, hat);
    GLQH_LAUNCH_CHECK("viterbi launch");
    return 0;
}

template <typename Kn>
int vt_set_lds(Kn kernel, size_t bytes) {
    return glqh_check_hip(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                              (int)bytes),
                          "viterbi attribute");
}

}  // namespace

int glqh_viterbi_init(void) {
    return vt_set_lds(viterbi_kernel<1>, 4 * 32768) || vt_set_lds(viterbi_kernel<2>, 2 * 4 * 16384) || vt_set_lds(viterbi_kernel<3>, 2 * 4 * 8192) ||
           vt_set_lds(viterbi_kernel<4>, 2 * 4 * 4096);
}

// persistent workgroups: one per CU (K = 2 fills the LDS of a CU), two for K >= 3
int glqh_viterbi_grid(int K, int64_t n_tiles) {
    int64_t g = (int64_t)glqh_device_cus() * (K >= 3 ? 2 : 1);
    return (int)(n_tiles < g ? n_tiles : g);
}

size_t glqh_viterbi_scratch_bytes(int K, int64_t n_tiles) {
    const size_t G = (size_t)1 << (16 - K);
    return (size_t)glqh_viterbi_grid(K, n_tiles) * (VT_T * G + (K == 1 ? G * sizeof(float) : 0));
}

int glqh_launch_viterbi(const float *tiles, int64_t n_tiles, int K, uint8_t *scratch, int32_t *states,
                        float *hat, hipStream_t stream) {
    const int grid = glqh_viterbi_grid(K, n_tiles);
    switch (K) {
    case 1: return vt_launch<1>(tiles, n_tiles, scratch, grid, states, hat, stream);
    case 2: return vt_launch<2>(tiles, n_tiles, scratch, grid, states, hat, stream);
    case 3: return vt_launch<3>(tiles, n_tiles, scratch, grid, states, hat, stream);
    case 4: return vt_launch<4>(tiles, n_tiles, scratch, grid, states, hat, stream);
    }
    return glqh_fail("trellis encoder supports K (bits/weight) 1-4, got %d", K);
}

int glqh_launch_pack_states(const int32_t *states, int64_t m, int64_t n, int K, void *packed, hipStream_t stream) {
    const int64_t threads = (m / 32) * (n / 32) * 128;
    hipLaunchKernelGGL(pack_states_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, states,
                       (int)m, (int)n, K, (uint8_t *)packed);
    GLQH_LAUNCH_CHECK("pack states launch");
    return 0;
}

int glqh_launch_viterbi_acs_step(const float *cost, const void *x_f16, const float *lut, float *cost_out,
                                 int32_t *prev, int64_t B, int K, hipStream_t stream) {
    switch (K) {
    case 1: return acs_launch<1>(cost, x_f16, lut, cost_out, prev, B, stream);
    case 2: return acs_launch<2>(cost, x_f16, lut, cost_out, prev, B, stream);
    case 3: return acs_launch<3>(cost, x_f16, lut, cost_out, prev, B, stream);
    case 4: return acs_launch<4>(cost, x_f16, lut, cost_out, prev, B, stream);
    }
    return glqh_fail("viterbi step supports K (bits/weight) 1-4, got %d", K);
}
