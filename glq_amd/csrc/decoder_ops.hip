// Glue kernels of the batch-1 decode loop around the quantized linears (RMSNorm, rotary
// embedding + KV-cache append, single-query grouped-query attention, SiLU gate).  They keep
// the end-to-end decode measurement from being dominated by dozens of tiny framework kernels
// per layer; arithmetic follows the usual Llama-family definitions in fp32 with bf16 storage.
#include <type_traits>

#include "common.h"
#include "fht_device.h"

namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, GLQH_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, GLQH_WAVE));
    return v;
}

// out[t] = bf16( bf16(x[t] * rsqrt(mean(x[t]^2) + eps)) * w ), one workgroup per token
__global__ void __launch_bounds__(256)
rmsnorm_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ w, uint16_t *__restrict__ out,
               int H, float eps) {
    __shared__ float red[4];
    const uint16_t *xr = x + (int64_t)blockIdx.x * H;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < H; i += 256) {
        const float v = bf16_bits_to_f32(xr[i]);
        ss += v * v;
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float r = rsqrtf((red[0] + red[1] + red[2] + red[3]) / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += 256) {
        const float n = bf16_bits_to_f32(f32_to_bf16_bits(bf16_bits_to_f32(xr[i]) * r));
        out[(int64_t)blockIdx.x * H + i] = f32_to_bf16_bits(n * bf16_bits_to_f32(w[i]));
    }
}

// Rotate q and k (pairs (i, i + D/2), angle row pos[t]) and append k, v to the caches.
// grid = (T, heads + 2*kv_heads); block = D/2 threads.
__global__ void rope_kv_store_kernel(const uint16_t *__restrict__ q, const uint16_t *__restrict__ k,
                                     const uint16_t *__restrict__ v, const int64_t *__restrict__ pos,
                                     const uint16_t *__restrict__ cos_t, const uint16_t *__restrict__ sin_t,
                                     uint16_t *__restrict__ q_out, uint16_t *__restrict__ kc,
                                     uint16_t *__restrict__ vc, int heads, int kv_heads, int D, int max_len,
                                     int apply_rope) {
    const int t = blockIdx.x, h = blockIdx.y, i = threadIdx.x, half = D >> 1;
    const int64_t p = pos[t];
    if (p < 0 || p >= max_len) return;             // position outside the cache: this token writes nothing
    const uint16_t *src;
    uint16_t *dst;
    bool rot = apply_rope != 0;
    if (h < heads) {
        src = q + ((int64_t)t * heads + h) * D;
        dst = q_out + ((int64_t)t * heads + h) * D;
    } else if (h < heads + kv_heads) {
        src = k + ((int64_t)t * kv_heads + (h - heads)) * D;
        dst = kc + ((int64_t)(h - heads) * max_len + p) * D;
    } else {
        src = v + ((int64_t)t * kv_heads + (h - heads - kv_heads)) * D;
        dst = vc + ((int64_t)(h - heads - kv_heads) * max_len + p) * D;
        rot = false;
    }
    const float a = bf16_bits_to_f32(src[i]), b = bf16_bits_to_f32(src[i + half]);
    if (!rot) {
        dst[i] = src[i];
        dst[i + half] = src[i + half];
        return;
    }
    const float c0 = bf16_bits_to_f32(cos_t[p * D + i]), s0 = bf16_bits_to_f32(sin_t[p * D + i]);
    const float c1 = bf16_bits_to_f32(cos_t[p * D + i + half]), s1 = bf16_bits_to_f32(sin_t[p * D + i + half]);
    dst[i] = f32_to_bf16_bits(a * c0 - b * s0);
    dst[i + half] = f32_to_bf16_bits(b * c1 + a * s1);
}

// One query token: out[h] = softmax(q[h] . K[g][0..pos] / sqrt(D)) V[g][0..pos], g = h / (heads/kv_heads).
// One workgroup of 16 waves per head; D = 128; scores live in LDS (max_len floats).
// Scores: 8 lanes per key with 16-byte loads, four keys per thread in flight.  Output: 16
// lanes per row of V with 16-byte loads, four rows in flight per thread; the waves' partial rows
// are summed through LDS in wave order.
constexpr int AT_THREADS = 1024;
constexpr int AT_WAVES = AT_THREADS / 64;

// The attention of one head once its scaled query sits in qs (LDS, D floats): scores over
// keys 0..n-1, softmax, weighted rows of V, result to out (D bf16).  NEWROW: row n-1 of K and V
// is not read from the cache but from knew / vnew (LDS, D bf16 each) -- the caller has just
// produced it and another workgroup is writing it to the cache at the same time.
// four keys of a thread's round (keys j0 + u * AT_THREADS / 8; 8 lanes per key, 16 + 16 bytes each)
struct attn_kregs {
    u32x4 k0[4], k1[4];
};

__device__ __forceinline__ attn_kregs attn_load_k(const uint16_t *__restrict__ K, int j0, int last) {
    constexpr int D = 128;
    const int sub = threadIdx.x & 7;
    attn_kregs r;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int j = min(j0 + u * (AT_THREADS / 8), last);
        r.k0[u] = *(const u32x4 *)(K + (int64_t)j * D + sub * 8);
        r.k1[u] = *(const u32x4 *)(K + (int64_t)j * D + 64 + sub * 8);
    }
    return r;
}

// four rows of V of a thread's round (rows j0 + u * 4 * AT_WAVES; 16 lanes per row, 16 bytes each)
struct attn_vregs {
    u32x4 v[4];
};

__device__ __forceinline__ attn_vregs attn_load_v(const uint16_t *__restrict__ V, int j0, int last) {
    constexpr int D = 128;
    const int vcol = threadIdx.x & 15;
    attn_vregs r;
#pragma unroll
    for (int u = 0; u < 4; ++u) r.v[u] = *(const u32x4 *)(V + (int64_t)min(j0 + u * 4 * AT_WAVES, last) * D + 8 * vcol);
    return r;
}

// FIRST: `first_k` holds the thread's first round of keys, which the caller has requested already
// (attn_load_k(K, j_lo + threadIdx.x >> 3, last) with last as computed here).
// Keys j_lo .. j_hi - 1 of the n: the whole row (0, n) or one workgroup's share of it.  With `pbuf` the share's
// running maximum, sum of exponentials and unnormalised weighted rows go there (2 + D floats, written past the
// L2 of this XCD for the workgroup that merges the shares) instead of the finished row to `out`.
constexpr int AT_PART = 2 + 128;

template <bool NEWROW, bool FIRST = false>
__device__ __forceinline__ void attn_core(const float *qs, const uint16_t *__restrict__ K,
                                          const uint16_t *__restrict__ V, int n, const uint16_t *knew,
                                          const uint16_t *vnew, float *sc, float *red,
                                          float (*part)[128], uint16_t *__restrict__ out,
                                          const attn_kregs first_k = {}, int j_lo = 0, int j_hi = -1,
                                          float *pbuf = nullptr) {
    constexpr int D = 128;
    if (j_hi < 0) j_hi = n;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // last row that is read from the cache (row n - 1 comes from knew / vnew when NEWROW)
    const int last = NEWROW && j_hi == n ? max(n - 2, 0) : j_hi - 1;
    const int sub = threadIdx.x & 7;
    float mx = -3.0e38f;
    // four keys per thread in flight (512 keys per round of the workgroup)
    for (int j0 = j_lo + (threadIdx.x >> 3); j0 < j_hi; j0 += 4 * (AT_THREADS / 8)) {
        attn_kregs kr;
        if (FIRST && j0 == j_lo + (int)(threadIdx.x >> 3)) kr = first_k;
        else kr = attn_load_k(K, j0, last);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int j = j0 + u * (AT_THREADS / 8);
            u32x4 k0 = kr.k0[u], k1 = kr.k1[u];
            if (NEWROW && j == n - 1) {
                k0 = *(const u32x4 *)(knew + sub * 8);
                k1 = *(const u32x4 *)(knew + 64 + sub * 8);
            }
            float s = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t w0 = k0[e], w1 = k1[e];
                s += qs[sub * 8 + 2 * e] * bf16_bits_to_f32((uint16_t)(w0 & 0xFFFFu));
                s += qs[sub * 8 + 2 * e + 1] * bf16_bits_to_f32((uint16_t)(w0 >> 16));
                s += qs[64 + sub * 8 + 2 * e] * bf16_bits_to_f32((uint16_t)(w1 & 0xFFFFu));
                s += qs[64 + sub * 8 + 2 * e + 1] * bf16_bits_to_f32((uint16_t)(w1 >> 16));
            }
            s += __shfl_xor(s, 1, GLQH_WAVE);
            s += __shfl_xor(s, 2, GLQH_WAVE);
            s += __shfl_xor(s, 4, GLQH_WAVE);
            if (j < j_hi) {
                if (sub == 0) sc[j - j_lo] = s;
                mx = fmaxf(mx, s);
            }
        }
    }
    // weighted rows of V: 16 lanes per row (8 columns, one 16-byte load each), 4 rows per wave
    // per load and four loads in flight: 256 keys per round of the workgroup.  The first round
    // is requested here, ahead of the softmax, every later one a round ahead of its use.
    const int vr = lane >> 4, vcol = lane & 15;
    const int vj0 = j_lo + wave * 4 + vr;
    attn_vregs vcur = attn_load_v(V, vj0, last);
    mx = wave_max(mx);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = red[0];
#pragma unroll
    for (int w = 1; w < AT_WAVES; ++w) mx = fmaxf(mx, red[w]);
    __syncthreads();
    float sum = 0.0f;
    for (int j = threadIdx.x; j < j_hi - j_lo; j += AT_THREADS) {
        const float e = __expf(sc[j] - mx);
        sc[j] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int w = 0; w < AT_WAVES; ++w) tot += red[w];
    float a[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) a[e] = 0.0f;
    for (int j0 = vj0; j0 < j_hi; j0 += 4 * 4 * AT_WAVES) {
        attn_vregs vnext = vcur;
        if (j0 + 4 * 4 * AT_WAVES < j_hi) vnext = attn_load_v(V, j0 + 4 * 4 * AT_WAVES, last);
        float pw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int j = j0 + u * 4 * AT_WAVES;
            if (NEWROW && j == n - 1) vcur.v[u] = *(const u32x4 *)(vnew + 8 * vcol);
            pw[u] = j < j_hi ? sc[j - j_lo] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t w = vcur.v[u][e];
                a[2 * e] += pw[u] * bf16_bits_to_f32((uint16_t)(w & 0xFFFFu));
                a[2 * e + 1] += pw[u] * bf16_bits_to_f32((uint16_t)(w >> 16));
            }
        vcur = vnext;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {                               // the wave's four row lanes
        a[e] += __shfl_xor(a[e], 16, GLQH_WAVE);
        a[e] += __shfl_xor(a[e], 32, GLQH_WAVE);
    }
    if (vr == 0) {
#pragma unroll
        for (int e = 0; e < 8; ++e) part[wave][8 * vcol + e] = a[e];
    }
    __syncthreads();
    if (threadIdx.x < D) {
        float acc = 0.0f;
#pragma unroll
        for (int w = 0; w < AT_WAVES; ++w) acc += part[w][threadIdx.x];
        if (pbuf) {
            __hip_atomic_store(pbuf + 2 + threadIdx.x, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (threadIdx.x == 0) {
                __hip_atomic_store(pbuf, mx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(pbuf + 1, tot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        } else {
            out[threadIdx.x] = f32_to_bf16_bits(acc / tot);
        }
    }
}

// The shares of one head, ns of them, merged by the workgroup that finishes last: every workgroup waits until
// its own share has left, then adds one to the head's counter; the one that brings it to ns resets it (the
// state is all zeros again when the launch ends), reads the shares past its L2 and writes the row:
//   out = sum_s e^(m_s - M) acc_s / sum_s e^(m_s - M) l_s,  M = max_s m_s, shares in ascending order.
// Nobody waits for anybody: a workgroup that is not the last simply ends.
__device__ __forceinline__ void attn_merge_shares(float *hbuf, unsigned int *cnt, int ns, uint16_t *__restrict__ out,
                                                  int *flag) {
    constexpr int D = 128;
    __builtin_amdgcn_s_waitcnt(0);                               // this wave's share has left
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned int before = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int lastone = before + 1u == (unsigned int)ns;
        if (lastone) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = lastone;
    }
    __syncthreads();
    if (!*flag || threadIdx.x >= D) return;
    float M = -3.0e38f;
    for (int s = 0; s < ns; ++s)
        M = fmaxf(M, __hip_atomic_load(hbuf + s * AT_PART, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    float L = 0.0f, o = 0.0f;
    for (int s = 0; s < ns; ++s) {
        const float *pb = hbuf + s * AT_PART;
        const float w = __expf(__hip_atomic_load(pb, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - M);
        L += w * __hip_atomic_load(pb + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        o += w * __hip_atomic_load(pb + 2 + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    out[threadIdx.x] = f32_to_bf16_bits(o / L);
}

__global__ void __launch_bounds__(AT_THREADS)
attn_decode_kernel(const uint16_t *__restrict__ q, const uint16_t *__restrict__ kc,
                   const uint16_t *__restrict__ vc, const int64_t *__restrict__ pos_ptr,
                   uint16_t *__restrict__ out, int heads, int kv_heads, int max_len, float scale) {
    constexpr int D = 128;
    extern __shared__ float sc[];                  // max_len scores
    __shared__ float qs[D];
    __shared__ float red[AT_WAVES];
    __shared__ float part[AT_WAVES][D];
    const int h = blockIdx.x, g = h / (heads / kv_heads);
    const int64_t p = pos_ptr[0];
    if (p < 0 || p >= max_len) return;             // position outside the cache (sc holds max_len scores)
    const int n = (int)p + 1;                      // keys 0..pos (the current token is already cached)
    if (threadIdx.x < D) qs[threadIdx.x] = bf16_bits_to_f32(q[(int64_t)h * D + threadIdx.x]) * scale;
    __syncthreads();
    attn_core<false>(qs, kc + (int64_t)g * max_len * D, vc + (int64_t)g * max_len * D, n, nullptr, nullptr, sc, red,
                     part, out + (int64_t)h * D);
}

// x_out = bf16(x + delta); h_out = RMSNorm(x_out) * w as in rmsnorm_kernel (one pass, one launch)
__global__ void __launch_bounds__(256)
add_rmsnorm_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ delta,
                   const uint16_t *__restrict__ w, uint16_t *__restrict__ x_out, uint16_t *__restrict__ h_out,
                   int H, float eps) {
    __shared__ float red[4];
    extern __shared__ float row[];                 // H floats
    const int64_t base = (int64_t)blockIdx.x * H;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < H; i += 256) {
        const uint16_t sb = f32_to_bf16_bits(bf16_bits_to_f32(x[base + i]) + bf16_bits_to_f32(delta[base + i]));
        x_out[base + i] = sb;
        const float v = bf16_bits_to_f32(sb);
        row[i] = v;
        ss += v * v;
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float r = rsqrtf((red[0] + red[1] + red[2] + red[3]) / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += 256) {
        const float nrm = bf16_bits_to_f32(f32_to_bf16_bits(row[i] * r));
        h_out[base + i] = f32_to_bf16_bits(nrm * bf16_bits_to_f32(w[i]));
    }
}

// out = bf16( bf16(silu(g)) * u )
__global__ void __launch_bounds__(256)
silu_mul_kernel(const uint16_t *__restrict__ g, const uint16_t *__restrict__ u, uint16_t *__restrict__ out,
                int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float a = bf16_bits_to_f32(g[i]);
    const float s = bf16_bits_to_f32(f32_to_bf16_bits(a / (1.0f + __expf(-a))));
    out[i] = f32_to_bf16_bits(s * bf16_bits_to_f32(u[i]));
}

// ---- output transform fused with what follows it in the decode loop (one token) --------
// o_proj / down_proj: split-K partial sums -> output transform -> x_out = bf16(resid + bf16(y))
// -> h_out = RMSNorm(x_out) * w, with the terms, order and roundings of
// output_rht_group_kernel + add_rmsnorm_kernel.  One workgroup, the row is 2-8 K values: a
// Hadamard block is cut into the same 1024-point slices, one per group of 256 threads, but
// every group sums the split-K terms of its own 1024 rows only and the groups then combine
// each other's sums through LDS (the separate launch re-reads the whole block per slice).
constexpr int FN_THREADS = 1024;
constexpr int FN_GROUPS = FN_THREADS / 256;
constexpr int FN_LOG_SLICE = 10;
constexpr int FN_MAX_ROWS = 8192;

__global__ void __launch_bounds__(FN_THREADS)
out_add_rmsnorm_kernel(const float *__restrict__ part, int ksplit, float scale, const f16 *__restrict__ su,
                       int m, const uint16_t *__restrict__ resid, const uint16_t *__restrict__ w, float eps,
                       uint16_t *__restrict__ x_out, uint16_t *__restrict__ h_out) {
    // FN_GROUPS exchange buffers and FN_GROUPS sum buffers of one slice each, then m floats: the row
    extern __shared__ float s[];
    __shared__ float red[FN_THREADS / 64];
    const int grp = threadIdx.x >> 8, gt = threadIdx.x & 255;
    float *xchg = s + (grp << FN_LOG_SLICE);
    float *sums = s + (FN_GROUPS << FN_LOG_SLICE);
    float *row = s + (2 * FN_GROUPS << FN_LOG_SLICE);
    glqh_ysrc src = {};
    src.part = part;
    src.part_kstride = m;
    src.ksplit = ksplit;
    src.scale[0] = scale;
    src.nparts = 1;
    glqh_meta_args margs;
    margs.canon = m;
    const int nb = __builtin_popcount((unsigned)m);
    uint16_t w_raw[FN_MAX_ROWS / FN_THREADS];                // the norm weights of the last loop, requested first
#pragma unroll
    for (int u = 0; u < FN_MAX_ROWS / FN_THREADS; ++u) w_raw[u] = w[min((int)threadIdx.x + u * FN_THREADS, m - 1)];
    for (int j = 0; j < nb; ++j) {
        const glqh_block_meta bm = glqh_meta_row(margs, nullptr, j);
        const int log_len = min(bm.log_bs, FN_LOG_SLICE);
        const int nsub = bm.bs >> log_len;                   // <= FN_GROUPS (checked by the launcher)
        const bool mine = grp < nsub, live = mine && 4 * gt < (1 << log_len);
        const int base = bm.offset + (grp << log_len);       // this group's rows: slice grp of the block
        const float norm = rsqrt_pow2(bm.log_bs);
        float z[4];
        f16 su_raw[4];                                       // requested before the partial sums and
        uint16_t rs_raw[4];                                  // not touched until those have arrived
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int r = base + fht_wave_index<4>(log_len, live ? gt : 0, q);
            su_raw[q] = su[mine ? r : 0];
            rs_raw[q] = resid[mine ? r : 0];
        }
        if (mine) {
            // v_h for h = grp: the split-K terms of rows base .. base + len - 1, in slot order
            rht_slice own = {};
            own.off = base; own.bs = 1 << log_len; own.log_bs = own.log_len = log_len;
            own.nsub = 1; own.r = 0; own.live = true;
            float v[4];
            if (ksplit <= 8) stage_partials_quad<8>(v, src, own, 0, m, gt);
            else stage_partials_quad<12>(v, src, own, 0, m, gt);   // 24 terms in flight would spill registers
            if (live) *(f32x4 *)(sums + (grp << FN_LOG_SLICE) + 4 * gt) = f32x4{v[0], v[1], v[2], v[3]};
        }
        __syncthreads();
        // slice r = grp of the block: z = sum_h sign(r, h) v_h, h ascending
#pragma unroll
        for (int e = 0; e < 4; ++e) z[e] = 0.0f;
        if (live) {
            for (int h = 0; h < nsub; ++h) {
                const f32x4 vh = *(const f32x4 *)(sums + (h << FN_LOG_SLICE) + 4 * gt);
#pragma unroll
                for (int e = 0; e < 4; ++e) z[e] += had_sign(grp, h, vh[e]);
            }
        }
        fht_wave<4, true>(z, log_len, xchg, gt);
        if (live) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int r = base + fht_wave_index<4>(log_len, gt, q);
                const float y = bf16_bits_to_f32(f32_to_bf16_bits(z[q] * (norm * (float)su_raw[q])));
                const uint16_t sb = f32_to_bf16_bits(bf16_bits_to_f32(rs_raw[q]) + y);
                x_out[r] = sb;
                row[r] = bf16_bits_to_f32(sb);
            }
        }
        __syncthreads();                                     // row written, buffers free for the next block
    }
    float ss = 0.0f;
    for (int j = 0; j < nb; ++j) {
        const glqh_block_meta bm = glqh_meta_row(margs, nullptr, j);
        for (int i = threadIdx.x; i < bm.bs; i += FN_THREADS) {
            const float v = row[bm.offset + i];
            ss += v * v;
        }
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int i = 0; i < FN_THREADS / 64; ++i) tot += red[i];
    const float r = rsqrtf(tot / (float)m + eps);
#pragma unroll
    for (int u = 0; u < FN_MAX_ROWS / FN_THREADS; ++u) {
        const int i = threadIdx.x + u * FN_THREADS;
        if (i < m) {
            const float nrm = bf16_bits_to_f32(f32_to_bf16_bits(row[i] * r));
            h_out[i] = f32_to_bf16_bits(nrm * bf16_bits_to_f32(w_raw[u]));
        }
    }
}

// gate_proj / up_proj: both layers' partial sums -> the two output transforms, slice by slice
// as output_rht_group_kernel cuts them -> act = bf16(bf16(silu(bf16 gate)) * bf16 up), the
// roundings of output_rht_group_kernel + silu_mul_kernel (bit-identical to the two launches).
__global__ void __launch_bounds__(512)
out_silu_mul_kernel(const float *__restrict__ part_g, const float *__restrict__ part_u, int ksplit, float sc_g,
                    float sc_u, const f16 *__restrict__ su_g, const f16 *__restrict__ su_u, int m_pad,
                    int out_features, uint16_t *__restrict__ act, int spb, int log_slice, int buf_floats) {
    extern __shared__ float s[];                   // two transform buffers, then the gate values
    glqh_meta_args margs;
    margs.canon = m_pad;
    const rht_slice blk = rht_get_slice(nullptr, margs, 0.0f, spb, log_slice);
    if (!blk.live) return;
    const int len = 1 << blk.log_len;
    const int base = blk.off + (blk.r << blk.log_len);
    // threads 0..255 transform the gate slice, 256..511 the up slice, side by side
    const int layer = threadIdx.x >> 8, tid = threadIdx.x & 255;
    float *buf = s + layer * buf_floats;
    float *gv = s + 2 * buf_floats;
    glqh_ysrc src = {};
    src.part = layer ? part_u : part_g;
    src.part_kstride = m_pad;
    src.ksplit = ksplit;
    src.scale[0] = layer ? sc_u : sc_g;
    src.nparts = 1;
    const f16 *su = layer ? su_u : su_g;
    const bool live = 4 * tid < len;
    float z[4];
    f16 su_raw[4];                                 // requested before the partial sums, used after
    int idx[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) su_raw[q] = su[base + fht_wave_index<4>(blk.log_len, live ? tid : 0, q)];
    partials_fht_quad(z, idx, src, blk, 0, m_pad, buf, tid);
    float y[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        y[q] = bf16_bits_to_f32(f32_to_bf16_bits(z[q] * (blk.norm * (float)su_raw[q])));
        if (layer == 0 && live) gv[idx[q]] = y[q];
    }
    __syncthreads();
    if (layer == 1 && live) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int i = idx[q];
            if (base + i < out_features) {
                const float a = gv[i];
                const float sl = bf16_bits_to_f32(f32_to_bf16_bits(a / (1.0f + __expf(-a))));
                act[base + i] = f32_to_bf16_bits(sl * y[q]);
            }
        }
    }
}

// q_proj / k_proj / v_proj (blockIdx.y = layer): output transform slice by slice as
// output_rht_group_kernel cuts it, then what rope_kv_store_kernel does with the bf16 result:
// rotate q and k by the angle row of position *pos, q -> q_out, k and v -> cache row *pos.
// Slices are whole heads (len % D == 0).  Bit-identical to the two separate launches.
struct qkv_fin {
    const float *part[3];
    const f16 *su[3];
    float scale[3];
    int m[3];
};

__global__ void __launch_bounds__(256)
out_rope_store_kernel(qkv_fin a, int ksplit, const int64_t *__restrict__ pos, const uint16_t *__restrict__ cos_t,
                      const uint16_t *__restrict__ sin_t, uint16_t *__restrict__ q_out, uint16_t *__restrict__ kc,
                      uint16_t *__restrict__ vc, int D, int max_len, int apply_rope, int spb, int log_slice) {
    extern __shared__ float s[];
    const int z = blockIdx.y;
    const float *part = z == 0 ? a.part[0] : z == 1 ? a.part[1] : a.part[2];
    const f16 *su = z == 0 ? a.su[0] : z == 1 ? a.su[1] : a.su[2];
    const float scale = z == 0 ? a.scale[0] : z == 1 ? a.scale[1] : a.scale[2];
    const int m = z == 0 ? a.m[0] : z == 1 ? a.m[1] : a.m[2];
    if ((int)blockIdx.x >= __builtin_popcount((unsigned)m) * spb) return;
    glqh_meta_args margs;
    margs.canon = m;
    const rht_slice blk = rht_get_slice(nullptr, margs, 0.0f, spb, log_slice);
    if (!blk.live) return;
    glqh_ysrc src = {};
    src.part = part;
    src.part_kstride = m;
    src.ksplit = ksplit;
    src.scale[0] = scale;
    src.nparts = 1;
    const int len = 1 << blk.log_len, base = blk.off + (blk.r << blk.log_len), half = D >> 1;
    const int64_t p = *pos;
    if (p < 0 || p >= max_len) return;             // position outside the cache: nothing is written
    {
        const int tid = threadIdx.x;
        const bool live = 4 * tid < len;
        float zq[4];
        f16 su_raw[4];                             // requested before the partial sums, used after
        int idx[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) su_raw[q] = su[base + fht_wave_index<4>(blk.log_len, live ? tid : 0, q)];
        partials_fht_quad(zq, idx, src, blk, 0, m, s, tid);
        __syncthreads();                           // the exchange has been read: s takes the result
        // y rounded to bf16, as the separate output transform stores it
        if (live) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
                s[lds_pad(idx[q])] = bf16_bits_to_f32(f32_to_bf16_bits(zq[q] * (blk.norm * (float)su_raw[q])));
        }
        __syncthreads();
    }
    auto yv = [&](int i) { return s[lds_pad(i)]; };
    for (int e = threadIdx.x; e < len / 2; e += 256) {
        const int hl = e / half, d = e - hl * half;            // head inside the slice, column pair (d, d + half)
        const int i0 = hl * D + d, i1 = i0 + half;
        const int head = (base + i0) / D;
        const float va = yv(i0), vb = yv(i1);
        uint16_t *dst = z == 0 ? q_out + (int64_t)head * D
                      : (z == 1 ? kc : vc) + ((int64_t)head * max_len + p) * D;
        if (z == 2 || !apply_rope) {
            dst[d] = f32_to_bf16_bits(va);
            dst[d + half] = f32_to_bf16_bits(vb);
        } else {
            const float c0 = bf16_bits_to_f32(cos_t[p * D + d]), s0 = bf16_bits_to_f32(sin_t[p * D + d]);
            const float c1 = bf16_bits_to_f32(cos_t[p * D + d + half]), s1 = bf16_bits_to_f32(sin_t[p * D + d + half]);
            dst[d] = f32_to_bf16_bits(va * c0 - vb * s0);
            dst[d + half] = f32_to_bf16_bits(vb * c1 + va * s1);
        }
    }
}

// q_proj / k_proj / v_proj finished inside the attention launch: workgroup h (one per query
// head) transforms the 1024-point slice of q that holds its head and the slices of k and v that
// hold its key/value head -- three transforms side by side on thread groups of 512 / 256 / 256
// with shared barriers -- rotates q and k, and attends over cache rows 0..pos-1 plus the new
// row, which it keeps in LDS; the first query head of each group also appends the row to the
// caches.  Same slices, term order and roundings as out_rope_store_kernel + attn_decode_kernel:
// bit-identical to the two launches.
__device__ __forceinline__ rht_slice slice_of_row(int m, int row, int log_slice) {
    glqh_meta_args margs;
    margs.canon = m;
    const int nb = __builtin_popcount((unsigned)m);
    rht_slice blk = {};
    for (int j = 0; j < nb; ++j) {
        const glqh_block_meta bm = glqh_meta_row(margs, nullptr, j);
        if (row < bm.offset + bm.bs || j == nb - 1) {
            blk.off = bm.offset;
            blk.bs = bm.bs;
            blk.log_bs = bm.log_bs;
            blk.log_len = min(bm.log_bs, log_slice);
            blk.nsub = bm.bs >> blk.log_len;
            blk.r = (row - bm.offset) >> blk.log_len;
            blk.norm = rsqrt_pow2(bm.log_bs);
            blk.live = true;
            break;
        }
    }
    return blk;
}

template <bool SHARED>
__global__ void __launch_bounds__(AT_THREADS)
out_rope_attn_kernel(qkv_fin a, int ksplit, const int64_t *__restrict__ pos_ptr,
                     const uint16_t *__restrict__ cos_t, const uint16_t *__restrict__ sin_t,
                     uint16_t *__restrict__ kc, uint16_t *__restrict__ vc, uint16_t *__restrict__ out, int heads,
                     int kv_heads, int max_len, int apply_rope, float scale, int log_slice, int sc_floats,
                     int buf_floats, float *split_buf, unsigned int *split_cnt, int split_min) {
    constexpr int D = 128, half = D / 2;
    extern __shared__ float lds[];                 // scores, then the three transform buffers
    __shared__ float qs[D];
    __shared__ float red[AT_WAVES];
    __shared__ float part[AT_WAVES][D];
    __shared__ __align__(16) uint16_t knew[D], vnew[D];
    float *sc = lds;
    const int h = blockIdx.x, per = heads / kv_heads, g = h / per;
    const int64_t p = pos_ptr[0];
    if (p < 0 || p >= max_len) return;             // position outside the cache and the score buffer
    const int n = (int)p + 1;
    // gridDim.y workgroups per head share the keys once there are split_min of them for each: share s takes
    // keys [s * chunk, (s + 1) * chunk), the last one the new row as well; a head with one share is finished by
    // its workgroup alone, exactly as without shares
    int ns = 1, share = 0, j_lo = 0, j_hi = n;
    if constexpr (SHARED) {
        ns = min((int)gridDim.y, max(n / split_min, 1));
        share = blockIdx.y;
        if (share >= ns) return;                                // uniform over the workgroup
        const int chunk = (n + ns - 1) / ns;
        j_lo = share * chunk;
        j_hi = min(n, j_lo + chunk);
    }
    const int tid = threadIdx.x;
    const int grp = tid < 512 ? 0 : tid < 768 ? 1 : 2;         // q | k | v, whole waves each
    const int gt = grp == 0 ? tid : grp == 1 ? tid - 512 : tid - 768;
    const int m = grp == 0 ? a.m[0] : grp == 1 ? a.m[1] : a.m[2];
    const int row0 = (grp == 0 ? h : g) * D;
    const rht_slice blk = slice_of_row(m, row0, log_slice);
    float *buf = lds + sc_floats + grp * buf_floats;
    glqh_ysrc src = {};
    src.part = grp == 0 ? a.part[0] : grp == 1 ? a.part[1] : a.part[2];
    src.part_kstride = m;
    src.ksplit = ksplit;
    src.scale[0] = grp == 0 ? a.scale[0] : grp == 1 ? a.scale[1] : a.scale[2];
    src.nparts = 1;
    const f16 *su = grp == 0 ? a.su[0] : grp == 1 ? a.su[1] : a.su[2];
    // sign, cosine and sine values of the rotation step: requested now, used after the transform
    const int d = min(gt, half - 1);
    const f16 su_a = su[row0 + d], su_b = su[row0 + d + half];
    uint16_t cs[4] = {0, 0, 0, 0};
    if (grp != 2 && apply_rope) {
        cs[0] = cos_t[p * D + d]; cs[1] = sin_t[p * D + d];
        cs[2] = cos_t[p * D + d + half]; cs[3] = sin_t[p * D + d + half];
    }
    const uint16_t *Kh = kc + (int64_t)g * max_len * D, *Vh = vc + (int64_t)g * max_len * D;
    attn_kregs first_k;
    {
        // three transforms of possibly different sizes side by side: one shared barrier each
        float zq[4];
        int idx[4];
        const bool live = 4 * gt < (1 << blk.log_len);
#pragma unroll
        for (int q = 0; q < 4; ++q) idx[q] = fht_wave_index<4>(blk.log_len, live ? gt : 0, q);
        stage_partials_quad_n(zq, src, blk, 0, m, gt);
        // the first round of cached keys travels while the transform and the rotation run
        first_k = attn_load_k(Kh, j_lo + (tid >> 3), j_hi == n ? max(n - 2, 0) : j_hi - 1);
        // barriers that wait for LDS only: the key loads stay in flight across them
        fht_wave<4, true, true>(zq, blk.log_len, buf, gt);
        fht_barrier<true>();                       // the exchanges have been read: buf takes the result
        if (live) {
#pragma unroll
            for (int q = 0; q < 4; ++q) buf[lds_pad(idx[q])] = zq[q];
        }
    }
    fht_barrier<true>();
    if (gt < half) {
        const int li = row0 - (blk.off + (blk.r << blk.log_len));  // the head inside the slice
        const float va = bf16_bits_to_f32(f32_to_bf16_bits(buf[lds_pad(li + d)] * (blk.norm * (float)su_a)));
        const float vb = bf16_bits_to_f32(f32_to_bf16_bits(buf[lds_pad(li + d + half)] * (blk.norm * (float)su_b)));
        uint16_t o0 = f32_to_bf16_bits(va), o1 = f32_to_bf16_bits(vb);
        if (grp != 2 && apply_rope) {
            const float c0 = bf16_bits_to_f32(cs[0]), s0 = bf16_bits_to_f32(cs[1]);
            const float c1 = bf16_bits_to_f32(cs[2]), s1 = bf16_bits_to_f32(cs[3]);
            o0 = f32_to_bf16_bits(va * c0 - vb * s0);
            o1 = f32_to_bf16_bits(vb * c1 + va * s1);
        }
        if (grp == 0) {
            qs[d] = bf16_bits_to_f32(o0) * scale;
            qs[d + half] = bf16_bits_to_f32(o1) * scale;
        } else {
            uint16_t *nw = grp == 1 ? knew : vnew;
            nw[d] = o0;
            nw[d + half] = o1;
            if (h % per == 0 && share == 0) {                    // one writer per key/value head
                uint16_t *dst = (grp == 1 ? kc : vc) + ((int64_t)g * max_len + p) * D;
                dst[d] = o0;
                dst[d + half] = o1;
            }
        }
    }
    fht_barrier<true>();                           // qs, knew, vnew are in LDS
    if constexpr (!SHARED) {
        attn_core<true, true>(qs, Kh, Vh, n, knew, vnew, sc, red, part, out + (int64_t)h * D, first_k);
    } else {
        float *hbuf = split_buf + (int64_t)h * gridDim.y * AT_PART;
        attn_core<true, true>(qs, Kh, Vh, n, knew, vnew, sc, red, part, out + (int64_t)h * D, first_k, j_lo, j_hi,
                        ns > 1 ? hbuf + share * AT_PART : nullptr);
        if (ns > 1) attn_merge_shares(hbuf, split_cnt + h, ns, out + (int64_t)h * D, (int *)red);
    }
}

// Output head of the decode step: logits[r] = <h, E[r, :]> (bf16 x bf16, fp32 sums) over a
// (vocab, hidden) bf16 table, and the arg-max of the row.  A wave takes rows r, r + W, ...;
// every lane keeps its 8*HC activations in registers and reads HC 16-byte runs of each row, two
// rows at a time (2*HC loads in flight per lane).  Streams the table once: bound by HBM.
// Ties go to the lowest row.  best: [waves] (value, row) pairs for lm_head_argmax_kernel.
template <int HC>
__global__ void __launch_bounds__(256)
lm_head_kernel(const uint16_t *__restrict__ h, const uint16_t *__restrict__ E, float *__restrict__ logits,
               float *__restrict__ best_val, int *__restrict__ best_row, int vocab) {
    constexpr int hidden = 512 * HC;
    const int lane = threadIdx.x & 63;
    const int wid = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int nw = gridDim.x * 4;
    float x[HC][8];
#pragma unroll
    for (int c = 0; c < HC; ++c) {
        const u32x4 v = *(const u32x4 *)(h + 8 * (lane + 64 * c));
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            x[c][2 * e] = __builtin_bit_cast(float, v[e] << 16);
            x[c][2 * e + 1] = __builtin_bit_cast(float, v[e] & 0xFFFF0000u);
        }
    }
    float bv = -__builtin_inff();
    int br = 0x7FFFFFFF;
    for (int r0 = wid; r0 < vocab; r0 += 2 * nw) {
        const int r1 = r0 + nw;
        const int r1c = r1 < vocab ? r1 : r0;                    // clamped: the loads stay unconditional
        u32x4 a[HC], b[HC];
#pragma unroll
        for (int c = 0; c < HC; ++c) {
            a[c] = __builtin_nontemporal_load((const u32x4 *)(E + (int64_t)r0 * hidden + 8 * (lane + 64 * c)));
            b[c] = __builtin_nontemporal_load((const u32x4 *)(E + (int64_t)r1c * hidden + 8 * (lane + 64 * c)));
        }
        float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
        for (int c = 0; c < HC; ++c)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                s0 += x[c][2 * e] * __builtin_bit_cast(float, a[c][e] << 16);
                s0 += x[c][2 * e + 1] * __builtin_bit_cast(float, a[c][e] & 0xFFFF0000u);
                s1 += x[c][2 * e] * __builtin_bit_cast(float, b[c][e] << 16);
                s1 += x[c][2 * e + 1] * __builtin_bit_cast(float, b[c][e] & 0xFFFF0000u);
            }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            s0 += __shfl_xor(s0, d, GLQH_WAVE);
            s1 += __shfl_xor(s1, d, GLQH_WAVE);
        }
        if (lane == 0) {
            if (logits) {
                logits[r0] = s0;
                if (r1 < vocab) logits[r1] = s1;
            }
        }
        if (s0 > bv) { bv = s0; br = r0; }                       // rows ascend within a wave
        if (r1 < vocab && s1 > bv) { bv = s1; br = r1; }
    }
    if (lane == 0) {
        best_val[wid] = bv;
        best_row[wid] = br;
    }
}

__global__ void __launch_bounds__(256)
lm_head_argmax_kernel(const float *__restrict__ best_val, const int *__restrict__ best_row, int n,
                      int64_t *__restrict__ token) {
    __shared__ float sv[256];
    __shared__ int sr[256];
    float bv = -__builtin_inff();
    int br = 0x7FFFFFFF;
    for (int i = threadIdx.x; i < n; i += 256) {
        const float v = best_val[i];
        const int r = best_row[i];
        if (v > bv || (v == bv && r < br)) { bv = v; br = r; }
    }
    sv[threadIdx.x] = bv;
    sr[threadIdx.x] = br;
    __syncthreads();
    for (int d = 128; d >= 1; d >>= 1) {
        if ((int)threadIdx.x < d) {
            const float v = sv[threadIdx.x + d];
            const int r = sr[threadIdx.x + d];
            if (v > sv[threadIdx.x] || (v == sv[threadIdx.x] && r < sr[threadIdx.x])) {
                sv[threadIdx.x] = v;
                sr[threadIdx.x] = r;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) *token = sr[0];
}

}  // namespace

extern "C" int glqh_rmsnorm_bf16(const void *x, const void *w, void *out, int64_t T, int64_t H, double eps,
                                 void *stream) {
    GLQH_REQUIRE(x && w && out && T >= 1 && H >= 1, "rmsnorm: bad arguments");
    hipLaunchKernelGGL(rmsnorm_kernel, dim3((unsigned)T), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t *)x, (const uint16_t *)w, (uint16_t *)out, (int)H, (float)eps);
    GLQH_LAUNCH_CHECK("rmsnorm launch");
    return 0;
}

extern "C" int glqh_rope_kv_store_bf16(const void *q, const void *k, const void *v, const int64_t *pos,
                                       const void *cos_t, const void *sin_t, void *q_out, void *k_cache,
                                       void *v_cache, int64_t T, int64_t heads, int64_t kv_heads,
                                       int64_t head_dim, int64_t max_len, int apply_rope, void *stream) {
    GLQH_REQUIRE(q && k && v && pos && q_out && k_cache && v_cache, "rope: null pointer");
    GLQH_REQUIRE(head_dim >= 2 && head_dim <= 1024 && (head_dim & 1) == 0, "rope: bad head_dim");
    GLQH_REQUIRE(!apply_rope || (cos_t && sin_t), "rope: missing angle tables");
    hipLaunchKernelGGL(rope_kv_store_kernel, dim3((unsigned)T, (unsigned)(heads + 2 * kv_heads)),
                       dim3((unsigned)(head_dim / 2)), 0, (hipStream_t)stream, (const uint16_t *)q,
                       (const uint16_t *)k, (const uint16_t *)v, pos, (const uint16_t *)cos_t,
                       (const uint16_t *)sin_t, (uint16_t *)q_out, (uint16_t *)k_cache, (uint16_t *)v_cache,
                       (int)heads, (int)kv_heads, (int)head_dim, (int)max_len, apply_rope);
    GLQH_LAUNCH_CHECK("rope launch");
    return 0;
}

extern "C" int glqh_attn_decode_bf16(const void *q, const void *k_cache, const void *v_cache,
                                     const int64_t *pos, void *out, int64_t heads, int64_t kv_heads,
                                     int64_t head_dim, int64_t max_len, void *stream) {
    GLQH_REQUIRE(q && k_cache && v_cache && pos && out, "attention: null pointer");
    GLQH_REQUIRE(head_dim == 128, "attention: head_dim must be 128, got %lld", (long long)head_dim);
    GLQH_REQUIRE(kv_heads >= 1 && heads % kv_heads == 0, "attention: heads must be a multiple of kv_heads");
    const size_t lds = (size_t)max_len * sizeof(float);
    GLQH_REQUIRE(lds <= 48 * 1024, "attention: cache of %lld positions does not fit the score buffer",
                 (long long)max_len);
    hipLaunchKernelGGL(attn_decode_kernel, dim3((unsigned)heads), dim3(AT_THREADS), lds, (hipStream_t)stream,
                       (const uint16_t *)q, (const uint16_t *)k_cache, (const uint16_t *)v_cache, pos,
                       (uint16_t *)out, (int)heads, (int)kv_heads, (int)max_len,
                       1.0f / sqrtf((float)head_dim));
    GLQH_LAUNCH_CHECK("attention launch");
    return 0;
}

extern "C" int glqh_add_rmsnorm_bf16(const void *x, const void *delta, const void *w, void *x_out,
                                     void *h_out, int64_t T, int64_t H, double eps, void *stream) {
    GLQH_REQUIRE(x && delta && w && x_out && h_out && T >= 1 && H >= 1 && H <= 12288, "add_rmsnorm: bad arguments");
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3((unsigned)T), dim3(256), (size_t)H * sizeof(float),
                       (hipStream_t)stream, (const uint16_t *)x, (const uint16_t *)delta, (const uint16_t *)w,
                       (uint16_t *)x_out, (uint16_t *)h_out, (int)H, (float)eps);
    GLQH_LAUNCH_CHECK("add_rmsnorm launch");
    return 0;
}

extern "C" int glqh_silu_mul_bf16(const void *gate, const void *up, void *out, int64_t n, void *stream) {
    GLQH_REQUIRE(gate && up && out && n >= 1, "silu_mul: bad arguments");
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t *)gate, (const uint16_t *)up, (uint16_t *)out, n);
    GLQH_LAUNCH_CHECK("silu_mul launch");
    return 0;
}

int glqh_launch_out_add_rmsnorm(const float *part, int ksplit, float scale, const void *su, int64_t m,
                                const void *resid, const void *norm_w, float eps, void *x_out, void *h_out,
                                hipStream_t stream) {
    GLQH_REQUIRE(part && su && resid && norm_w && x_out && h_out && ksplit >= 1, "out+add+rmsnorm: bad arguments");
    GLQH_REQUIRE(m >= 32 && m <= FN_MAX_ROWS, "out+add+rmsnorm: %lld rows (32..%d)", (long long)m, FN_MAX_ROWS);
    int64_t top = 1;
    while (top * 2 <= m) top *= 2;
    const size_t lds = (size_t)((2 * FN_GROUPS << FN_LOG_SLICE) + m) * sizeof(float);
    GLQH_REQUIRE(top <= (int64_t)FN_GROUPS << FN_LOG_SLICE, "out+add+rmsnorm: %lld rows: blocks of more than %d rows",
                 (long long)m, FN_GROUPS << FN_LOG_SLICE);
    GLQH_REQUIRE(lds <= 64 * 1024, "out+add+rmsnorm: %lld rows need %zu bytes of LDS (64 KB at most)", (long long)m, lds);
    GLQH_REQUIRE((m & 3) == 0 && ((uintptr_t)part & 15) == 0,
                 "out+add+rmsnorm: rows must be a multiple of 4 and the partial sums 16-byte aligned");
    hipLaunchKernelGGL(out_add_rmsnorm_kernel, dim3(1), dim3(FN_THREADS), lds, stream, part, ksplit, scale,
                       (const f16 *)su, (int)m, (const uint16_t *)resid, (const uint16_t *)norm_w, eps,
                       (uint16_t *)x_out, (uint16_t *)h_out);
    GLQH_LAUNCH_CHECK("out+add+rmsnorm launch");
    return 0;
}

int glqh_launch_out_silu_mul(const float *part_gate, const float *part_up, int ksplit, float scale_gate,
                             float scale_up, const void *su_gate, const void *su_up, int64_t m_pad,
                             int64_t out_features, void *act_out, hipStream_t stream) {
    GLQH_REQUIRE(part_gate && part_up && su_gate && su_up && act_out && ksplit >= 1, "out+silu: bad arguments");
    GLQH_REQUIRE(m_pad >= 32 && m_pad <= 0x40000000ll && out_features >= 1 && out_features <= m_pad,
                 "out+silu: bad shape");
    GLQH_REQUIRE((m_pad & 3) == 0 && (((uintptr_t)part_gate | (uintptr_t)part_up) & 15) == 0,
                 "out+silu: rows must be a multiple of 4 and the partial sums 16-byte aligned");
    int64_t top = 1;
    while (top * 2 <= m_pad) top *= 2;
    const int log_slice = 10;                      // the slices of the few-token output transform
    const int spb = top >> log_slice < 1 ? 1 : (int)(top >> log_slice);
    const int nwg = __builtin_popcountll((unsigned long long)m_pad) * spb;
    const int buf_floats = (1 << log_slice) + (1 << log_slice) / 32 + 32;
    const size_t lds = (size_t)(2 * buf_floats + (1 << log_slice)) * sizeof(float);
    hipLaunchKernelGGL(out_silu_mul_kernel, dim3((unsigned)nwg), dim3(512), lds, stream, part_gate, part_up, ksplit,
                       scale_gate, scale_up, (const f16 *)su_gate, (const f16 *)su_up, (int)m_pad, (int)out_features,
                       (uint16_t *)act_out, spb, log_slice, buf_floats);
    GLQH_LAUNCH_CHECK("out+silu launch");
    return 0;
}

int glqh_launch_out_rope_store(const float *const part[3], const void *const su[3], const float scale[3],
                               const int64_t m[3], int ksplit, const int64_t *pos, const void *cos_t,
                               const void *sin_t, void *q_out, void *k_cache, void *v_cache, int64_t head_dim,
                               int64_t max_len, int apply_rope, hipStream_t stream) {
    GLQH_REQUIRE(pos && q_out && k_cache && v_cache && ksplit >= 1, "out+rope: bad arguments");
    GLQH_REQUIRE(!apply_rope || (cos_t && sin_t), "out+rope: missing angle tables");
    GLQH_REQUIRE(head_dim >= 2 && (head_dim & (head_dim - 1)) == 0 && head_dim <= 1024, "out+rope: bad head_dim");
    const int log_slice = 10;
    qkv_fin a = {};
    int64_t top_max = 1;
    int max_nwg = 0;
    for (int i = 0; i < 3; ++i) {
        GLQH_REQUIRE(part[i] && su[i] && m[i] >= head_dim && m[i] <= 0x40000000ll && m[i] % head_dim == 0,
                     "out+rope: layer %d: rows must be whole heads", i);
        GLQH_REQUIRE((m[i] & (head_dim - 1)) == 0, "out+rope: every output block must hold whole heads");
        GLQH_REQUIRE(head_dim >= 4 && ((uintptr_t)part[i] & 15) == 0, "out+rope: layer %d: partial sums must be 16-byte aligned", i);
        a.part[i] = part[i]; a.su[i] = (const f16 *)su[i]; a.scale[i] = scale[i]; a.m[i] = (int)m[i];
        int64_t top = 1;
        while (top * 2 <= m[i]) top *= 2;
        if (top > top_max) top_max = top;
    }
    const int spb = top_max >> log_slice < 1 ? 1 : (int)(top_max >> log_slice);
    for (int i = 0; i < 3; ++i) {
        const int nwg = __builtin_popcountll((unsigned long long)m[i]) * spb;
        if (nwg > max_nwg) max_nwg = nwg;
    }
    const size_t lds = (size_t)((1 << log_slice) + (1 << log_slice) / 32 + 32) * sizeof(float);
    hipLaunchKernelGGL(out_rope_store_kernel, dim3((unsigned)max_nwg, 3), dim3(256), lds, stream, a, ksplit, pos,
                       (const uint16_t *)cos_t, (const uint16_t *)sin_t, (uint16_t *)q_out, (uint16_t *)k_cache,
                       (uint16_t *)v_cache, (int)head_dim, (int)max_len, apply_rope, spb, log_slice);
    GLQH_LAUNCH_CHECK("out+rope launch");
    return 0;
}

#ifndef ATTN_SPLIT_MIN
#define ATTN_SPLIT_MIN 512                                      // keys per share at least
#endif
constexpr int ATTN_SPLIT_MAX_HEADS = 256;                       // counters at the head of the state buffer

int glqh_attn_split_shares(int64_t max_len) {
    const int64_t s = (max_len - 1) / ATTN_SPLIT_MIN;            // a cache of 1024 positions never holds two shares
    return s < 1 ? 1 : s > 8 ? 8 : (int)s;
}

extern "C" size_t glqh_attn_split_state_bytes(int64_t heads, int64_t max_len) {
    if (glqh_attn_split_shares(max_len) == 1) return 0;         // too short for shares: no state needed
    return ATTN_SPLIT_MAX_HEADS * sizeof(unsigned int) +
           (size_t)heads * glqh_attn_split_shares(max_len) * AT_PART * sizeof(float);
}

int glqh_launch_out_rope_attn(const float *const part[3], const void *const su[3], const float scale[3],
                              const int64_t m[3], int ksplit, const int64_t *pos, const void *cos_t,
                              const void *sin_t, void *k_cache, void *v_cache, void *out, int64_t heads,
                              int64_t kv_heads, int64_t head_dim, int64_t max_len, int apply_rope,
                              void *split_state, size_t split_state_bytes, hipStream_t stream) {
    GLQH_REQUIRE(pos && k_cache && v_cache && out && ksplit >= 1, "out+rope+attention: bad arguments");
    GLQH_REQUIRE(!apply_rope || (cos_t && sin_t), "out+rope+attention: missing angle tables");
    GLQH_REQUIRE(head_dim == 128, "out+rope+attention: head_dim must be 128, got %lld", (long long)head_dim);
    GLQH_REQUIRE(kv_heads >= 1 && heads % kv_heads == 0, "out+rope+attention: heads must be a multiple of kv_heads");
    GLQH_REQUIRE(m[0] == heads * head_dim && m[1] == kv_heads * head_dim && m[2] == m[1],
                 "out+rope+attention: layer heights do not match the head counts");
    qkv_fin a = {};
    for (int i = 0; i < 3; ++i) {
        GLQH_REQUIRE(part[i] && su[i] && m[i] <= 0x40000000ll && (m[i] & (head_dim - 1)) == 0,
                     "out+rope+attention: layer %d: every output block must hold whole heads", i);
        GLQH_REQUIRE(((uintptr_t)part[i] & 15) == 0, "out+rope+attention: layer %d: partial sums must be 16-byte aligned", i);
        a.part[i] = part[i]; a.su[i] = (const f16 *)su[i]; a.scale[i] = scale[i]; a.m[i] = (int)m[i];
    }
    const int log_slice = 10;
    const int buf_floats = (1 << log_slice) + (1 << log_slice) / 32 + 32;
    // With a state buffer the keys of a long context are shared by up to eight workgroups per head, each with at
    // least ATTN_SPLIT_MIN keys: a share then holds fewer than 2 * ATTN_SPLIT_MIN keys or an eighth of the cache.
    int shares = 1;
    if (split_state && glqh_attn_split_shares(max_len) > 1) {
        shares = glqh_attn_split_shares(max_len);
        GLQH_REQUIRE(split_state_bytes >= glqh_attn_split_state_bytes(heads, max_len) && ((uintptr_t)split_state & 15) == 0,
                     "out+rope+attention: state buffer of %zu bytes needed (16-byte aligned), got %zu",
                     glqh_attn_split_state_bytes(heads, max_len), split_state_bytes);
        GLQH_REQUIRE(heads <= ATTN_SPLIT_MAX_HEADS, "out+rope+attention: at most %d heads with a state buffer", ATTN_SPLIT_MAX_HEADS);
    }
    const int64_t longest = shares == 1 ? max_len : std::max<int64_t>(2 * ATTN_SPLIT_MIN, (max_len + shares - 1) / shares);
    const int sc_floats = (int)((longest + 31) / 32 * 32);
    const size_t lds = (size_t)(sc_floats + 3 * buf_floats) * sizeof(float);
    GLQH_REQUIRE(lds <= 60 * 1024, "out+rope+attention: cache of %lld positions does not fit the score buffer",
                 (long long)max_len);
    unsigned int *cnt = (unsigned int *)split_state;
    float *sbuf = split_state ? (float *)((char *)split_state + ATTN_SPLIT_MAX_HEADS * sizeof(unsigned int)) : nullptr;
#define GLQH_ATTN_LAUNCH(SHARED)                                                                              \
    hipLaunchKernelGGL(out_rope_attn_kernel<SHARED>, dim3((unsigned)heads, (unsigned)shares), dim3(AT_THREADS), lds, \
                       stream, a, ksplit, pos, (const uint16_t *)cos_t, (const uint16_t *)sin_t,                  \
                       (uint16_t *)k_cache, (uint16_t *)v_cache, (uint16_t *)out, (int)heads, (int)kv_heads,      \
                       (int)max_len, apply_rope, 1.0f / sqrtf((float)head_dim), log_slice, sc_floats, buf_floats, \
                       sbuf, cnt, ATTN_SPLIT_MIN)
    if (shares > 1) GLQH_ATTN_LAUNCH(true);
    else GLQH_ATTN_LAUNCH(false);
#undef GLQH_ATTN_LAUNCH
    GLQH_LAUNCH_CHECK("out+rope+attention launch");
    return 0;
}

static int lm_head_wgs(void) { return glqh_device_cus() * 4; }

extern "C" size_t glqh_lm_head_workspace_bytes(void) { return (size_t)lm_head_wgs() * 4 * 8; }

extern "C" int glqh_lm_head_argmax_bf16(const void *h, const void *table, int64_t vocab, int64_t hidden,
                                        float *logits_out, int64_t *token_out, void *ws, size_t ws_bytes,
                                        void *stream) {
    GLQH_REQUIRE(h && table && token_out && ws, "lm_head: null pointer");
    GLQH_REQUIRE(vocab >= 1 && vocab < ((int64_t)1 << 31), "lm_head: vocab %lld out of range", (long long)vocab);
    GLQH_REQUIRE(hidden == 2048 || hidden == 4096, "lm_head: hidden size %lld (2048 or 4096)", (long long)hidden);
    GLQH_REQUIRE((((uintptr_t)h | (uintptr_t)table) & 15) == 0, "lm_head: pointers must be 16-byte aligned");
    const int wgs = lm_head_wgs(), nw = wgs * 4;
    GLQH_REQUIRE(ws_bytes >= (size_t)nw * 8, "lm_head: workspace of %zu bytes needed, got %zu", (size_t)nw * 8, ws_bytes);
    float *bv = (float *)ws;
    int *br = (int *)ws + nw;
    hipStream_t st = (hipStream_t)stream;
    if (hidden == 2048)
        hipLaunchKernelGGL(lm_head_kernel<4>, dim3((unsigned)wgs), dim3(256), 0, st, (const uint16_t *)h,
                           (const uint16_t *)table, logits_out, bv, br, (int)vocab);
    else
        hipLaunchKernelGGL(lm_head_kernel<8>, dim3((unsigned)wgs), dim3(256), 0, st, (const uint16_t *)h,
                           (const uint16_t *)table, logits_out, bv, br, (int)vocab);
    GLQH_LAUNCH_CHECK("lm_head launch");
    hipLaunchKernelGGL(lm_head_argmax_kernel, dim3(1), dim3(256), 0, st, bv, br, nw, token_out);
    GLQH_LAUNCH_CHECK("lm_head argmax launch");
    return 0;
}
