// extern "C" entry points of libglq_hip.so: argument checks, dispatch, no allocation.
#include <unordered_map>
#include <vector>

#include "common.h"

#include <atomic>
#include <mutex>
#include <string.h>
#include <stdlib.h>

int glqh_rht_init(void);
int glqh_e8_init(void);
int glqh_launch_trellis_decompress(const void *packed, int R, int64_t m, int64_t k, void *out,
                                   hipStream_t stream);
int glqh_trellis_mma_plan(int64_t m, int64_t k, int *S_out, int *ksplit_out);
int glqh_launch_trellis_mma(const void *x_f16, int64_t B, const void *packed, int R, int64_t m, int64_t k,
                            int S, int ksplit, float *part, int direct, float scale, int accum,
                            int64_t out_stride, hipStream_t stream);
int glqh_trellis_mma_init(void);
int glqh_viterbi_init(void);

// many-token E8 kernel on the compressed indices (e8_tile.hip)
int glqh_e8_tile_init(void);
int glqh_trellis_tile_init(void);
int glqh_e8_tile_ksplit(int64_t m_pad, int64_t n_pad, int64_t M, int nstages, int fold);
size_t glqh_e8_tile_xb_bytes(int64_t n_pad, int64_t M);
int glqh_launch_e8_tile(const void *x_f16, void *xb_scratch, int64_t M, const void *const q[4], int nstages,
                        const uint32_t *t1, const uint32_t *t2, int64_t n2, const float rel[3], int64_t m_pad,
                        int64_t n_pad, float *part, hipStream_t stream, const glqh_e8_folded *fold, int out_f16 = 0,
                        float f16_scale = 1.0f);
int glqh_e8_tile_f16_sums_ok(int64_t M, int fold, int64_t m_pad);
// Above 16 tokens the weights are decoded once per 128 x 512 tile instead of once per 16 tokens.
#define GLQH_E8_SMALL_BATCH 16
static int e8_tile_ks(int64_t m_pad, int64_t n_pad, int64_t B, int nstages, bool fold) {
    return B > GLQH_E8_SMALL_BATCH ? glqh_e8_tile_ksplit(m_pad, n_pad, B, nstages, fold) : 0;
}

int glqh_trellis_mma_fusein_plan(int64_t wgs_rows, int64_t k, int64_t B, int *S_out, int *ksplit_out);
int glqh_launch_trellis_mma_rvq(const void *x_f16, int64_t B, const void *packed, const void *packed2, int R2, float rs2,
                                int64_t m, int64_t k, int S, int ksplit, float *part, hipStream_t stream);
int glqh_launch_trellis_mma_fusein_rvq(const void *const packed[], const void *const packed2[], int R2, const float rs2[],
                                       const void *const sv[], float *const part[], const int64_t m[], int n_layers,
                                       const void *x, int x_dtype, int64_t x_stride, int64_t k, int64_t in_features,
                                       int S, int ksplit, const glqh_block_meta *bn_meta, const int64_t *blocks_host,
                                       int n_blocks, hipStream_t stream);
int glqh_launch_trellis_mma_fusein(const void *const packed[], const void *const sv[], float *const part[],
                                   const int64_t m[], int n_layers, int R, const void *x, int x_dtype,
                                   int64_t x_stride, int64_t B, int64_t k, int64_t in_features, int S,
                                   int ksplit, const glqh_block_meta *bn_meta, const int64_t *blocks_host,
                                   int n_blocks, float pscale, hipStream_t stream);
// K plan of the fused-input GEMV for layers of the given padded heights sharing one input.
// Returns 0 (not eligible), 1 (32-row workgroups, v_dot2 decode) or 2 (64-row workgroups, MFMA
// decode: fewer vector-ALU operations per weight and half as many redundant input transforms).
// The MFMA form wins from 32 strips of 64 rows on (measured on the 2048-row attention / down
// shapes: 9.8 vs 10.7 us per launch on average); below that the launch is pure latency and the
// smaller workgroups of the v_dot2 form spread it over more CUs.
#define GLQH_FUSEIN_MMA_MIN_STRIPS 32
static int tr_fusein_plan(const int64_t *m_pads, int n, int64_t n_pad, int64_t B, int *S, int *ks,
                          int mma_min_strips = GLQH_FUSEIN_MMA_MIN_STRIPS) {
    int64_t total = 0, wgs = 0;
    for (int i = 0; i < n; ++i) { total += m_pads[i]; wgs += (m_pads[i] + 63) / 64; }
    if (wgs >= mma_min_strips) return glqh_trellis_mma_fusein_plan(wgs, n_pad, B, S, ks) ? 2 : 0;
    return glqh_trellis_fusein_plan(total, n_pad, B, S, ks) ? 1 : 0;
}
// many-token kernel (trellis_tile.hip): weights decoded once per 128-row x 512-token tile
size_t glqh_trellis_tile_xb_bytes(int64_t k, int64_t M);
int glqh_trellis_tile_ksplit(int64_t m, int64_t k, int64_t M, int two_stage = 0);
int glqh_launch_trellis_tile(const void *x_f16, void *xb_scratch, int64_t M, const void *packed, int R, int64_t m,
                             int64_t k, float *out, int direct, float scale, int accum, int64_t out_stride,
                             hipStream_t stream, int out_f16 = 0, const void *packed2 = nullptr, int R2 = 0,
                             float rs2 = 0.0f);
int64_t glqh_trellis_tile_padded_tokens(int64_t M);
int glqh_trellis_tile_group_ksplit(const int64_t *m, int n_layers, int64_t k, int64_t M);
int glqh_launch_trellis_tile_group(const void *const xb[], int64_t M, const void *const packed[], int R,
                                   const int64_t m[], int n_layers, int64_t k, float *const out[], int out_f16,
                                   hipStream_t stream, const float f16_scale[] = nullptr);
int glqh_launch_trellis_pack(const void *x_f16, void *xb, int64_t M, int64_t k, hipStream_t stream);
int64_t glqh_e8_tile_padded_tokens(int64_t M, int nstages);
// several sign vectors on the same few rows in one launch (fht.hip); -1 = not eligible, nothing launched
int glqh_launch_input_rht_multi(const void *x, int x_dtype, int64_t x_stride, const void *const sv[], void *const out[],
                                int n, int64_t B, int64_t in_features, int64_t n_pad, const glqh_block_meta *meta_dev,
                                const int64_t *blocks_host, int64_t n_blocks, hipStream_t stream);
int glqh_launch_input_rht_blocked_multi(const void *x, int x_dtype, int64_t x_stride, const void *const sv[],
                                        void *const xb[], int n, int64_t Mp, int64_t B, int64_t in_features, int64_t n_pad,
                                        const int64_t *blocks_host, int64_t n_blocks, hipStream_t stream);
// input transform straight into a tile kernel's operand layout (fht.hip); -1 = not eligible, nothing launched
int glqh_launch_input_rht_blocked(const void *x, int x_dtype, int64_t x_stride, const void *sv, void *xb,
                                  int layout, int64_t Mp, int64_t B, int64_t in_features, int64_t n_pad,
                                  const int64_t *blocks_host, int64_t n_blocks, hipStream_t stream);

// Plan for activations already in the transformed domain: up to 16 tokens share one pass over
// the packed stream with K split by shape only; larger batches use the tile kernels, which
// need scratch for their repacked activations (xb_bytes).  The small-batch kernel decodes the
// stream once per 16 tokens, the tile kernels once (whole linear, us, small-batch / tile kernel:
// 4096 x 4096 23.5 / 19.8 at 17 tokens, 26.9 / 21.2 at 32, 35.6 / 24.1 at 48, 39.3 / 25.4 at 64;
// 2048 x 11008 27.3 / 23.2, 30.9 / 25.1, 41.0 / 30.6, 44.5 / 31.8; 11008 x 2048 32.0 / 24.0, 30.2 / 24.5,
// 38.6 / 27.2, 42.8 / 28.0; 2048 x 2048 15.3 / 16.6, 16.9 / 16.3, 22.2 / 18.3, 21.9 / 18.9).
// GLQ_TRELLIS_TILE_MIN=<n> (17..65, read once): the tile kernels take calls of n tokens and more
static int tr_small_batch() {
    static const int v = [] {
        const char *e = getenv("GLQ_TRELLIS_TILE_MIN");
        const int n = e ? atoi(e) : 0;
        return n >= 17 && n <= 65 ? n - 1 : 16;
    }();
    return v;
}
struct tr_plan {
    int ks, S, tile;
    size_t xb_bytes;
};
static tr_plan tr_plain_plan(int64_t m, int64_t k, int64_t B) {
    tr_plan p = {1, 0, B > tr_small_batch(), 0};
    if (p.tile) {
        p.ks = glqh_trellis_tile_ksplit(m, k, B);
        p.xb_bytes = (glqh_trellis_tile_xb_bytes(k, B) + 255) & ~(size_t)255;
    } else {
        glqh_trellis_mma_plan(m, k, &p.S, &p.ks);
    }
    return p;
}
// pscale multiplies the partial sums as they are written (small-batch kernel only): a second
// stage stored pre-scaled is just more K slots to whoever sums them.  xb: scratch of
// plan.xb_bytes for the tile kernel (unused otherwise).
static int tr_plain_partial(tr_plan p, const void *x_f16, int64_t B, const void *packed, int R, int64_t m,
                            int64_t k, float *part, void *xb, hipStream_t st, float pscale = 1.0f, int f16_sums = 0,
                            float f16_scale = 1.0f) {
    glqh_range range("dequant_matmul");
    // fp16 sums leave the tile kernel times f16_scale (the layer's scale: a long row of large activations then stays
    // inside the fp16 range wherever the layer's output does)
    if (p.tile) return glqh_launch_trellis_tile(x_f16, xb, B, packed, R, m, k, part, 0, f16_sums ? f16_scale : 1.0f, 0, 0, st, f16_sums);
    return glqh_launch_trellis_mma(x_f16, B, packed, R, m, k, p.S, p.ks, part, 0, pscale, 0, 0, st);
}
static int tr_plain_direct(tr_plan p, const void *x_f16, int64_t B, const void *packed, int R, int64_t m,
                           int64_t k, float scale, float *out, int64_t out_stride, int accum, void *xb,
                           hipStream_t st) {
    glqh_range range("dequant_matmul");
    if (p.tile) return glqh_launch_trellis_tile(x_f16, xb, B, packed, R, m, k, out, 1, scale, accum, out_stride, st);
    return glqh_launch_trellis_mma(x_f16, B, packed, R, m, k, p.S, 1, out, 1, scale, accum, out_stride, st);
}

// ---- error plumbing -------------------------------------------------------------
static thread_local char g_err[512] = "";

int glqh_fail(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return 1;
}

int glqh_check_hip(hipError_t e, const char *what) {
    if (e == hipSuccess) return 0;
    return glqh_fail("%s: %s", what, hipGetErrorString(e));
}

// ---- profiling ranges ---------------------------------------------------------------
#include <dlfcn.h>
static struct {
    std::once_flag once;
    int (*push)(const char *);
    int (*pop)(void);
} g_roctx;

static void roctx_resolve() {
    const char *e = getenv("GLQ_ROCTX");
    if (e && e[0] == '0') return;
    const int mode = (e && e[0] == '1') ? RTLD_NOW | RTLD_GLOBAL : RTLD_NOW | RTLD_NOLOAD;
    const char *names[] = {"librocprofiler-sdk-roctx.so.1", "librocprofiler-sdk-roctx.so", "libroctx64.so.4",
                           "libroctx64.so"};
    for (const char *n : names) {
        void *h = dlopen(n, mode);
        if (!h) continue;
        void *pu = dlsym(h, "roctxRangePushA"), *po = dlsym(h, "roctxRangePop");
        if (pu && po) {
            g_roctx.push = (int (*)(const char *))pu;
            g_roctx.pop = (int (*)(void))po;
            return;
        }
    }
}

glqh_range::glqh_range(const char *name) {
    std::call_once(g_roctx.once, roctx_resolve);
    on = g_roctx.push != nullptr;
    if (on) g_roctx.push(name);
}
glqh_range::~glqh_range() {
    if (on) g_roctx.pop();
}

static int g_cus = 0;
static int g_init_rc = -1;
static std::once_flag g_once;

int glqh_device_cus(void) { return g_cus > 0 ? g_cus : 256; }

extern "C" const char *glqh_last_error(void) { return g_err; }
extern "C" int glqh_version(void) { return 1; }

// Scratch of the entry point that allocates nothing (glqh_fused_linear_trellis_3inst_noalloc, below):
// a file-scope device array.  Every GPU holds its own copy at its own address; the address is
// resolved once per device -- by glqh_init() for whichever device is current when any entry of the
// library is first called there -- and host code uses that address only, never the array's name.
#define GLQH_NOALLOC_SCRATCH_BYTES ((size_t)8 << 20)
#define GLQH_NOALLOC_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[GLQH_NOALLOC_SCRATCH_BYTES];
static std::atomic<void *> g_scratch_ptr[GLQH_NOALLOC_MAX_DEVICES];
static std::mutex g_scratch_mu;

static int noalloc_scratch_for_current_device(void **out) {
    int dev = -1;
    if (glqh_check_hip(hipGetDevice(&dev), "hipGetDevice")) return 1;
    GLQH_REQUIRE(dev >= 0 && dev < GLQH_NOALLOC_MAX_DEVICES, "no-alloc entry: device index %d out of range", dev);
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> lk(g_scratch_mu);
        p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (!p) {
            if (glqh_check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return 1;
            GLQH_REQUIRE(p != nullptr, "no-alloc entry: scratch array has no device address");
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    if (out) *out = p;
    return 0;
}

extern "C" int glqh_init(void) {
    std::call_once(g_once, [] {
        int dev = 0;
        hipDeviceProp_t prop;
        if (glqh_check_hip(hipGetDevice(&dev), "hipGetDevice") ||
            glqh_check_hip(hipGetDeviceProperties(&prop, dev), "hipGetDeviceProperties")) {
            g_init_rc = 1;
            return;
        }
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
            g_init_rc = glqh_fail("libglq_hip is built for gfx950 only, device is %s", prop.gcnArchName);
            return;
        }
        g_cus = prop.multiProcessorCount;
        g_init_rc = glqh_rht_init() || glqh_e8_init() || glqh_e8_tile_init() || glqh_trellis_init() || glqh_trellis_tile_init() || glqh_trellis_mma_init() || glqh_viterbi_init();
    });
    if (g_init_rc != 0 && g_err[0] == 0) glqh_fail("libglq_hip initialisation failed earlier");
    if (g_init_rc != 0) return g_init_rc;
    // per device, so that the no-alloc entry has nothing left to set up when it runs under capture
    return noalloc_scratch_for_current_device(nullptr);
}

#define GLQH_INIT()                      \
    do {                                 \
        if (glqh_init() != 0) return 1;  \
    } while (0)

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// GLQ_TRELLIS_FUSE_STAGES=0: one token of a two-stage layer decodes its stages in two launches again.
static bool tr_fuse_stages_enabled() {
    static const bool on = [] {
        const char *e = getenv("GLQ_TRELLIS_FUSE_STAGES");
        return !(e && e[0] == '0');
    }();
    return on;
}

// GLQ_TRELLIS_FUSE_INPUT=0 keeps the input transform a launch of its own at every token count,
// the reference's switch of the same name (glq/csrc/glq_trellis.cu:1270-1274).  Read once.
static bool tr_fuse_input_enabled() {
    static const bool on = [] {
        const char *e = getenv("GLQ_TRELLIS_FUSE_INPUT");
        return !(e && e[0] == '0');
    }();
    return on;
}

static int tr_f16_sums_max_slots() {                           // GLQ_TRELLIS_F16_SUMS_SLOTS: K slots up to which the sums are fp16
    static const int v = [] {
        const char *e = getenv("GLQ_TRELLIS_F16_SUMS_SLOTS");
        return e ? atoi(e) : 16;
    }();
    return v;
}

static bool tr_f16_sums_enabled() {
    static const bool on = [] {
        const char *e = getenv("GLQ_TRELLIS_F16_SUMS");
        return !(e && e[0] == '0');
    }();
    return on;
}

// ---- trellis ---------------------------------------------------------------------
extern "C" int glqh_trellis_kernel_supported(int64_t m, int64_t k) {
    return m > 0 && k > 0 && m % 32 == 0 && k % 64 == 0;
}

static int tr_bits_from_packed(int64_t packed_cols, int allow_r1, int *R) {
    int r = (int)(packed_cols / 16);
    int lo = allow_r1 ? 1 : 2;
    GLQH_REQUIRE(packed_cols % 16 == 0 && r >= lo && r <= 4,
                 "trellis kernel supports R (bits/weight) %d-4, got packed width %lld", lo,
                 (long long)packed_cols);
    *R = r;
    return 0;
}

static int tr_check_shape(int64_t m, int64_t k, int64_t packed_rows) {
    GLQH_REQUIRE(m > 0 && m % 32 == 0, "trellis kernel needs m %% 32 == 0, got %lld", (long long)m);
    GLQH_REQUIRE(k > 0 && k % 64 == 0, "trellis kernel needs k %% 64 == 0, got %lld", (long long)k);
    GLQH_REQUIRE(packed_rows == (m / 16) * (k / 16), "trellis_packed rows %lld != (m/16)*(k/16)",
                 (long long)packed_rows);
    GLQH_REQUIRE(m / 32 <= 65535, "trellis kernel: m too large");
    return 0;
}

extern "C" int glqh_decompress_trellis_3inst(const void *packed, int64_t packed_rows,
                                             int64_t packed_cols, int64_t m, int64_t k, int allow_r1,
                                             void *out_f16, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(packed && out_f16, "decompress: null pointer");
    int R;
    if (tr_bits_from_packed(packed_cols, allow_r1, &R) || tr_check_shape(m, k, packed_rows)) return 1;
    return glqh_launch_trellis_decompress(packed, R, m, k, out_f16, (hipStream_t)stream);
}

extern "C" size_t glqh_trellis_gemv_workspace_bytes(int64_t m, int64_t k, int64_t B) {
    if (!glqh_trellis_kernel_supported(m, k) || B < 1) return 0;
    glqh_init();
    const tr_plan p = tr_plain_plan(m, k, B);
    // (the many-token kernel's figure also serves glqh_trellis_gemv_partials, which always stores the sums)
    return (p.ks > 1 || p.tile ? align256((size_t)p.ks * B * m * sizeof(float)) : 0) + p.xb_bytes;
}

extern "C" int glqh_decode_matmul_trellis_3inst(const void *x_f16, int64_t B, const void *packed,
                                                int64_t packed_rows, int64_t packed_cols, int64_t m,
                                                int64_t k, double wscale, float *out,
                                                int64_t out_stride, int accum, void *ws,
                                                size_t ws_bytes, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(x_f16 && packed && out, "trellis matmul: null pointer");
    GLQH_REQUIRE(B >= 1 && B <= 65535 * 8, "trellis matmul: B=%lld out of range", (long long)B);
    GLQH_REQUIRE(out_stride >= m, "trellis matmul: out stride %lld < m", (long long)out_stride);
    int R;
    if (tr_bits_from_packed(packed_cols, accum, &R) || tr_check_shape(m, k, packed_rows)) return 1;
    hipStream_t st = (hipStream_t)stream;
    const tr_plan plan = tr_plain_plan(m, k, B);
    const int ks = plan.ks;
    const size_t pbytes = ks > 1 ? align256((size_t)ks * B * m * sizeof(float)) : 0;
    const size_t need = pbytes + plan.xb_bytes;
    GLQH_REQUIRE(need == 0 || (ws && ws_bytes >= need), "trellis matmul: workspace of %zu bytes needed, got %zu",
                 need, ws_bytes);
    void *xb = (char *)ws + pbytes;
    if (ks == 1)
        return tr_plain_direct(plan, x_f16, B, packed, R, m, k, (float)wscale, out, out_stride, accum, xb, st);
    if (tr_plain_partial(plan, x_f16, B, packed, R, m, k, (float *)ws, xb, st)) return 1;
    return glqh_launch_reduce_splits((const float *)ws, ks, B * m, B, m, (float)wscale, out, out_stride, accum, st);
}

extern "C" int glqh_trellis_gemv_partials(const void *x_f16, int64_t B, const void *packed,
                                          int64_t packed_rows, int64_t packed_cols, int64_t m,
                                          int64_t k, float *part, size_t part_bytes, int *ksplit_out,
                                          void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(x_f16 && packed && part && ksplit_out, "trellis partials: null pointer");
    GLQH_REQUIRE(B >= 1 && B <= 65535 * 8, "trellis partials: B=%lld out of range", (long long)B);
    int R;
    if (tr_bits_from_packed(packed_cols, 1, &R) || tr_check_shape(m, k, packed_rows)) return 1;
    const tr_plan plan = tr_plain_plan(m, k, B);
    const int ks = plan.ks;
    // in the tile kernel's range its repacked activations follow the partial sums
    const size_t pbytes = align256((size_t)ks * B * m * sizeof(float));
    const size_t need = plan.tile ? pbytes + plan.xb_bytes : (size_t)ks * B * m * sizeof(float);
    GLQH_REQUIRE(part_bytes >= need, "trellis partials: buffer of %zu bytes needed, got %zu", need, part_bytes);
    *ksplit_out = ks;
    return tr_plain_partial(plan, x_f16, B, packed, R, m, k, part, (char *)part + pbytes, (hipStream_t)stream);
}

// ---- RHT -------------------------------------------------------------------------
extern "C" int glqh_input_rht(const void *x, int x_dtype, int64_t x_stride, const void *sv_f16,
                              void *out, int out_dtype, int64_t B, int64_t in_features,
                              int64_t n_pad, const glqh_block_meta *meta_dev,
                              const int64_t *blocks_host, int64_t n_blocks, double rsqrt_n,
                              void *stream) {
    GLQH_INIT();
    return glqh_launch_input_rht(x, x_dtype, x_stride, sv_f16, out, out_dtype, B, in_features, n_pad,
                                 meta_dev, blocks_host, n_blocks, (float)rsqrt_n, (hipStream_t)stream);
}

extern "C" int glqh_output_rht(const float *y_rht, int64_t y_rht_stride, const void *su_f16, void *y,
                               int y_dtype, int64_t y_stride, int64_t B, int64_t out_features,
                               int64_t m_pad, const glqh_block_meta *meta_dev,
                               const int64_t *blocks_host, int64_t n_blocks, double rsqrt_m,
                               void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(y_rht && y, "output_rht: null pointer");
    GLQH_REQUIRE(y_rht_stride >= m_pad && y_stride >= out_features, "output_rht: bad strides");
    glqh_ysrc src = {};
    src.direct = y_rht;
    src.stride = y_rht_stride;
    return glqh_launch_output_rht(src, su_f16, y, y_dtype, y_stride, B, out_features, m_pad, meta_dev,
                                  blocks_host, n_blocks, 0, (float)rsqrt_m, (hipStream_t)stream);
}

extern "C" int glqh_output_rht_scaled(const float *y_rht, double scale, const void *su_f16, void *y,
                                      int y_dtype, int64_t y_stride, int64_t B, int64_t out_features,
                                      int64_t m_pad, const glqh_block_meta *meta_dev,
                                      const int64_t *blocks_host, int64_t n_blocks, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(y_rht && y, "output_rht: null pointer");
    GLQH_REQUIRE(y_stride >= out_features, "output_rht: bad strides");
    glqh_ysrc src = {};                                          // one "partial sum" per element, one stage
    src.part = y_rht;
    src.ksplit = 1;
    src.nparts = 1;
    src.scale[0] = (float)scale;
    return glqh_launch_output_rht(src, su_f16, y, y_dtype, y_stride, B, out_features, m_pad, meta_dev,
                                  blocks_host, n_blocks, 0, 0.0f, (hipStream_t)stream);
}

extern "C" int glqh_output_rht_shards(const float *y_rht, const void *su_f16, void *y, int y_dtype,
                                      int64_t B, int64_t out_features, int64_t total_m,
                                      const glqh_block_meta *shard_meta_dev, int64_t n_rows,
                                      int64_t max_bs, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(y_rht && y && shard_meta_dev, "output_rht_shards: null pointer");
    GLQH_REQUIRE(n_rows >= 1 && n_rows <= 65535, "output_rht_shards: %lld meta rows", (long long)n_rows);
    GLQH_REQUIRE(max_bs >= 1 && max_bs <= total_m, "output_rht_shards: max_bs %lld out of range",
                 (long long)max_bs);
    glqh_ysrc src = {};
    src.direct = y_rht;
    src.stride = total_m;
    return glqh_launch_output_rht(src, su_f16, y, y_dtype, out_features, B, out_features, total_m,
                                  shard_meta_dev, nullptr, n_rows, max_bs, 0.0f, (hipStream_t)stream);
}

// ---- fused trellis linear ----------------------------------------------------------
// workspace layout: [x_rht f16 (B, n_pad)] [partials stage 1] [partials stage 2]
static size_t tr_fused_part_bytes(int64_t B, int64_t n_pad, int64_t m_pad) {
    int ks = tr_plain_plan(m_pad, n_pad, B).ks;
    if (B > tr_small_batch()) ks = std::max(ks, glqh_trellis_tile_ksplit(m_pad, n_pad, B, 1));   // a stacked layer's plan
    int steps = 0, ks2 = 0;
    if (tr_fusein_plan(&m_pad, 1, n_pad, B, &steps, &ks2) && ks2 > ks) ks = ks2;
    // one token of a two-stage layer plans the MFMA form at every height
    if (B == 1 && tr_fusein_plan(&m_pad, 1, n_pad, B, &steps, &ks2, 1) && ks2 > ks) ks = ks2;
    return align256((size_t)ks * B * m_pad * sizeof(float));
}

extern "C" size_t glqh_fused_linear_trellis_workspace_bytes(int64_t B, int64_t n_pad, int64_t m_pad) {
    if (!glqh_trellis_kernel_supported(m_pad, n_pad) || B < 1) return 0;
    glqh_init();
    return align256((size_t)B * n_pad * sizeof(f16)) + 2 * tr_fused_part_bytes(B, n_pad, m_pad) +
           tr_plain_plan(m_pad, n_pad, B).xb_bytes;
}

extern "C" int glqh_fused_linear_trellis_3inst(
    const void *x, int x_dtype, int64_t x_stride, int64_t B, const void *sv_f16, const void *su_f16,
    const void *packed, int64_t packed_rows, int64_t packed_cols, const void *packed2,
    int64_t packed2_rows, int64_t packed2_cols, const int64_t *blocks_n, int64_t n_blocks_n,
    const int64_t *blocks_m, int64_t n_blocks_m, const glqh_block_meta *bn_meta_dev,
    const glqh_block_meta *bm_meta_dev, double wscale, double inv_resid_scale2, int64_t in_features,
    int64_t out_features, int64_t n_pad, int64_t m_pad, void *y, int y_dtype, int64_t y_stride,
    float *y_rht_out, int64_t y_rht_stride, void *ws, size_t ws_bytes, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(x && sv_f16 && packed, "fused trellis linear: null pointer");
    GLQH_REQUIRE(y || y_rht_out, "fused trellis linear: no output buffer");
    GLQH_REQUIRE(!y || su_f16, "fused trellis linear: null su");
    GLQH_REQUIRE(B >= 1 && B <= 65535, "fused trellis linear: B=%lld out of range", (long long)B);
    const bool has_s2 = packed2 != nullptr && packed2_rows > 0;
    GLQH_REQUIRE(has_s2 == (inv_resid_scale2 != 0.0),
                 "trellis RVQ stage 2 is half-configured: trellis_packed2 is %s but inv_resid_scale2 = %g. "
                 "Refusing rather than silently decoding stage 1 only.",
                 has_s2 ? "present" : "absent", inv_resid_scale2);
    int R1, R2 = 0;
    if (tr_bits_from_packed(packed_cols, 0, &R1) || tr_check_shape(m_pad, n_pad, packed_rows)) return 1;
    if (has_s2 && (tr_bits_from_packed(packed2_cols, 1, &R2) || tr_check_shape(m_pad, n_pad, packed2_rows)))
        return 1;
    GLQH_REQUIRE(in_features <= n_pad && out_features <= m_pad, "fused trellis linear: features exceed padded dims");
    GLQH_REQUIRE(!y_rht_out || y_rht_stride >= m_pad, "fused trellis linear: y_rht stride %lld < m_pad",
                 (long long)y_rht_stride);
    hipStream_t st = (hipStream_t)stream;

    const size_t xb = align256((size_t)B * n_pad * sizeof(f16));
    const size_t pb = tr_fused_part_bytes(B, n_pad, m_pad);
    const size_t tile_xb = tr_plain_plan(m_pad, n_pad, B).xb_bytes;
    GLQH_REQUIRE(ws && ws_bytes >= xb + 2 * pb + tile_xb, "fused trellis linear: workspace of %zu bytes needed, got %zu",
                 xb + 2 * pb + tile_xb, ws_bytes);
    void *xb_tile = (char *)ws + xb + 2 * pb;                  // repacked activations of the many-token kernel
    f16 *x_rht = (f16 *)ws;
    float *part1 = (float *)((char *)ws + xb);
    float *part2 = (float *)((char *)ws + xb + pb);

    // Two stages at a small batch with canonical output blocks: the second stage's partial
    // sums are written already multiplied by inv_resid_scale2, right behind the first stage's
    // slots, and the finishing kernels of the single-stage path sum all 2*ks slots (the generic
    // two-part transform takes twice as long: 14.3 against 6.8 us at 4096 x 4096).
    glqh_meta_args canon_m;
    // The slice kernels of the grouped launcher finish canonical layers faster than the generic
    // transform at every small batch (4096 x 4096 whole linear: 20.7 -> 17.5 us at 8 tokens, 27.5 ->
    // 23.5 at 24); tall layers at 32 tokens, and every layer in the tile kernel's range, take whole
    // blocks instead (the tile kernel does not pre-scale a second stage's sums).
    const bool canon_out = (B <= 31 || (B == 32 && m_pad < 8192)) &&
                           glqh_fill_meta_args(&canon_m, n_blocks_m > 1 ? blocks_m : nullptr,
                                               n_blocks_m > 1 ? n_blocks_m : 1, m_pad) &&
                           canon_m.canon == m_pad;
    bool merge2 = has_s2 && canon_out && !(y && y_rht_out) && !tr_plain_plan(m_pad, n_pad, B).tile;
    const float ps2 = merge2 ? (float)inv_resid_scale2 : 1.0f;
    bool two_parts = has_s2;                                   // false once one launch has added both stages

    // Up to four tokens the input transform is folded into the GEMV launch.  A two-stage layer
    // at one token decodes both streams in that one launch (first stage of 4 bits/weight, as the
    // reference's recipes have it; any other repeats the transform in two launches: 2048 x 2048 14.5
    // against 17.4 us; at four tokens 23.9 against 18.0, so two to four tokens transform x once).
    // Everything else transforms x once into scratch and reads it from every workgroup.
    int ks = 0, fi_steps = 0, fi_mode = 0, f16_sums = 0;
    const bool pow2_n = (n_pad & (n_pad - 1)) == 0;
    const bool fi_blocks = n_blocks_n > 1 ? (bn_meta_dev != nullptr && blocks_n != nullptr) : pow2_n;
    // Where folding pays (whole linear, us, folded vs separate transform): one token 8.6 vs 11.1
    // at 2048 x 2048, 12.0 vs 15.6 at 4096 x 4096, 13.9 vs 17.0 at 2048 x 11008, but 21.8 vs 21.0 at
    // 14336 x 4096 and 63 vs 49 at 28672 x 8192 (every workgroup repeats the prologue); the
    // folded form grows by a quarter per extra token and the separate one hardly at all, so two
    // tokens fold only single power-of-two blocks (10.8 vs 11.3, 14.7 vs 15.8; 960 x 960: 12.7 vs
    // 9.4) and three or four tokens never do (2048 x 2048: 13.6 vs 11.5; 8192 x 8192: 38 vs 26).
    // Checked on other model widths (one token, folded / separate, us: 3072 x 3072 10.4 / 11.3, 4096 x 4096
    // 12.1 / 15.5, 8192 x 3072 15.2 / 17.3, 2048 x 6144 10.9 / 12.9, 6144 x 2048 11.5 / 12.6, 1536 x 1536 8.1 / 9.3,
    // 5120 x 5120 17.0 / 15.8 -- the one loss; two tokens: 4096 x 4096 15.0 / 16.1, but 3072 x 8192 19.3 / 16.2 and
    // 6144 x 2048 14.7 / 13.2, hence the size bound on two tokens).
    // One token of a two-stage layer (first stage 4 bits/weight) takes the MFMA form at every height and up to
    // four times the size, both streams in one launch: the alternative is a transform, two decode launches
    // and a finishing one (whole linear, us, one launch / two or three: 4096 x 4096 at 4+2 15.5 / 22.0, 2048 x 2048
    // 9.5 / 14.4, 11008 x 2048 17.7 / 25.0, 512 x 2048 8.7 / 15.0, 128 x 4096 10.9 / 17.0, 14336 x 4096 at 4+4
    // 28.7 / 35.2, 8192 x 8192 32.4 / 41.2, 16384 x 8192 52.3 / 59.2; 28672 x 8192: 94.4 / 95.4 at 4+4 but
    // 108.8 / 98.6 at 4+2, hence the bound).
    const bool fuse2 = has_s2 && B == 1 && R1 == 4 && tr_fuse_stages_enabled();
    const bool fi_pays = tr_fuse_input_enabled() && m_pad * n_pad <= ((int64_t)(fuse2 ? 128 : 32) << 20) &&
                         (B == 1 || (B == 2 && pow2_n && n_pad <= 4096 && m_pad <= 4096));
    if (fi_pays && fi_blocks && (x_dtype == GLQH_F16 || x_dtype == GLQH_BF16) &&
        (fi_mode = tr_fusein_plan(&m_pad, 1, n_pad, B, &fi_steps, &ks, fuse2 ? 1 : GLQH_FUSEIN_MMA_MIN_STRIPS)) != 0 &&
        (!has_s2 || (B == 1 && fi_mode == 2 && (merge2 || fuse2)))) {
        if (n_blocks_n > 1) {
            int64_t sum = 0;
            for (int64_t i = 0; i < n_blocks_n; ++i) {
                GLQH_REQUIRE(blocks_n[i] > 0 && (blocks_n[i] & (blocks_n[i] - 1)) == 0,
                             "fused trellis linear: block size %lld is not a power of two",
                             (long long)blocks_n[i]);
                sum += blocks_n[i];
            }
            GLQH_REQUIRE(sum == n_pad, "fused trellis linear: block sizes sum to %lld, expected %lld",
                         (long long)sum, (long long)n_pad);
        }
        GLQH_REQUIRE(in_features >= 1, "fused trellis linear: in_features must be positive");
        // One token of a 4 + R2 layer: both streams in one launch against one transform of x, the second
        // stage's sums added in registers (4096 x 4096 at 6 bpw: three launches become two).
        if (fuse2) {
            const void *pk1[1] = {packed}, *pk2[1] = {packed2}, *svs[1] = {sv_f16};
            const float rs[1] = {(float)inv_resid_scale2};
            float *pt[1] = {part1};
            if (glqh_launch_trellis_mma_fusein_rvq(pk1, pk2, R2, rs, svs, pt, &m_pad, 1, x, x_dtype, x_stride, n_pad,
                                                   in_features, fi_steps, ks, bn_meta_dev, blocks_n, (int)n_blocks_n, st))
                return 1;
            two_parts = merge2 = false;
        }
        if (merge2) part2 = part1 + (int64_t)ks * B * m_pad;
        const int n_launches = has_s2 ? (two_parts ? 2 : 0) : 1;
        for (int stage = 0; stage < n_launches; ++stage) {
            const void *pk[1] = {stage ? packed2 : packed}, *svs[1] = {sv_f16};
            float *pt[1] = {stage ? part2 : part1};
            const int R = stage ? R2 : R1;
            if (fi_mode == 2) {
                if (glqh_launch_trellis_mma_fusein(pk, svs, pt, &m_pad, 1, R, x, x_dtype, x_stride, B, n_pad,
                                                   in_features, fi_steps, ks, bn_meta_dev, blocks_n, (int)n_blocks_n,
                                                   stage ? ps2 : 1.0f, st))
                    return 1;
            } else if (glqh_launch_trellis_fusein(pk[0], R, x, x_dtype, x_stride, sv_f16, B, m_pad, n_pad,
                                                  in_features, fi_steps, ks, bn_meta_dev, blocks_n, (int)n_blocks_n, pt[0], st))
                return 1;
        }
    } else {
        const tr_plan plan = tr_plain_plan(m_pad, n_pad, B);
        // tile kernel: the transform writes the kernel's blocked operand layout itself where it can
        // (one pass over the activations less, and one repack instead of one per stage)
        const void *x_in = x_rht;
        int rc = -1;
        if (plan.tile)
            rc = glqh_launch_input_rht_blocked(x, x_dtype, x_stride, sv_f16, xb_tile, 2, glqh_trellis_tile_padded_tokens(B),
                                               B, in_features, n_pad, blocks_n, n_blocks_n, st);
        if (rc > 0) return 1;
        if (rc == 0) x_in = nullptr;
        else if (glqh_launch_input_rht(x, x_dtype, x_stride, sv_f16, x_rht, GLQH_F16, B, in_features, n_pad,
                                       bn_meta_dev, blocks_n, n_blocks_n, 0.0f, st))
            return 1;
        // 17 tokens and more of a 4 + R2 layer: the tile kernels decode both streams into one operand,
        // W = fp16(W1 + inv_resid_scale2 * W2) -- the weight of the reference's many-token route -- in tiles of at
        // most 256 tokens: one launch with the products of a single-stage layer instead of two
        const bool tile2 = has_s2 && plan.tile && R1 == 4 && tr_fuse_stages_enabled();
        ks = tile2 ? glqh_trellis_tile_ksplit(m_pad, n_pad, B, 1) : plan.ks;
        if (merge2) part2 = part1 + (int64_t)ks * B * m_pad;
        // Many tokens: the tile kernel rounds its sums to fp16 on the way out, as the reference's
        // many-token route does (its library GEMM of two fp16 matrices returns fp16,
        // glq/csrc/glq_trellis.cu:1322-1334) -- half the bytes between the product and the output
        // transform.  With several K slots (small layers at a few hundred tokens) every slot's sum is
        // rounded and the transform adds them in fp32 (3B-shape layer at 512 tokens: 413 -> 394 us for
        // its seven linears).  GLQ_TRELLIS_F16_SUMS=0 keeps them fp32.
        // (the whole-block output transform, the one that reads fp16 sums, stores 16 bytes at a time: rows of y
        // that do not start on 16 bytes -- out_features not a multiple of 8 -- keep fp32 sums)
        const int64_t y_esz = y_dtype == GLQH_F32 ? 4 : 2;
        f16_sums = plan.tile && ks <= tr_f16_sums_max_slots() && B > 64 && !y_rht_out && y && tr_f16_sums_enabled() &&
                   glqh_output_rht_wide_eligible(B, blocks_m, n_blocks_m, m_pad) && ((uintptr_t)y & 15) == 0 &&
                   ((uintptr_t)su_f16 & 15) == 0 && (y_stride * y_esz) % 16 == 0;
        if (tile2) {
            glqh_range range("dequant_matmul");
            if (glqh_launch_trellis_tile(x_in, xb_tile, B, packed, R1, m_pad, n_pad, part1, 0, f16_sums ? (float)wscale : 1.0f,
                                         0, 0, st, f16_sums, packed2, R2, (float)inv_resid_scale2))
                return 1;
            two_parts = merge2 = false;
        } else if (has_s2 && !plan.tile && R1 == 4 && tr_fuse_stages_enabled()) {
            // up to 16 tokens of a 4 + R2 layer: both streams in one pass over the staged activations
            glqh_range range("dequant_matmul");
            if (glqh_launch_trellis_mma_rvq(x_in, B, packed, packed2, R2, (float)inv_resid_scale2, m_pad, n_pad, plan.S,
                                            plan.ks, part1, st))
                return 1;
            two_parts = merge2 = false;
        } else {
            if (tr_plain_partial(plan, x_in, B, packed, R1, m_pad, n_pad, part1, xb_tile, st, 1.0f, f16_sums, (float)wscale))
                return 1;
            if (has_s2 && tr_plain_partial(plan, x_in, B, packed2, R2, m_pad, n_pad, part2, xb_tile, st, ps2, f16_sums,
                                           (float)(wscale * inv_resid_scale2)))
                return 1;
        }
    }

    const float s1 = (float)wscale, s2 = (float)(wscale * inv_resid_scale2);
    const int ks_all = merge2 ? 2 * ks : ks;
    if (!y) {
        // stop at the RHT-domain product: combine the split-K partials into the caller's rows
        if (glqh_launch_reduce_splits(part1, ks_all, B * m_pad, B, m_pad, s1, y_rht_out, y_rht_stride, 0, st)) return 1;
        if (two_parts && !merge2 &&
            glqh_launch_reduce_splits(part2, ks, B * m_pad, B, m_pad, s2, y_rht_out, y_rht_stride, 1, st))
            return 1;
        return 0;
    }
    if ((!two_parts || merge2) && !y_rht_out && canon_out) {
        // canonical blocks, small batch: the grouped launcher's kernels (a group of one)
        const float *pt[1] = {part1};
        const void *sus[1] = {su_f16};
        void *ys[1] = {y};
        const float sc[1] = {s1};
        return glqh_launch_output_rht_group(pt, sus, ys, sc, &m_pad, &out_features, 1, y_dtype, y_stride, B, ks_all, st);
    }
    glqh_ysrc src = {};
    src.nparts = two_parts ? 2 : 1;
    src.part = part1;
    src.part_sstride = (int64_t)(pb / (f16_sums ? sizeof(f16) : sizeof(float)));
    src.part_kstride = B * m_pad;
    src.ksplit = ks;
    src.part_f16 = f16_sums;
    src.scale[0] = f16_sums ? 1.0f : s1;                       // fp16 sums carry their scales already
    src.scale[1] = f16_sums ? 1.0f : s2;
    src.copy_out = y_rht_out;
    src.copy_stride = y_rht_stride;
    return glqh_launch_output_rht(src, su_f16, y, y_dtype, y_stride, B, out_features, m_pad, bm_meta_dev,
                                  blocks_m, n_blocks_m, 0, 0.0f, st);
}

// ---- the same linear for callers that cannot allocate -----------------------------------
// Scratch of the fused trellis linear (x_rht + split-K partial sums) in the file-scope device
// array defined above glqh_init() instead of a caller-provided workspace.  Nothing in it has to
// start at zero: the decode launch writes every [slot][token][row] partial sum before the
// finishing launch reads it.
extern "C" size_t glqh_noalloc_scratch_bytes(void) { return GLQH_NOALLOC_SCRATCH_BYTES; }

extern "C" int glqh_fused_linear_trellis_3inst_noalloc(
    const void *x, int x_dtype, int64_t x_stride, int64_t B, const void *sv_f16, const void *su_f16,
    const void *packed, int64_t packed_rows, int64_t packed_cols, const void *packed2,
    int64_t packed2_rows, int64_t packed2_cols, const int64_t *blocks_n, int64_t n_blocks_n,
    const int64_t *blocks_m, int64_t n_blocks_m, const glqh_block_meta *bn_meta_dev,
    const glqh_block_meta *bm_meta_dev, double wscale, double inv_resid_scale2, int64_t in_features,
    int64_t out_features, int64_t n_pad, int64_t m_pad, void *y, int y_dtype, int64_t y_stride,
    float *y_rht_out, int64_t y_rht_stride, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(glqh_trellis_kernel_supported(m_pad, n_pad) && B >= 1,
                 "fused trellis linear (no-alloc): needs m %% 32 == 0, k %% 64 == 0 and B >= 1");
    const size_t need = glqh_fused_linear_trellis_workspace_bytes(B, n_pad, m_pad);
    GLQH_REQUIRE(need <= GLQH_NOALLOC_SCRATCH_BYTES,
                 "fused trellis linear (no-alloc): %lld tokens of a %lld x %lld layer need %zu bytes of scratch, "
                 "the built-in buffer holds %zu; use glqh_fused_linear_trellis_3inst with a workspace",
                 (long long)B, (long long)m_pad, (long long)n_pad, need, (size_t)GLQH_NOALLOC_SCRATCH_BYTES);
    void *ws = nullptr;
    if (noalloc_scratch_for_current_device(&ws)) return 1;
    return glqh_fused_linear_trellis_3inst(x, x_dtype, x_stride, B, sv_f16, su_f16, packed, packed_rows, packed_cols,
                                           packed2, packed2_rows, packed2_cols, blocks_n, n_blocks_n, blocks_m,
                                           n_blocks_m, bn_meta_dev, bm_meta_dev, wscale, inv_resid_scale2,
                                           in_features, out_features, n_pad, m_pad, y, y_dtype, y_stride, y_rht_out,
                                           y_rht_stride, ws, GLQH_NOALLOC_SCRATCH_BYTES, stream);
}

// ---- grouped trellis linears -------------------------------------------------------
// Two to four tokens on a large group: every workgroup of the fused-input launch repeats the
// transform of all tokens, and one transform launch + one plain GEMV per layer is faster
// (gate/up 4096 -> 2 x 14336 at four tokens: 63 us folded, 46 us as separate per-layer calls).
static bool tr_group_plain(int64_t total_m_pad, int64_t n_pad, int64_t B) {
    const int64_t w = total_m_pad * n_pad;
    // q/k/v of a 4096-wide model (25M weights): 22.1 / 25.6 / 28.5 us folded at 2 / 3 / 4 tokens,
    // 24.5 / 24.5 / 25.1 us separate; gate/up 2048 -> 2 x 11008 (45M): 19-22 us folded, 25-26 separate
    // Checked on nine other groups (q/k/v and gate/up of 2048- to 8192-wide models, 1-4 tokens, folded /
    // separate, us): one token folds with a gain of 5-8 us up to 50M weights (gate/up 3072 -> 2 x 8192: 18.1 /
    // 24.4) and loses above 96M (4096 -> 2 x 14336: 37.4 / 33.9; 8192 -> 2 x 28672: 103.9 / 92.3; 5120 -> 2 x 13824
    // ties); three and four tokens on q/k/v of a 3072-wide model lose 1-4 us folded (21.7 / 20.5, 24.4 / 20.2),
    // which the rule below does not catch.
    if (!tr_fuse_input_enabled()) return true;
    if (B > 4) return true;                                  // 5..16 tokens: the fused-input launches serve up to four
    if (B == 1) return w > ((int64_t)96 << 20);
    return w > ((int64_t)48 << 20) || (B >= 3 && n_pad >= 4096 && w > ((int64_t)16 << 20));
}
// The grouped call at many tokens: more than 64 tokens, at most four layers.  The K split of a group is at most
// that of a single 128-row layer of the same width (fewer row tiles, more slots).
constexpr int64_t TR_GROUP_MANY_MIN = 64;
// 5..16 tokens: one transform launch per distinct sign vector, one small-batch decode launch per layer under the
// K plan of the tallest, one finishing launch for all layers (no K-slot sum launches, no shared fp32 buffer)
constexpr int64_t TR_GROUP_SMALL_MAX = 16;
constexpr int TR_GROUP_MANY_MAX = 4;
constexpr int64_t TT_GROUP_ROWS_FLOOR = 128;

static int tr_group_plan(const int64_t *m_pads, int n_shards, int64_t n_pad, int64_t B, int *steps, int *ks) {
    int64_t total = 0;
    for (int i = 0; i < n_shards; ++i) total += m_pads[i];
    (void)total;
    return tr_fusein_plan(m_pads, n_shards, n_pad, B, steps, ks);
}

extern "C" size_t glqh_fused_linear_trellis_group_workspace_bytes(int64_t B, int64_t n_pad, int64_t total_m_pad,
                                                                  int n_shards) {
    if (B > TR_GROUP_MANY_MIN && n_shards >= 1 && n_shards <= TR_GROUP_MANY_MAX && total_m_pad >= 32 && n_pad >= 64) {
        // many tokens: every layer's blocked activations, a row-major copy for transforms that cannot write
        // them, and the partial sums of the largest K split a group of these rows can get (fp32)
        glqh_init();
        const int64_t one[1] = {TT_GROUP_ROWS_FLOOR};
        const int ks = glqh_trellis_tile_group_ksplit(one, 1, n_pad, B);
        return (size_t)n_shards * (256 + align256(glqh_trellis_tile_xb_bytes(n_pad, B))) +
               align256((size_t)B * n_pad * sizeof(f16)) + align256((size_t)ks * B * total_m_pad * sizeof(float));
    }
    if (B < 1 || B > TR_GROUP_MANY_MIN || n_shards < 1 || n_shards > GLQH_MAX_SHARDS || total_m_pad < 32 || n_pad < 64)
        return 0;
    glqh_init();
    if (B > TR_GROUP_SMALL_MAX) {
        // 17..64 tokens: blocked and row-major activations and every layer's sums under its own K plan, bounded by
        // the plan of a 128-row layer (fewer row tiles, more slots)
        const int ks1 = glqh_trellis_tile_ksplit(TT_GROUP_ROWS_FLOOR, n_pad, B), ks2 = glqh_trellis_tile_ksplit(TT_GROUP_ROWS_FLOOR, n_pad, B, 1);
        const int ksb = ks1 > ks2 ? ks1 : ks2;                 // (single-stage and stacked layers)
        return (size_t)n_shards * (256 + align256(glqh_trellis_tile_xb_bytes(n_pad, B))) +
               align256((size_t)B * n_pad * sizeof(f16)) + align256((size_t)ksb * B * total_m_pad * sizeof(float));
    }
    if (B > 4) {
        // x_rht and the partial sums under the K plan of the tallest layer, which has at least total / n_shards
        // rows (the plan's slot count does not grow with the rows)
        int S = 0, ksb = 0;
        const int64_t mmin = total_m_pad / n_shards / 32 * 32;
        glqh_trellis_mma_plan(mmin < 32 ? 32 : mmin, n_pad, &S, &ksb);
        return (size_t)n_shards * (256 + align256((size_t)B * n_pad * sizeof(f16))) +
               align256((size_t)ksb * B * total_m_pad * sizeof(float));
    }
    int steps = 0, ks = 0;
    // upper bound over how the rows may be split among the layers: the most workgroups (and
    // so the fewest K slots) arise from many short layers, the most slots from one tall layer
    int ks2 = 0;
    if (!glqh_trellis_fusein_plan(total_m_pad, n_pad, B, &steps, &ks)) return 0;
    if (glqh_trellis_mma_fusein_plan((total_m_pad + 63) / 64, n_pad, B, &steps, &ks2) && ks2 > ks) ks = ks2;
    // the separate-transform route of large groups: slots of the plain plan (at most 64) and x_rht
    size_t plain = 0;
    if (tr_group_plain(total_m_pad, n_pad, B))
        plain = (size_t)n_shards * align256((size_t)B * n_pad * sizeof(f16)) + align256((size_t)64 * B * total_m_pad * sizeof(float));
    const size_t fused = align256((size_t)ks * B * total_m_pad * sizeof(float));
    // (2..4 tokens of stacked layers, glqh_fused_linear_trellis_3inst_group_rvq2: x_rht and the sums under the K
    // plan of the tallest layer, which has at least total / n_shards rows)
    size_t stacked = 0;
    if (B > 1) {
        int S = 0, ksb = 0;
        const int64_t mmin = total_m_pad / n_shards / 32 * 32;
        glqh_trellis_mma_plan(mmin < 32 ? 32 : mmin, n_pad, &S, &ksb);
        stacked = (size_t)n_shards * align256((size_t)B * n_pad * sizeof(f16)) +
                  align256((size_t)ksb * B * total_m_pad * sizeof(float));
    }
    const size_t most = plain > fused ? plain : fused;
    return (size_t)n_shards * 256 + (stacked > most ? stacked : most);
}

// Decode launch of a group: checks, K plan, partial-sum layout in ws.  On return parts[i] holds
// layer i's [slot][token][row] fp32 partial sums and *ks_out the slot count.
// Layers that read the same activations, many tokens (prefill of fused q/k/v, gate/up): per distinct sign vector
// one input transform straight into the tile kernel's layout, ONE launch of the tile kernel over the row tiles of
// all layers (small layers do not fill the chip one by one: 512 tokens x (2048 -> 2048 + 512 + 512): 16 + 4 + 4
// row tiles), then every layer's output transform from fp16 sums.
static int tr_group_many(const void *x, int x_dtype, int64_t x_stride, int64_t B, const glqh_trellis_shard *shards,
                         int n_shards, const int64_t *blocks_n, int64_t n_blocks_n, const glqh_block_meta *bn_meta_dev,
                         int64_t in_features, int64_t n_pad, int y_dtype, int64_t y_stride, void *ws, size_t ws_bytes,
                         hipStream_t st) {
    GLQH_REQUIRE(x && shards && ws, "trellis group: null pointer");
    GLQH_REQUIRE(n_shards >= 1 && n_shards <= TR_GROUP_MANY_MAX, "trellis group: %d layers at %lld tokens (1..%d)",
                 n_shards, (long long)B, TR_GROUP_MANY_MAX);
    GLQH_REQUIRE(B <= 65535, "trellis group: B=%lld out of range", (long long)B);
    GLQH_REQUIRE(x_dtype == GLQH_F16 || x_dtype == GLQH_BF16, "trellis group: x must be f16 or bf16");
    GLQH_REQUIRE(in_features >= 1 && in_features <= n_pad && n_pad % 64 == 0, "trellis group: bad in_features / n_pad");
    GLQH_REQUIRE(n_blocks_n > 1 ? (bn_meta_dev != nullptr && blocks_n != nullptr) : (n_pad & (n_pad - 1)) == 0,
                 "trellis group: input block sizes missing");
    int R = 0;
    int64_t total = 0, m_pads[TR_GROUP_MANY_MAX];
    const void *packed[TR_GROUP_MANY_MAX];
    for (int i = 0; i < n_shards; ++i) {
        const glqh_trellis_shard &sh = shards[i];
        GLQH_REQUIRE(sh.sv_f16 && sh.packed && sh.su_f16 && sh.y, "trellis group: null pointer in shard %d", i);
        int Ri;
        if (tr_bits_from_packed(sh.packed_cols, 0, &Ri) || tr_check_shape(sh.m_pad, n_pad, sh.packed_rows)) return 1;
        GLQH_REQUIRE(i == 0 || Ri == R, "trellis group: shards of %d and %d bits/weight cannot share a launch", R, Ri);
        R = Ri;
        GLQH_REQUIRE(sh.out_features >= 1 && sh.out_features <= sh.m_pad, "trellis group: out_features exceeds m_pad");
        m_pads[i] = sh.m_pad;
        packed[i] = sh.packed;
        total += sh.m_pad;
    }
    const int ks = glqh_trellis_tile_group_ksplit(m_pads, n_shards, n_pad, B);
    const size_t xb_one = align256(glqh_trellis_tile_xb_bytes(n_pad, B));
    const size_t rows = align256((size_t)B * n_pad * sizeof(f16));
    const size_t need = (size_t)n_shards * xb_one + rows + align256((size_t)ks * B * total * sizeof(float));
    GLQH_REQUIRE(ws_bytes >= need, "trellis group: workspace of %zu bytes needed, got %zu", need, ws_bytes);
    char *base = (char *)ws;
    f16 *x_rows = (f16 *)(base + (size_t)n_shards * xb_one);
    char *pbase = base + (size_t)n_shards * xb_one + rows;
    const int64_t Mp = glqh_trellis_tile_padded_tokens(B);
    const void *xb[TR_GROUP_MANY_MAX];
    float *parts[TR_GROUP_MANY_MAX];
    // fp16 sums need the whole-block output kernels for every layer (canonical blocks of at most 8192 rows)
    bool f16_sums = tr_f16_sums_enabled() && ks <= tr_f16_sums_max_slots();
    for (int i = 0; i < n_shards && f16_sums; ++i) {
        int64_t top = 1;
        while (top * 2 <= m_pads[i]) top *= 2;
        if (top > 8192 || m_pads[i] % 8 != 0) f16_sums = false;
        // and rows of y that start on 16 bytes (the whole-block transform stores 16 bytes at a time)
        const int64_t ys = y_stride > 0 ? y_stride : shards[i].out_features, y_esz = y_dtype == GLQH_F32 ? 4 : 2;
        if (((uintptr_t)shards[i].y & 15) != 0 || ((uintptr_t)shards[i].su_f16 & 15) != 0 || (ys * y_esz) % 16 != 0)
            f16_sums = false;
    }
    const size_t esz = f16_sums ? sizeof(f16) : sizeof(float);
    size_t poff = 0;
    // all distinct sign vectors in one transform launch where it applies (layer i's activations in buffer i)
    int all = -1;
    {
        const void *dsv[GLQH_MAX_SHARDS];
        void *dout[GLQH_MAX_SHARDS];
        int nd = 0;
        for (int i = 0; i < n_shards; ++i) {
            int j = 0;
            while (j < nd && dsv[j] != shards[i].sv_f16) ++j;
            if (j == nd) {
                dsv[nd] = shards[i].sv_f16;
                dout[nd] = base + (size_t)i * xb_one;
                ++nd;
            }
        }
        if (nd > 1)
            all = glqh_launch_input_rht_blocked_multi(x, x_dtype, x_stride, dsv, dout, nd, Mp, B, in_features, n_pad, blocks_n,
                                                      n_blocks_n, st);
        if (all > 0) return 1;
    }
    for (int i = 0; i < n_shards; ++i) {
        // layers quantized with the same sign vector share one transform of x
        int same = -1;
        for (int j = 0; j < i; ++j)
            if (shards[j].sv_f16 == shards[i].sv_f16) { same = j; break; }
        if (same >= 0) {
            xb[i] = xb[same];
        } else if (all == 0) {
            xb[i] = base + (size_t)i * xb_one;
        } else {
            void *dst = base + (size_t)i * xb_one;
            const int rc = glqh_launch_input_rht_blocked(x, x_dtype, x_stride, shards[i].sv_f16, dst, 2, Mp, B, in_features,
                                                         n_pad, blocks_n, n_blocks_n, st);
            if (rc > 0) return 1;
            if (rc < 0) {                                        // rows first, then repacked
                if (glqh_launch_input_rht(x, x_dtype, x_stride, shards[i].sv_f16, x_rows, GLQH_F16, B, in_features, n_pad,
                                          bn_meta_dev, blocks_n, n_blocks_n, 0.0f, st) ||
                    glqh_launch_trellis_pack(x_rows, dst, B, n_pad, st))
                    return 1;
            }
            xb[i] = dst;
        }
        parts[i] = (float *)(pbase + poff);
        poff += align256((size_t)ks * B * m_pads[i] * esz);
    }
    float wscales[TR_GROUP_MANY_MAX];                          // fp16 sums carry the layer's scale already
    for (int i = 0; i < n_shards; ++i) wscales[i] = (float)shards[i].wscale;
    if (glqh_launch_trellis_tile_group(xb, B, packed, R, m_pads, n_shards, n_pad, parts, f16_sums ? 1 : 0, st, wscales)) return 1;
    for (int i = 0; i < n_shards; ++i) {
        const glqh_trellis_shard &sh = shards[i];
        glqh_ysrc src = {};
        src.nparts = 1;
        src.part = parts[i];
        src.part_kstride = B * sh.m_pad;
        src.ksplit = ks;
        src.part_f16 = f16_sums;
        src.scale[0] = f16_sums ? 1.0f : (float)sh.wscale;
        const int64_t ys = y_stride > 0 ? y_stride : sh.out_features;   // y_stride 0: every layer's rows packed
        int rc = glqh_launch_output_rht_canon_wide(src, sh.su_f16, sh.y, y_dtype, ys, B, sh.out_features, sh.m_pad, st);
        if (rc > 0) return 1;
        if (rc < 0) {
            GLQH_REQUIRE(!f16_sums, "trellis group: layer %d: output blocks not served by the whole-block transform", i);
            // canonical blocks above 8192 rows: the sliced kernels of the grouped launcher
            const float *pt[1] = {parts[i]};
            const void *sus[1] = {sh.su_f16};
            const float sc[1] = {(float)sh.wscale};
            void *yl[1] = {sh.y};
            if (glqh_launch_output_rht_group(pt, sus, yl, sc, &sh.m_pad, &sh.out_features, 1, y_dtype, ys, B, ks, st))
                return 1;
        }
    }
    return 0;
}

struct tr_group_ctx {
    int R, ks, fi_mode;
    int ks_layer[GLQH_MAX_SHARDS];                             // 17..64 tokens: every layer's own slot count (ks = 0 when they differ)
    int64_t m_pads[GLQH_MAX_SHARDS], outs[GLQH_MAX_SHARDS];
    const void *su[GLQH_MAX_SHARDS];
    void *ys[GLQH_MAX_SHARDS];
    float scale[GLQH_MAX_SHARDS];
    float *parts[GLQH_MAX_SHARDS];
};

// x under every distinct sign vector of a group of layers, fp16 rows at ws + j * xb_one (few tokens): one launch for
// all of them where the small-batch kernel serves the call, one per sign vector otherwise.  x_of[i] = layer i's rows.
static int tr_group_transform(const void *x, int x_dtype, int64_t x_stride, int64_t B, const void *const sv[], int n_shards,
                              const int64_t *blocks_n, int64_t n_blocks_n, const glqh_block_meta *bn_meta_dev,
                              int64_t in_features, int64_t n_pad, void *ws, size_t xb_one, const f16 *x_of[],
                              hipStream_t st) {
    const void *dsv[GLQH_MAX_SHARDS];
    void *dout[GLQH_MAX_SHARDS];
    int nd = 0;
    for (int i = 0; i < n_shards; ++i) {
        int j = 0;
        while (j < nd && dsv[j] != sv[i]) ++j;
        if (j == nd) {
            dsv[nd] = sv[i];
            dout[nd] = (char *)ws + (size_t)nd * xb_one;
            ++nd;
        }
        x_of[i] = (const f16 *)dout[j];
    }
    int rc = nd > 1 ? glqh_launch_input_rht_multi(x, x_dtype, x_stride, dsv, dout, nd, B, in_features, n_pad, bn_meta_dev,
                                                  blocks_n, n_blocks_n, st)
                    : -1;
    if (rc > 0) return 1;
    if (rc == 0) return 0;
    for (int j = 0; j < nd; ++j)
        if (glqh_launch_input_rht(x, x_dtype, x_stride, dsv[j], dout[j], GLQH_F16, B, in_features, n_pad, bn_meta_dev,
                                  blocks_n, n_blocks_n, 0.0f, st))
            return 1;
    return 0;
}

// 17..64 tokens: x under every distinct sign vector of a group straight into the tile kernels' layout, buffer j at
// ws + j * xbb, in one launch.  0: done, xb_of[i] = layer i's buffer; -1: not applicable, nothing launched.
static int tr_group_transform_blocked(const void *x, int x_dtype, int64_t x_stride, int64_t B, const void *const sv[],
                                      int n_shards, const int64_t *blocks_n, int64_t n_blocks_n, int64_t in_features,
                                      int64_t n_pad, void *ws, size_t xbb, void *xb_of[], hipStream_t st) {
    const void *dsv[GLQH_MAX_SHARDS];
    void *dout[GLQH_MAX_SHARDS];
    int nd = 0;
    for (int i = 0; i < n_shards; ++i) {
        int j = 0;
        while (j < nd && dsv[j] != sv[i]) ++j;
        if (j == nd) {
            dsv[nd] = sv[i];
            dout[nd] = (char *)ws + (size_t)nd * xbb;
            ++nd;
        }
        xb_of[i] = dout[j];
    }
    if (nd < 2) return -1;
    return glqh_launch_input_rht_blocked_multi(x, x_dtype, x_stride, dsv, dout, nd, glqh_trellis_tile_padded_tokens(B), B,
                                               in_features, n_pad, blocks_n, n_blocks_n, st);
}

// One finishing launch for all layers of a group; at 17..64 tokens, where every layer has its own K plan, one per
// layer when their slot counts differ.
static int tr_group_finish(const tr_group_ctx &c, int n_shards, int64_t B, int y_dtype, int64_t y_stride, hipStream_t st) {
    if (B > TR_GROUP_SMALL_MAX && c.ks == 0) {
        for (int i = 0; i < n_shards; ++i) {
            glqh_ysrc src = {};
            src.nparts = 1;
            src.part = c.parts[i];
            src.part_kstride = B * c.m_pads[i];
            src.ksplit = c.ks_layer[i];
            src.scale[0] = c.scale[i];
            if (glqh_launch_output_rht_canon_wide(src, c.su[i], c.ys[i], y_dtype, y_stride, B, c.outs[i], c.m_pads[i], st) != 0) {
                const float *pt[1] = {c.parts[i]};
                if (glqh_launch_output_rht_group(pt, &c.su[i], &c.ys[i], &c.scale[i], &c.m_pads[i], &c.outs[i], 1, y_dtype,
                                                 y_stride, B, c.ks_layer[i], st))
                    return 1;
            }
        }
        return 0;
    }
    return glqh_launch_output_rht_group(c.parts, c.su, c.ys, c.scale, c.m_pads, c.outs, n_shards, y_dtype, y_stride,
                                        B, c.ks, st);
}

static int tr_group_decode(const void *x, int x_dtype, int64_t x_stride, int64_t B,
                           const glqh_trellis_shard *shards, int n_shards, const int64_t *blocks_n,
                           int64_t n_blocks_n, const glqh_block_meta *bn_meta_dev, int64_t in_features,
                           int64_t n_pad, void *ws, size_t ws_bytes, hipStream_t st, tr_group_ctx *c) {
    GLQH_REQUIRE(x && shards, "trellis group: null pointer");
    GLQH_REQUIRE(n_shards >= 1 && n_shards <= GLQH_MAX_SHARDS, "trellis group: %d shards (1..%d)", n_shards,
                 GLQH_MAX_SHARDS);
    GLQH_REQUIRE(B >= 1 && B <= TR_GROUP_MANY_MIN, "trellis group: B=%lld", (long long)B);
    GLQH_REQUIRE(x_dtype == GLQH_F16 || x_dtype == GLQH_BF16, "trellis group: x must be f16 or bf16");
    GLQH_REQUIRE(in_features >= 1 && in_features <= n_pad, "trellis group: in_features exceeds n_pad");
    const bool pow2_n = (n_pad & (n_pad - 1)) == 0;
    GLQH_REQUIRE(n_blocks_n > 1 ? (bn_meta_dev != nullptr && blocks_n != nullptr) : pow2_n,
                 "trellis group: input block sizes missing");
    if (n_blocks_n > 1) {
        int64_t sum = 0;
        for (int64_t i = 0; i < n_blocks_n; ++i) {
            GLQH_REQUIRE(blocks_n[i] > 0 && (blocks_n[i] & (blocks_n[i] - 1)) == 0,
                         "trellis group: block size %lld is not a power of two", (long long)blocks_n[i]);
            sum += blocks_n[i];
        }
        GLQH_REQUIRE(sum == n_pad, "trellis group: block sizes sum to %lld, expected %lld", (long long)sum,
                     (long long)n_pad);
    }
    int R = 0;
    const void *packed[GLQH_MAX_SHARDS], *sv[GLQH_MAX_SHARDS];
    int64_t total = 0;
    for (int i = 0; i < n_shards; ++i) {
        const glqh_trellis_shard &sh = shards[i];
        GLQH_REQUIRE(sh.sv_f16 && sh.packed, "trellis group: null pointer in shard %d", i);
        GLQH_REQUIRE((sh.y != nullptr) == (shards[0].y != nullptr) && (!sh.y || sh.su_f16),
                     "trellis group: shard %d: outputs must be given for all shards or for none", i);
        int Ri;
        if (tr_bits_from_packed(sh.packed_cols, 0, &Ri) || tr_check_shape(sh.m_pad, n_pad, sh.packed_rows)) return 1;
        GLQH_REQUIRE(i == 0 || Ri == R, "trellis group: shards of %d and %d bits/weight cannot share a launch", R, Ri);
        GLQH_REQUIRE(Ri >= 2, "trellis group: the grouped launch serves 2-4 bits/weight");
        R = Ri;
        GLQH_REQUIRE(sh.out_features >= 1 && sh.out_features <= sh.m_pad, "trellis group: out_features exceeds m_pad");
        c->m_pads[i] = sh.m_pad; c->outs[i] = sh.out_features;
        packed[i] = sh.packed; sv[i] = sh.sv_f16; c->su[i] = sh.su_f16; c->ys[i] = sh.y;
        c->scale[i] = (float)sh.wscale;
        total += sh.m_pad;
    }
    int steps = 0, ks = 0;
    if (B > TR_GROUP_SMALL_MAX) {
        // 17..64 tokens: one transform launch per distinct sign vector, straight into the tile kernel's layout where
        // it can, one launch of the small-tile kernel per layer (its own K plan), sums left for the finishing launch
        const size_t xbb = align256(glqh_trellis_tile_xb_bytes(n_pad, B)), xrm = align256((size_t)B * n_pad * sizeof(f16));
        size_t sums = 0;
        bool same = true;
        for (int i = 0; i < n_shards; ++i) {
            c->ks_layer[i] = glqh_trellis_tile_ksplit(c->m_pads[i], n_pad, B);
            same = same && c->ks_layer[i] == c->ks_layer[0];
            sums += align256((size_t)c->ks_layer[i] * B * c->m_pads[i] * sizeof(float));
        }
        const size_t need = (size_t)n_shards * xbb + xrm + sums;
        GLQH_REQUIRE(ws && ws_bytes >= need, "trellis group: workspace of %zu bytes needed, got %zu", need, ws_bytes);
        void *xb = ws;
        f16 *x_rht = (f16 *)((char *)ws + (size_t)n_shards * xbb);
        char *p = (char *)ws + (size_t)n_shards * xbb + xrm;
        c->R = R; c->ks = same ? c->ks_layer[0] : 0; c->fi_mode = 0;
        void *xb_of[GLQH_MAX_SHARDS];
        const int all = tr_group_transform_blocked(x, x_dtype, x_stride, B, sv, n_shards, blocks_n, n_blocks_n, in_features,
                                                   n_pad, ws, xbb, xb_of, st);
        if (all > 0) return 1;
        int blocked = -1;
        for (int i = 0; i < n_shards; ++i) {
            if (all == 0) {                                    // every sign vector's activations are in place
                c->parts[i] = (float *)p;
                p += align256((size_t)c->ks_layer[i] * B * c->m_pads[i] * sizeof(float));
                glqh_range range("dequant_matmul");
                if (glqh_launch_trellis_tile(nullptr, xb_of[i], B, packed[i], R, c->m_pads[i], n_pad, c->parts[i], 0, 1.0f, 0,
                                             0, st, 0))
                    return 1;
                continue;
            }
            if (i == 0 || sv[i] != sv[i - 1]) {
                blocked = glqh_launch_input_rht_blocked(x, x_dtype, x_stride, sv[i], xb, 2, glqh_trellis_tile_padded_tokens(B),
                                                        B, in_features, n_pad, blocks_n, n_blocks_n, st);
                if (blocked > 0) return 1;
                if (blocked != 0 && glqh_launch_input_rht(x, x_dtype, x_stride, sv[i], x_rht, GLQH_F16, B, in_features, n_pad,
                                                          bn_meta_dev, blocks_n, n_blocks_n, 0.0f, st))
                    return 1;
            }
            c->parts[i] = (float *)p;
            p += align256((size_t)c->ks_layer[i] * B * c->m_pads[i] * sizeof(float));
            glqh_range range("dequant_matmul");
            if (glqh_launch_trellis_tile(blocked == 0 ? nullptr : x_rht, xb, B, packed[i], R, c->m_pads[i], n_pad, c->parts[i],
                                         0, 1.0f, 0, 0, st, 0))
                return 1;
        }
        return 0;
    }
    if (tr_group_plain(total, n_pad, B)) {
        // one K plan for all layers (that of the tallest), so that the finishing launch sees one slot count
        int64_t mmax = 0;
        for (int i = 0; i < n_shards; ++i) mmax = c->m_pads[i] > mmax ? c->m_pads[i] : mmax;
        int S = 0;
        glqh_trellis_mma_plan(mmax, n_pad, &S, &ks);
        const size_t xb = align256((size_t)B * n_pad * sizeof(f16));
        const size_t need = (size_t)n_shards * xb + align256((size_t)ks * B * total * sizeof(float));
        GLQH_REQUIRE(ws && ws_bytes >= need, "trellis group: workspace of %zu bytes needed, got %zu", need, ws_bytes);
        float *p = (float *)((char *)ws + (size_t)n_shards * xb);
        c->R = R; c->ks = ks; c->fi_mode = 0;
        // layers quantized with the same sign vector share one transform of x
        const f16 *x_of[GLQH_MAX_SHARDS];
        if (tr_group_transform(x, x_dtype, x_stride, B, sv, n_shards, blocks_n, n_blocks_n, bn_meta_dev, in_features, n_pad,
                               ws, xb, x_of, st))
            return 1;
        for (int i = 0; i < n_shards; ++i) {
            c->parts[i] = p;
            p += (size_t)ks * B * c->m_pads[i];
            if (glqh_launch_trellis_mma(x_of[i], B, packed[i], R, c->m_pads[i], n_pad, S, ks, c->parts[i], 0, 1.0f, 0, 0, st))
                return 1;
        }
        return 0;
    }
    const int fi_mode = tr_group_plan(c->m_pads, n_shards, n_pad, B, &steps, &ks);
    GLQH_REQUIRE(fi_mode != 0, "trellis group: shape not eligible");
    const size_t need = align256((size_t)ks * B * total * sizeof(float));
    GLQH_REQUIRE(ws && ws_bytes >= need, "trellis group: workspace of %zu bytes needed, got %zu", need, ws_bytes);
    float *p = (float *)ws;
    for (int i = 0; i < n_shards; ++i) {
        c->parts[i] = p;
        p += (size_t)ks * B * c->m_pads[i];
    }
    c->R = R; c->ks = ks; c->fi_mode = fi_mode;
    if (fi_mode == 2)
        return glqh_launch_trellis_mma_fusein(packed, sv, c->parts, c->m_pads, n_shards, R, x, x_dtype, x_stride, B,
                                              n_pad, in_features, steps, ks, bn_meta_dev, blocks_n, (int)n_blocks_n, 1.0f, st);
    return glqh_launch_trellis_fusein_group(packed, sv, c->parts, c->m_pads, n_shards, R, x, x_dtype, x_stride, B,
                                            n_pad, in_features, steps, ks, bn_meta_dev, blocks_n, (int)n_blocks_n, st);
}

extern "C" int glqh_fused_linear_trellis_3inst_group(const void *x, int x_dtype, int64_t x_stride, int64_t B,
                                                     const glqh_trellis_shard *shards, int n_shards,
                                                     const int64_t *blocks_n, int64_t n_blocks_n,
                                                     const glqh_block_meta *bn_meta_dev, int64_t in_features,
                                                     int64_t n_pad, int y_dtype, int64_t y_stride, void *ws,
                                                     size_t ws_bytes, void *stream) {
    GLQH_INIT();
    hipStream_t st = (hipStream_t)stream;
    GLQH_REQUIRE(y_stride > 0 || B > TR_GROUP_MANY_MIN, "trellis group: y_stride 0 (packed rows per layer) needs more than %lld tokens",
                 (long long)TR_GROUP_MANY_MIN);
    if (B > TR_GROUP_MANY_MIN)
        return tr_group_many(x, x_dtype, x_stride, B, shards, n_shards, blocks_n, n_blocks_n, bn_meta_dev, in_features,
                             n_pad, y_dtype, y_stride, ws, ws_bytes, st);
    tr_group_ctx c;
    if (tr_group_decode(x, x_dtype, x_stride, B, shards, n_shards, blocks_n, n_blocks_n, bn_meta_dev, in_features,
                        n_pad, ws, ws_bytes, st, &c))
        return 1;
    if (!shards[0].y) return 0;                                // decode launch only: partial sums stay in ws
    return tr_group_finish(c, n_shards, B, y_dtype, y_stride, st);
}

// The same for stacked (two-stage) layers at one token: every layer's two streams decoded by one launch
// (first stage 4 bits/weight, the second stages of one rate), finished like single-stage layers.
extern "C" int glqh_fused_linear_trellis_3inst_group_rvq2(const void *x, int x_dtype, int64_t x_stride, int64_t B,
                                                          const glqh_trellis_shard *shards,
                                                          const glqh_trellis_stage2 *stage2, int n_shards,
                                                          const int64_t *blocks_n, int64_t n_blocks_n,
                                                          const glqh_block_meta *bn_meta_dev, int64_t in_features,
                                                          int64_t n_pad, int y_dtype, int64_t y_stride, void *ws,
                                                          size_t ws_bytes, void *stream) {
    GLQH_INIT();
    hipStream_t st = (hipStream_t)stream;
    GLQH_REQUIRE(x && shards && stage2, "trellis two-stage group: null pointer");
    GLQH_REQUIRE(n_shards >= 1 && n_shards <= GLQH_MAX_SHARDS, "trellis two-stage group: %d shards (1..%d)", n_shards,
                 GLQH_MAX_SHARDS);
    GLQH_REQUIRE(B >= 1 && B <= TR_GROUP_MANY_MIN, "trellis two-stage group: B=%lld (the grouped two-stage call serves 1..64 tokens)",
                 (long long)B);
    GLQH_REQUIRE(x_dtype == GLQH_F16 || x_dtype == GLQH_BF16, "trellis two-stage group: x must be f16 or bf16");
    GLQH_REQUIRE(in_features >= 1 && in_features <= n_pad, "trellis two-stage group: in_features exceeds n_pad");
    GLQH_REQUIRE(y_stride > 0, "trellis two-stage group: y_stride must be positive");
    const bool pow2_n = (n_pad & (n_pad - 1)) == 0;
    GLQH_REQUIRE(n_blocks_n > 1 ? (bn_meta_dev != nullptr && blocks_n != nullptr) : pow2_n,
                 "trellis two-stage group: input block sizes missing");
    if (n_blocks_n > 1) {
        int64_t sum = 0;
        for (int64_t i = 0; i < n_blocks_n; ++i) {
            GLQH_REQUIRE(blocks_n[i] > 0 && (blocks_n[i] & (blocks_n[i] - 1)) == 0,
                         "trellis two-stage group: block size %lld is not a power of two", (long long)blocks_n[i]);
            sum += blocks_n[i];
        }
        GLQH_REQUIRE(sum == n_pad, "trellis two-stage group: block sizes sum to %lld, expected %lld", (long long)sum,
                     (long long)n_pad);
    }
    tr_group_ctx c;
    const void *packed[GLQH_MAX_SHARDS], *packed2[GLQH_MAX_SHARDS], *sv[GLQH_MAX_SHARDS];
    float rs2[GLQH_MAX_SHARDS];
    int R2 = 0;
    int64_t total = 0;
    for (int i = 0; i < n_shards; ++i) {
        const glqh_trellis_shard &sh = shards[i];
        const glqh_trellis_stage2 &s2 = stage2[i];
        GLQH_REQUIRE(sh.sv_f16 && sh.packed && sh.su_f16 && sh.y && s2.packed2, "trellis two-stage group: null pointer in shard %d", i);
        GLQH_REQUIRE(s2.inv_resid_scale2 != 0.0, "trellis two-stage group: shard %d has a second stream but inv_resid_scale2 = 0", i);
        int R1, Ri;
        if (tr_bits_from_packed(sh.packed_cols, 0, &R1) || tr_check_shape(sh.m_pad, n_pad, sh.packed_rows)) return 1;
        if (tr_bits_from_packed(s2.packed2_cols, 1, &Ri) || tr_check_shape(sh.m_pad, n_pad, s2.packed2_rows)) return 1;
        GLQH_REQUIRE(R1 == 4, "trellis two-stage group: first stages of 4 bits/weight, shard %d has %d", i, R1);
        GLQH_REQUIRE(i == 0 || Ri == R2, "trellis two-stage group: second stages of %d and %d bits/weight cannot share a launch",
                     R2, Ri);
        R2 = Ri;
        GLQH_REQUIRE(sh.out_features >= 1 && sh.out_features <= sh.m_pad, "trellis two-stage group: out_features exceeds m_pad");
        c.m_pads[i] = sh.m_pad; c.outs[i] = sh.out_features;
        packed[i] = sh.packed; packed2[i] = s2.packed2; rs2[i] = (float)s2.inv_resid_scale2;
        sv[i] = sh.sv_f16; c.su[i] = sh.su_f16; c.ys[i] = sh.y;
        c.scale[i] = (float)sh.wscale;
        total += sh.m_pad;
    }
    int steps = 0, ks = 0;
    if (B > TR_GROUP_SMALL_MAX) {
        // 17..64 tokens: one transform launch per distinct sign vector, one launch of the small-tile kernel per layer,
        // which decodes both streams into one operand, finishing as for single-stage layers
        GLQH_REQUIRE(tr_fuse_stages_enabled(), "trellis two-stage group: more than 16 tokens need both streams in one operand");
        const size_t xbb = align256(glqh_trellis_tile_xb_bytes(n_pad, B)), xrm = align256((size_t)B * n_pad * sizeof(f16));
        size_t sums = 0;
        bool same = true;
        for (int i = 0; i < n_shards; ++i) {
            c.ks_layer[i] = glqh_trellis_tile_ksplit(c.m_pads[i], n_pad, B, 1);
            same = same && c.ks_layer[i] == c.ks_layer[0];
            sums += align256((size_t)c.ks_layer[i] * B * c.m_pads[i] * sizeof(float));
        }
        const size_t need = (size_t)n_shards * xbb + xrm + sums;
        GLQH_REQUIRE(ws && ws_bytes >= need, "trellis two-stage group: workspace of %zu bytes needed, got %zu", need, ws_bytes);
        void *xb = ws;
        f16 *x_rht = (f16 *)((char *)ws + (size_t)n_shards * xbb);
        char *p = (char *)ws + (size_t)n_shards * xbb + xrm;
        c.ks = same ? c.ks_layer[0] : 0;
        void *xb_of[GLQH_MAX_SHARDS];
        const int all = tr_group_transform_blocked(x, x_dtype, x_stride, B, sv, n_shards, blocks_n, n_blocks_n, in_features,
                                                   n_pad, ws, xbb, xb_of, st);
        if (all > 0) return 1;
        int blocked = -1;
        for (int i = 0; i < n_shards; ++i) {
            if (all == 0) {                                    // every sign vector's activations are in place
                c.parts[i] = (float *)p;
                p += align256((size_t)c.ks_layer[i] * B * c.m_pads[i] * sizeof(float));
                glqh_range range("dequant_matmul");
                if (glqh_launch_trellis_tile(nullptr, xb_of[i], B, packed[i], 4, c.m_pads[i], n_pad, c.parts[i], 0, 1.0f, 0, 0,
                                             st, 0, packed2[i], R2, rs2[i]))
                    return 1;
                continue;
            }
            if (i == 0 || sv[i] != sv[i - 1]) {
                blocked = glqh_launch_input_rht_blocked(x, x_dtype, x_stride, sv[i], xb, 2, glqh_trellis_tile_padded_tokens(B),
                                                        B, in_features, n_pad, blocks_n, n_blocks_n, st);
                if (blocked > 0) return 1;
                if (blocked != 0 && glqh_launch_input_rht(x, x_dtype, x_stride, sv[i], x_rht, GLQH_F16, B, in_features, n_pad,
                                                          bn_meta_dev, blocks_n, n_blocks_n, 0.0f, st))
                    return 1;
            }
            c.parts[i] = (float *)p;
            p += align256((size_t)c.ks_layer[i] * B * c.m_pads[i] * sizeof(float));
            glqh_range range("dequant_matmul");
            if (glqh_launch_trellis_tile(blocked == 0 ? nullptr : x_rht, xb, B, packed[i], 4, c.m_pads[i], n_pad, c.parts[i], 0,
                                         1.0f, 0, 0, st, 0, packed2[i], R2, rs2[i]))
                return 1;
        }
        return tr_group_finish(c, n_shards, B, y_dtype, y_stride, st);
    }
    if (B > 1) {
        // 2..16 tokens: one transform launch per distinct sign vector, one small-batch launch per layer that decodes
        // both streams against the staged activations, under the K plan of the tallest layer, one finishing launch
        int64_t mmax = 0;
        for (int i = 0; i < n_shards; ++i) mmax = c.m_pads[i] > mmax ? c.m_pads[i] : mmax;
        int S = 0;
        glqh_trellis_mma_plan(mmax, n_pad, &S, &ks);
        const size_t xb = align256((size_t)B * n_pad * sizeof(f16));
        const size_t need = (size_t)n_shards * xb + align256((size_t)ks * B * total * sizeof(float));
        GLQH_REQUIRE(ws && ws_bytes >= need, "trellis two-stage group: workspace of %zu bytes needed, got %zu", need, ws_bytes);
        float *p = (float *)((char *)ws + (size_t)n_shards * xb);
        const f16 *x_of[GLQH_MAX_SHARDS];
        if (tr_group_transform(x, x_dtype, x_stride, B, sv, n_shards, blocks_n, n_blocks_n, bn_meta_dev, in_features, n_pad,
                               ws, xb, x_of, st))
            return 1;
        for (int i = 0; i < n_shards; ++i) {
            c.parts[i] = p;
            p += (size_t)ks * B * c.m_pads[i];
            glqh_range range("dequant_matmul");
            if (glqh_launch_trellis_mma_rvq(x_of[i], B, packed[i], packed2[i], R2, rs2[i], c.m_pads[i], n_pad, S, ks,
                                            c.parts[i], st))
                return 1;
        }
        return glqh_launch_output_rht_group(c.parts, c.su, c.ys, c.scale, c.m_pads, c.outs, n_shards, y_dtype, y_stride,
                                            B, ks, st);
    }
    GLQH_REQUIRE(tr_fuse_input_enabled() && tr_fusein_plan(c.m_pads, n_shards, n_pad, 1, &steps, &ks, 1) == 2,
                 "trellis two-stage group: shape not eligible");
    const size_t need = align256((size_t)ks * total * sizeof(float));
    GLQH_REQUIRE(ws && ws_bytes >= need, "trellis two-stage group: workspace of %zu bytes needed, got %zu", need, ws_bytes);
    float *p = (float *)ws;
    for (int i = 0; i < n_shards; ++i) {
        c.parts[i] = p;
        p += (size_t)ks * c.m_pads[i];
    }
    if (glqh_launch_trellis_mma_fusein_rvq(packed, packed2, R2, rs2, sv, c.parts, c.m_pads, n_shards, x, x_dtype, x_stride,
                                           n_pad, in_features, steps, ks, bn_meta_dev, blocks_n, (int)n_blocks_n, st))
        return 1;
    return glqh_launch_output_rht_group(c.parts, c.su, c.ys, c.scale, c.m_pads, c.outs, n_shards, y_dtype, y_stride, 1,
                                        ks, st);
}

// ---- routed experts of a mixture-of-experts layer ------------------------------------------------
int glqh_launch_trellis_mma_fusein_moe(const void *packed, int64_t stride_bytes, int R, const int64_t *topk_ids,
                                       int n_slots, int n_experts, int x_div, const float *pscale_dev,
                                       const void *x, int x_dtype, int64_t x_stride, const void *sv, int64_t m,
                                       int64_t k, int64_t in_features, int S, int ksplit, float *part,
                                       const glqh_block_meta *bn_meta, const int64_t *blocks_host, int n_blocks,
                                       hipStream_t stream);
int glqh_launch_trellis_mma_fusein_moe_rvq(const void *packed, int64_t stride_bytes, const void *packed2,
                                           int64_t stride2_bytes, int R2, const float *inv_rs2_dev,
                                           const int64_t *topk_ids, int n_slots, int n_experts, int x_div, const void *x,
                                           int x_dtype, int64_t x_stride, const void *sv, int64_t m, int64_t k,
                                           int64_t in_features, int S, int ksplit, float *part,
                                           const glqh_block_meta *bn_meta, const int64_t *blocks_host, int n_blocks,
                                           hipStream_t stream);
int glqh_launch_moe_output_rht(const float *part, int ks, int part_f16, int n_slots, int n_experts, const int64_t *topk_ids,
                               const void *su_base, const float *wscale_dev, int64_t out_features, int64_t m_pad,
                               const int64_t *blocks_m, int64_t n_blocks_m, void *h_f16, int64_t h_stride,
                               hipStream_t stream);
int glqh_launch_moe_gated_act(const void *h_f16, int64_t h_stride, void *out_f16, int n_slots, int64_t intermediate,
                              int act, hipStream_t stream);
int glqh_launch_moe_weighted_sum(const void *y_f16, int64_t y_stride, int num_tokens, int top_k, int n_experts,
                                 const int64_t *topk_ids, const float *topk_w, int64_t out_features, void *out,
                                 int out_dtype, int64_t out_stride, hipStream_t stream);

int glqh_moe_mid_eligible(int64_t m_pad13, const int64_t *blocks_m13, int64_t n_blocks_m13, int64_t n_pad2,
                          const int64_t *blocks_n2, int64_t n_blocks_n2);
int glqh_launch_moe_mid(const float *part, int ks, int part_f16, int n_slots, int n_experts, const int64_t *topk_ids,
                        const void *su_base, const float *wscale_dev, int64_t out_features13, int64_t m_pad13,
                        const int64_t *blocks_m13, int64_t n_blocks_m13, const int *perm, const int *pexp, const int *n_valid,
                        int64_t intermediate, int act, const void *sv2, int64_t n_pad2, const int64_t *blocks_n2,
                        int64_t n_blocks_n2, void *out_f16, int layout, int64_t Mp, hipStream_t stream);
int glqh_launch_moe_final(const float *part, int ks, int part_f16, int num_tokens, int top_k, int n_experts,
                          const int64_t *topk_ids, const float *topk_w, const void *su_base, const float *wscale_dev,
                          int64_t out_features, int64_t m_pad, const int64_t *blocks_m, int64_t n_blocks_m, void *out,
                          int out_dtype, int64_t out_stride, hipStream_t stream);
int glqh_moe_route_segments(int n_slots, int n_experts);
size_t glqh_moe_route_scratch_ints(int n_slots, int n_experts);
int glqh_launch_moe_route(const int64_t *topk_ids, int n_slots, int n_experts, int *perm, int *pexp, int *offs,
                          int *scratch, hipStream_t stream);
int glqh_moe_grouped_wide(int n_slots, int n_experts);
int glqh_launch_trellis_mma_moe_grouped(const void *packed, int64_t stride_bytes, int R, const int *perm,
                                        const int *offs, int n_slots, int n_experts, int x_div,
                                        const float *pscale_dev, const void *x_f16, int64_t m, int64_t k, int S,
                                        int ksplit, float *part, hipStream_t stream, const void *packed2 = nullptr,
                                        int64_t stride2_bytes = 0, int R2 = 0);

// many rows per expert: the tile kernel on the expert-sorted slots (trellis_tile.hip)
int glqh_trellis_tile_moe_tokens(int64_t n_slots, int64_t n_experts);
int64_t glqh_trellis_tile_moe_padded(int64_t n_slots, int64_t n_experts);
int64_t glqh_trellis_tile_moe_max_tiles(int64_t n_slots, int64_t n_experts);
int glqh_launch_trellis_tile_moe_table(const int *offs, int n_slots, int n_experts, void *tiles, int *n_tiles,
                                       hipStream_t stream);
int glqh_launch_trellis_pack_moe(const void *x_f16, void *xb, const int *perm, const int *offs, int n_slots,
                                 int n_experts, int x_div, int64_t k, hipStream_t stream);
int glqh_launch_trellis_tile_moe(const void *xb, const void *packed, int64_t stride_bytes, int R, const int *perm,
                                 const void *tiles, const int *n_tiles, const float *pscale_dev, const float *wscale_dev,
                                 int n_slots, int n_experts, int64_t m, int64_t k, void *out, int out_f16,
                                 hipStream_t stream, const void *packed2 = nullptr, int64_t stride2_bytes = 0, int R2 = 0);

struct moe_plan {
    int R1, R2, S, ks, ks_all;
    int tile;                                                  // the tile kernel's form: one K slot, fp16 sums
    int fuse2;                                                 // two stages in one launch: ks slots (first stage 4 bits/weight)
    size_t part_bytes;
};

// From this many (token, choice) slots on the rows are grouped by expert and every expert's stream is read
// once per 16 of its rows; below, every slot reads its expert's stream for itself (no routing launch, no
// separate input transforms).  The grouped form pays three more launches and wins once slots share experts:
// measured on 128 experts of 2048 -> 2 x 768 -> 2048 with 8 choices, 64 slots 79.7 (per slot) against 84.4 us
// (grouped), 128 slots 135.9 against 107.6, 512 slots 466 against 147.  GLQ_MOE_GROUP_MIN overrides (read once).
static int64_t moe_group_min(int64_t n_experts) {
    static const int64_t v = [] {
        const char *e = getenv("GLQ_MOE_GROUP_MIN");
        const long long x = e && *e ? atoll(e) : 0;
        return (int64_t)(x > 0 ? x : 0);
    }();
    if (v > 0) return v;
    const int64_t d = 3 * n_experts / 4;
    return d < 16 ? 16 : d;
}

// From this many rows per expert on average (slots / experts that can have rows) the grouped form hands over to
// the tile kernel's: below, an expert's stream is read once per 64 of its rows by a GEMV-shaped workgroup; above,
// its decoded weights meet up to 256 rows at a time on the matrix cores.  GLQ_MOE_TILE_MIN_ROWS overrides (read
// once; 0 = never).
static int64_t moe_tile_min_rows() {
    static const int64_t v = [] {
        const char *e = getenv("GLQ_MOE_TILE_MIN_ROWS");
        return (int64_t)(e && *e ? atoll(e) : 24);
    }();
    return v;
}

static bool moe_tile_form(int64_t n_slots, int64_t n_experts) {
    const int64_t live = n_experts < n_slots ? n_experts : n_slots, mn = moe_tile_min_rows();
    return mn > 0 && n_slots >= moe_group_min(n_experts) && n_slots >= mn * live;
}

// GLQ_MOE_FUSE=0 (read once): the launches between and after the decode launches stay separate at every slot count
// (output transform, activation, input transform, repack; output transform, weighted sum).
static bool moe_fuse_enabled() {
    static const bool on = [] {
        const char *e = getenv("GLQ_MOE_FUSE");
        return !(e && e[0] == '0');
    }();
    return on;
}
// from this many slots on (below, the separate launches are as fast or faster: 128 slots 108.8 us separate against
// 112.6 fused, 512 slots 147.1 / 148.2, 1024 slots 161.2 / 161.5, 2048 slots 222 / 215, 8192 slots 531 / 493)
constexpr int MOE_FUSE_MIN_SLOTS = 1024;

static int moe_proj_plan(const glqh_moe_proj *w, int64_t n_slots, int64_t n_experts, const char *what, moe_plan *p) {
    GLQH_REQUIRE(w && w->packed && w->su_f16 && w->sv_f16 && w->wscale_dev, "routed experts %s: null pointer", what);
    if (tr_bits_from_packed(w->packed_cols, 0, &p->R1) || tr_check_shape(w->m_pad, w->n_pad, w->packed_rows)) return 1;
    p->R2 = 0;
    if (w->packed2) {
        GLQH_REQUIRE(w->inv_rs2_dev, "routed experts %s: stage 2 is half-configured: packed2 present, inv_resid_scale2 absent",
                     what);
        if (tr_bits_from_packed(w->packed2_cols, 1, &p->R2)) return 1;
    }
    GLQH_REQUIRE(w->in_features >= 1 && w->in_features <= w->n_pad && w->out_features >= 1 &&
                     w->out_features <= w->m_pad && w->out_features % 8 == 0,
                 "routed experts %s: features %lld -> %lld do not fit %lld x %lld (out_features %% 8)", what,
                 (long long)w->in_features, (long long)w->out_features, (long long)w->m_pad, (long long)w->n_pad);
    const bool pow2_n = (w->n_pad & (w->n_pad - 1)) == 0;
    GLQH_REQUIRE(w->n_blocks_n > 1 ? (w->bn_meta_dev != nullptr && w->blocks_n != nullptr) : pow2_n,
                 "routed experts %s: input block sizes missing", what);
    p->tile = 0;
    if (moe_tile_form(n_slots, n_experts)) {
        p->tile = 1;
        p->S = 0;
        p->ks = 1;
    } else if (n_slots >= moe_group_min(n_experts)) {
        // about four workgroups per CU if every expert that can have rows has some
        const int64_t nkp = w->n_pad / 32, wgs = ((w->m_pad + 63) / 64) * (n_experts < n_slots ? n_experts : n_slots);
        int64_t ks = ((int64_t)glqh_device_cus() * 4 + wgs - 1) / wgs;
        if (ks > 16) ks = 16;
        int64_t S = ((nkp + ks - 1) / ks + 3) / 4 * 4;
        p->S = (int)S;
        p->ks = (int)((nkp + S - 1) / S);
    } else {
        GLQH_REQUIRE(glqh_trellis_mma_fusein_plan((w->m_pad / 64) * n_slots, w->n_pad, 1, &p->S, &p->ks),
                     "routed experts %s: no plan", what);
    }
    // both stages in one launch: the per-slot form and the grouped form's passes of 16 rows add the sums in fp32, the
    // tile form multiplies with one fp16 operand; the grouped form's passes of up to 64 rows keep a launch per stage
    p->fuse2 = p->R2 && p->R1 == 4 && tr_fuse_stages_enabled() &&
               (p->tile || n_slots < moe_group_min(n_experts) || !glqh_moe_grouped_wide((int)n_slots, (int)n_experts));
    p->ks_all = p->R2 && !p->fuse2 ? 2 * p->ks : p->ks;
    p->part_bytes = align256((size_t)p->ks_all * n_slots * w->m_pad * sizeof(float));
    return 0;
}

// workspace: part13 | h (slots x 2I f16) | a (slots x I f16) | part2 | y (slots x hidden f16), and for the
// grouped form: perm | pexp (slots int each) | offs (experts + 1 int) | routing scratch | transformed activations (fp16 rows of both
// projections in turn)
// and for the tile form: the activations packed in sorted order | the token tiles (int4 each) | their number
struct moe_ws {
    size_t part13, h, a, part2, y, perm, pexp, offs, route, xhat, xb, tiles, n_tiles, total;
};

static moe_ws moe_ws_layout(const glqh_moe_proj *w13, const glqh_moe_proj *w2, const moe_plan &p13, const moe_plan &p2,
                            int64_t num_tokens, int64_t n_slots, int64_t n_experts) {
    moe_ws l;
    size_t o = 0;
    l.part13 = o; o += p13.part_bytes;
    l.h = o; o += align256((size_t)n_slots * w13->out_features * sizeof(f16));
    l.a = o; o += align256((size_t)n_slots * w2->in_features * sizeof(f16));
    l.part2 = o; o += p2.part_bytes;
    l.y = o; o += align256((size_t)n_slots * w2->out_features * sizeof(f16));
    l.perm = l.pexp = l.offs = l.route = l.xhat = o;
    if (n_slots >= moe_group_min(n_experts)) {
        l.perm = o; o += align256((size_t)n_slots * sizeof(int));
        l.pexp = o; o += align256((size_t)n_slots * sizeof(int));
        l.offs = o; o += align256((size_t)(n_experts + 1) * sizeof(int));
        l.route = o; o += align256(glqh_moe_route_scratch_ints((int)n_slots, (int)n_experts) * sizeof(int));
        const size_t x13 = (size_t)num_tokens * w13->n_pad, x2 = (size_t)n_slots * w2->n_pad;
        l.xhat = o; o += align256((x13 > x2 ? x13 : x2) * sizeof(f16));
    }
    l.xb = l.tiles = l.n_tiles = o;
    if (p13.tile) {
        const size_t Mp = (size_t)glqh_trellis_tile_moe_padded(n_slots, n_experts);
        l.xb = o; o += align256(Mp * (size_t)(w13->n_pad > w2->n_pad ? w13->n_pad : w2->n_pad) * sizeof(f16));
        l.tiles = o; o += align256((size_t)glqh_trellis_tile_moe_max_tiles(n_slots, n_experts) * 16);
        l.n_tiles = o; o += 256;
    }
    l.total = o;
    return l;
}

extern "C" size_t glqh_fused_moe_trellis_workspace_bytes(int64_t num_tokens, int64_t top_k, int64_t num_experts,
                                                         const glqh_moe_proj *w13, const glqh_moe_proj *w2) {
    if (glqh_init() != 0 || num_tokens < 1 || top_k < 1 || num_experts < 1 || !w13 || !w2) return 0;
    const int64_t n_slots = num_tokens * top_k;
    moe_plan p13, p2;
    if (moe_proj_plan(w13, n_slots, num_experts, "w13", &p13) || moe_proj_plan(w2, n_slots, num_experts, "w2", &p2))
        return 0;
    return moe_ws_layout(w13, w2, p13, p2, num_tokens, n_slots, num_experts).total;
}

// one projection, rows grouped by expert: input transform of the rows, then one decode launch per stage
static int moe_decode_grouped(const glqh_moe_proj *w, const moe_plan &p, const int *perm, const int *offs, int n_slots,
                              int n_experts, int x_div, const void *x, int x_dtype, int64_t x_stride, int64_t x_rows,
                              void *xhat, float *part, hipStream_t st) {
    // x == nullptr: xhat already holds the transformed rows
    if (x && glqh_launch_input_rht(x, x_dtype, x_stride, w->sv_f16, xhat, GLQH_F16, x_rows, w->in_features, w->n_pad,
                                   w->bn_meta_dev, w->blocks_n, w->n_blocks_n, 0.0f, st))
        return 1;
    if (p.fuse2)                                               // both streams of stacked experts in the same passes
        return glqh_launch_trellis_mma_moe_grouped(w->packed, w->packed_rows * w->packed_cols * 2, p.R1, perm, offs, n_slots,
                                                   n_experts, x_div, w->inv_rs2_dev, xhat, w->m_pad, w->n_pad, p.S, p.ks,
                                                   part, st, w->packed2, w->packed_rows * w->packed2_cols * 2, p.R2);
    if (glqh_launch_trellis_mma_moe_grouped(w->packed, w->packed_rows * w->packed_cols * 2, p.R1, perm, offs, n_slots,
                                            n_experts, x_div, nullptr, xhat, w->m_pad, w->n_pad, p.S, p.ks, part, st))
        return 1;
    if (p.R2 &&
        glqh_launch_trellis_mma_moe_grouped(w->packed2, w->packed_rows * w->packed2_cols * 2, p.R2, perm, offs, n_slots,
                                            n_experts, x_div, w->inv_rs2_dev, xhat, w->m_pad, w->n_pad, p.S, p.ks,
                                            part + (int64_t)p.ks * n_slots * w->m_pad, st))
        return 1;
    return 0;
}

// one projection through the tile kernel: input transform of the rows, their packed copy in sorted order, one
// launch per stage into fp16 sums [stage][slot][row], times the expert's scale (and the second stage's)
static int moe_decode_tile(const glqh_moe_proj *w, const moe_plan &p, const int *perm, const int *offs, const void *tiles,
                           const int *n_tiles, int n_slots, int n_experts, int x_div, const void *x, int x_dtype,
                           int64_t x_stride, int64_t x_rows, void *xhat, void *xb, float *part, hipStream_t st) {
    if (x) {                                                   // nullptr: xb already holds the packed activations
        if (glqh_launch_input_rht(x, x_dtype, x_stride, w->sv_f16, xhat, GLQH_F16, x_rows, w->in_features, w->n_pad,
                                  w->bn_meta_dev, w->blocks_n, w->n_blocks_n, 0.0f, st))
            return 1;
        if (glqh_launch_trellis_pack_moe(xhat, xb, perm, offs, n_slots, n_experts, x_div, w->n_pad, st)) return 1;
    }
    if (p.fuse2)                                               // both streams of a stacked expert into one operand
        return glqh_launch_trellis_tile_moe(xb, w->packed, w->packed_rows * w->packed_cols * 2, p.R1, perm, tiles, n_tiles,
                                            w->inv_rs2_dev, w->wscale_dev, n_slots, n_experts, w->m_pad, w->n_pad, part, 1, st, w->packed2,
                                            w->packed_rows * w->packed2_cols * 2, p.R2);
    if (glqh_launch_trellis_tile_moe(xb, w->packed, w->packed_rows * w->packed_cols * 2, p.R1, perm, tiles, n_tiles,
                                     nullptr, w->wscale_dev, n_slots, n_experts, w->m_pad, w->n_pad, part, 1, st))
        return 1;
    if (p.R2 && glqh_launch_trellis_tile_moe(xb, w->packed2, w->packed_rows * w->packed2_cols * 2, p.R2, perm, tiles,
                                             n_tiles, w->inv_rs2_dev, w->wscale_dev, n_slots, n_experts, w->m_pad, w->n_pad,
                                             (f16 *)part + (int64_t)n_slots * w->m_pad, 1, st))
        return 1;
    return 0;
}

// one projection: decode launch per stage into part[K slot][slot][row]
static int moe_decode(const glqh_moe_proj *w, const moe_plan &p, const int64_t *topk_ids, int n_slots, int n_experts,
                      int x_div, const void *x, int x_dtype, int64_t x_stride, float *part, hipStream_t st) {
    if (p.fuse2)
        return glqh_launch_trellis_mma_fusein_moe_rvq(w->packed, w->packed_rows * w->packed_cols * 2, w->packed2,
                                                      w->packed_rows * w->packed2_cols * 2, p.R2, w->inv_rs2_dev, topk_ids,
                                                      n_slots, n_experts, x_div, x, x_dtype, x_stride, w->sv_f16, w->m_pad,
                                                      w->n_pad, w->in_features, p.S, p.ks, part, w->bn_meta_dev, w->blocks_n,
                                                      (int)w->n_blocks_n, st);
    if (glqh_launch_trellis_mma_fusein_moe(w->packed, w->packed_rows * w->packed_cols * 2, p.R1, topk_ids, n_slots,
                                           n_experts, x_div, nullptr, x, x_dtype, x_stride, w->sv_f16, w->m_pad,
                                           w->n_pad, w->in_features, p.S, p.ks, part, w->bn_meta_dev, w->blocks_n,
                                           (int)w->n_blocks_n, st))
        return 1;
    if (p.R2 &&
        glqh_launch_trellis_mma_fusein_moe(w->packed2, w->packed_rows * w->packed2_cols * 2, p.R2, topk_ids, n_slots,
                                           n_experts, x_div, w->inv_rs2_dev, x, x_dtype, x_stride, w->sv_f16,
                                           w->m_pad, w->n_pad, w->in_features, p.S, p.ks,
                                           part + (int64_t)p.ks * n_slots * w->m_pad, w->bn_meta_dev, w->blocks_n,
                                           (int)w->n_blocks_n, st))
        return 1;
    return 0;
}

extern "C" int glqh_fused_moe_trellis_3inst(const void *x, int x_dtype, int64_t x_stride, int64_t num_tokens,
                                            const int64_t *topk_ids, const float *topk_weights, int64_t top_k,
                                            int64_t num_experts, const glqh_moe_proj *w13, const glqh_moe_proj *w2,
                                            int64_t intermediate_size, int activation_type, void *out, int out_dtype,
                                            int64_t out_stride, void *ws, size_t ws_bytes, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(x && topk_ids && topk_weights && out && w13 && w2, "routed experts: null pointer");
    GLQH_REQUIRE(num_tokens >= 1 && top_k >= 1 && num_tokens * top_k <= 65535 && num_experts >= 1,
                 "routed experts: %lld tokens x %lld choices (at most 65535 slots)", (long long)num_tokens,
                 (long long)top_k);
    GLQH_REQUIRE(x_dtype == GLQH_F16 || x_dtype == GLQH_BF16, "routed experts: x must be f16 or bf16");
    GLQH_REQUIRE(activation_type >= 0 && activation_type <= 2,
                 "routed experts: gated activations 0 (silu), 1 (gelu-tanh), 2 (relu2) only, got %d", activation_type);
    const int n_slots = (int)(num_tokens * top_k);
    moe_plan p13, p2;
    if (moe_proj_plan(w13, n_slots, num_experts, "w13", &p13) || moe_proj_plan(w2, n_slots, num_experts, "w2", &p2))
        return 1;
    GLQH_REQUIRE(w13->out_features == 2 * intermediate_size && w2->in_features == intermediate_size,
                 "routed experts: w13 yields %lld values, w2 takes %lld, intermediate size %lld (gate | up)",
                 (long long)w13->out_features, (long long)w2->in_features, (long long)intermediate_size);
    const moe_ws l = moe_ws_layout(w13, w2, p13, p2, num_tokens, n_slots, num_experts);
    GLQH_REQUIRE(ws && ws_bytes >= l.total, "routed experts: workspace of %zu bytes needed, got %zu", l.total, ws_bytes);
    hipStream_t st = (hipStream_t)stream;
    char *base = (char *)ws;
    float *part13 = (float *)(base + l.part13), *part2 = (float *)(base + l.part2);
    f16 *h = (f16 *)(base + l.h), *hact = (f16 *)(base + l.a), *yslot = (f16 *)(base + l.y);
    int *perm = (int *)(base + l.perm), *offs = (int *)(base + l.offs);
    void *xhat = base + l.xhat;
    const bool grouped = n_slots >= moe_group_min(num_experts);
    GLQH_REQUIRE(!grouped || num_experts <= 65535, "routed experts: at most 65535 experts, got %lld", (long long)num_experts);
    int *pexp = (int *)(base + l.pexp);
    if (grouped && glqh_launch_moe_route(topk_ids, n_slots, (int)num_experts, perm, pexp, offs, (int *)(base + l.route), st))
        return 1;
    const bool tile = p13.tile != 0;
    void *xb = base + l.xb, *tiles = base + l.tiles;
    int *n_tiles = (int *)(base + l.n_tiles);
    if (tile && glqh_launch_trellis_tile_moe_table(offs, n_slots, (int)num_experts, tiles, n_tiles, st)) return 1;
    // gate | up of every slot: decode on the token's row, output transform with the expert's signs
    if (tile ? moe_decode_tile(w13, p13, perm, offs, tiles, n_tiles, n_slots, (int)num_experts, (int)top_k, x, x_dtype,
                               x_stride, num_tokens, xhat, xb, part13, st)
        : grouped ? moe_decode_grouped(w13, p13, perm, offs, n_slots, (int)num_experts, (int)top_k, x, x_dtype, x_stride,
                                       num_tokens, xhat, part13, st)
                  : moe_decode(w13, p13, topk_ids, n_slots, (int)num_experts, (int)top_k, x, x_dtype, x_stride, part13, st))
        return 1;
    // between the decode launches: one launch per slot row for the grouped forms, three or four otherwise
    const bool mid = grouped && n_slots >= MOE_FUSE_MIN_SLOTS && moe_fuse_enabled() &&
                     glqh_moe_mid_eligible(w13->m_pad, w13->blocks_m, w13->n_blocks_m, w2->n_pad, w2->blocks_n,
                                           w2->n_blocks_n);
    const void *x2 = hact;
    if (mid) {
        if (glqh_launch_moe_mid(part13, p13.ks_all, tile, n_slots, (int)num_experts, topk_ids, w13->su_f16, w13->wscale_dev,
                                w13->out_features, w13->m_pad, w13->blocks_m, w13->n_blocks_m, perm, pexp, offs + num_experts,
                                intermediate_size, activation_type, w2->sv_f16, w2->n_pad, w2->blocks_n, w2->n_blocks_n,
                                tile ? xb : xhat, tile ? 2 : 0,
                                tile ? glqh_trellis_tile_moe_padded(n_slots, num_experts) : 0, st))
            return 1;
        x2 = nullptr;
    } else {
        if (glqh_launch_moe_output_rht(part13, p13.ks_all, tile, n_slots, (int)num_experts, topk_ids, w13->su_f16,
                                       w13->wscale_dev, w13->out_features, w13->m_pad, w13->blocks_m, w13->n_blocks_m, h,
                                       w13->out_features, st))
            return 1;
        if (glqh_launch_moe_gated_act(h, w13->out_features, hact, n_slots, intermediate_size, activation_type, st)) return 1;
    }
    // down projection of every slot, then the weighted sum over each token's choices, in their order
    if (tile ? moe_decode_tile(w2, p2, perm, offs, tiles, n_tiles, n_slots, (int)num_experts, 1, x2, GLQH_F16,
                               intermediate_size, n_slots, xhat, xb, part2, st)
        : grouped ? moe_decode_grouped(w2, p2, perm, offs, n_slots, (int)num_experts, 1, x2, GLQH_F16, intermediate_size,
                                       n_slots, xhat, part2, st)
                  : moe_decode(w2, p2, topk_ids, n_slots, (int)num_experts, 1, hact, GLQH_F16, intermediate_size, part2, st))
        return 1;
    if (n_slots >= MOE_FUSE_MIN_SLOTS && moe_fuse_enabled())
        return glqh_launch_moe_final(part2, p2.ks_all, tile, (int)num_tokens, (int)top_k, (int)num_experts, topk_ids,
                                     topk_weights, w2->su_f16, w2->wscale_dev, w2->out_features, w2->m_pad, w2->blocks_m,
                                     w2->n_blocks_m, out, out_dtype, out_stride, st);
    if (glqh_launch_moe_output_rht(part2, p2.ks_all, tile, n_slots, (int)num_experts, topk_ids, w2->su_f16, w2->wscale_dev,
                                   w2->out_features, w2->m_pad, w2->blocks_m, w2->n_blocks_m, yslot, w2->out_features,
                                   st))
        return 1;
    return glqh_launch_moe_weighted_sum(yslot, w2->out_features, (int)num_tokens, (int)top_k, (int)num_experts,
                                        topk_ids, topk_weights, w2->out_features, out, out_dtype, out_stride, st);
}

// ---- batch-1 decode loop: output transform fused with what follows it (glq_decoder_ops.h) ----
extern "C" int glqh_trellis_linear_add_rmsnorm_bf16(const void *x, int64_t in_features,
                                                    const glqh_trellis_shard *shard, const int64_t *blocks_n,
                                                    int64_t n_blocks_n, const glqh_block_meta *bn_meta_dev,
                                                    int64_t n_pad, const void *resid, const void *norm_w,
                                                    double eps, void *x_out, void *h_out, void *ws,
                                                    size_t ws_bytes, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(shard && resid && norm_w && x_out && h_out, "linear+add+rmsnorm: null pointer");
    GLQH_REQUIRE(shard->su_f16 && shard->out_features == shard->m_pad,
                 "linear+add+rmsnorm: needs su and out_features == m_pad");
    hipStream_t st = (hipStream_t)stream;
    glqh_trellis_shard sh = *shard;
    sh.y = nullptr;
    tr_group_ctx c;
    if (tr_group_decode(x, GLQH_BF16, in_features, 1, &sh, 1, blocks_n, n_blocks_n, bn_meta_dev, in_features, n_pad,
                        ws, ws_bytes, st, &c))
        return 1;
    return glqh_launch_out_add_rmsnorm(c.parts[0], c.ks, c.scale[0], c.su[0], c.m_pads[0], resid, norm_w, (float)eps,
                                       x_out, h_out, st);
}

extern "C" int glqh_trellis_gate_up_silu_bf16(const void *x, int64_t in_features,
                                              const glqh_trellis_shard *gate_up, const int64_t *blocks_n,
                                              int64_t n_blocks_n, const glqh_block_meta *bn_meta_dev,
                                              int64_t n_pad, void *act_out, void *ws, size_t ws_bytes,
                                              void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(gate_up && act_out, "gate/up+silu: null pointer");
    GLQH_REQUIRE(gate_up[0].m_pad == gate_up[1].m_pad && gate_up[0].out_features == gate_up[1].out_features &&
                     gate_up[0].su_f16 && gate_up[1].su_f16,
                 "gate/up+silu: the two layers must have the same shape and carry su");
    hipStream_t st = (hipStream_t)stream;
    glqh_trellis_shard sh[2] = {gate_up[0], gate_up[1]};
    sh[0].y = sh[1].y = nullptr;
    tr_group_ctx c;
    if (tr_group_decode(x, GLQH_BF16, in_features, 1, sh, 2, blocks_n, n_blocks_n, bn_meta_dev, in_features, n_pad,
                        ws, ws_bytes, st, &c))
        return 1;
    return glqh_launch_out_silu_mul(c.parts[0], c.parts[1], c.ks, c.scale[0], c.scale[1], c.su[0], c.su[1],
                                    c.m_pads[0], c.outs[0], act_out, st);
}

extern "C" int glqh_trellis_qkv_rope_store_bf16(const void *x, int64_t in_features, const glqh_trellis_shard *qkv,
                                                const int64_t *blocks_n, int64_t n_blocks_n,
                                                const glqh_block_meta *bn_meta_dev, int64_t n_pad,
                                                const int64_t *pos, const void *cos_t, const void *sin_t,
                                                void *q_out, void *k_cache, void *v_cache, int64_t head_dim,
                                                int64_t max_len, int apply_rope, void *ws, size_t ws_bytes,
                                                void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(qkv, "qkv+rope: null pointer");
    hipStream_t st = (hipStream_t)stream;
    glqh_trellis_shard sh[3] = {qkv[0], qkv[1], qkv[2]};
    for (int i = 0; i < 3; ++i) {
        GLQH_REQUIRE(sh[i].su_f16 && sh[i].out_features == sh[i].m_pad, "qkv+rope: needs su and out_features == m_pad");
        sh[i].y = nullptr;
    }
    tr_group_ctx c;
    if (tr_group_decode(x, GLQH_BF16, in_features, 1, sh, 3, blocks_n, n_blocks_n, bn_meta_dev, in_features, n_pad,
                        ws, ws_bytes, st, &c))
        return 1;
    return glqh_launch_out_rope_store(c.parts, c.su, c.scale, c.m_pads, c.ks, pos, cos_t, sin_t, q_out, k_cache,
                                      v_cache, head_dim, max_len, apply_rope, st);
}

extern "C" int glqh_trellis_qkv_rope_attn_shared_bf16(const void *x, int64_t in_features,
                                                      const glqh_trellis_shard *qkv, const int64_t *blocks_n,
                                                      int64_t n_blocks_n, const glqh_block_meta *bn_meta_dev,
                                                      int64_t n_pad, const int64_t *pos, const void *cos_t,
                                                      const void *sin_t, void *k_cache, void *v_cache, void *out,
                                                      int64_t heads, int64_t kv_heads, int64_t head_dim,
                                                      int64_t max_len, int apply_rope, void *ws, size_t ws_bytes,
                                                      void *state, size_t state_bytes, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(qkv, "qkv+rope+attention: null pointer");
    hipStream_t st = (hipStream_t)stream;
    glqh_trellis_shard sh[3] = {qkv[0], qkv[1], qkv[2]};
    for (int i = 0; i < 3; ++i) {
        GLQH_REQUIRE(sh[i].su_f16 && sh[i].out_features == sh[i].m_pad,
                     "qkv+rope+attention: needs su and out_features == m_pad");
        sh[i].y = nullptr;
    }
    tr_group_ctx c;
    if (tr_group_decode(x, GLQH_BF16, in_features, 1, sh, 3, blocks_n, n_blocks_n, bn_meta_dev, in_features, n_pad,
                        ws, ws_bytes, st, &c))
        return 1;
    return glqh_launch_out_rope_attn(c.parts, c.su, c.scale, c.m_pads, c.ks, pos, cos_t, sin_t, k_cache, v_cache,
                                     out, heads, kv_heads, head_dim, max_len, apply_rope, state, state_bytes, st);
}

extern "C" int glqh_trellis_qkv_rope_attn_bf16(const void *x, int64_t in_features, const glqh_trellis_shard *qkv,
                                               const int64_t *blocks_n, int64_t n_blocks_n,
                                               const glqh_block_meta *bn_meta_dev, int64_t n_pad,
                                               const int64_t *pos, const void *cos_t, const void *sin_t,
                                               void *k_cache, void *v_cache, void *out, int64_t heads,
                                               int64_t kv_heads, int64_t head_dim, int64_t max_len,
                                               int apply_rope, void *ws, size_t ws_bytes, void *stream) {
    return glqh_trellis_qkv_rope_attn_shared_bf16(x, in_features, qkv, blocks_n, n_blocks_n, bn_meta_dev, n_pad, pos,
                                                  cos_t, sin_t, k_cache, v_cache, out, heads, kv_heads, head_dim,
                                                  max_len, apply_rope, ws, ws_bytes, nullptr, 0, stream);
}

// ---- E8 shell ------------------------------------------------------------------------
extern "C" int glqh_e8_pack_table(const void *codebook_f16, int64_t n_entries, uint32_t *packed_out,
                                  int32_t *bad_dev, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(codebook_f16 && packed_out && bad_dev, "e8 pack table: null pointer");
    GLQH_REQUIRE(n_entries >= 1 && n_entries <= 65536, "e8 pack table: %lld entries (1..65536)",
                 (long long)n_entries);
    return glqh_launch_e8_pack_table(codebook_f16, n_entries, packed_out, bad_dev, (hipStream_t)stream);
}

extern "C" int glqh_e8_repack_table(const uint32_t *codebook_packed, int64_t n_entries,
                                    uint32_t *packed_out, int32_t *bad_dev, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(codebook_packed && packed_out && bad_dev, "e8 repack table: null pointer");
    GLQH_REQUIRE(n_entries >= 1 && n_entries <= 65536, "e8 repack table: %lld entries (1..65536)",
                 (long long)n_entries);
    return glqh_launch_e8_repack_table(codebook_packed, n_entries, packed_out, bad_dev, (hipStream_t)stream);
}

extern "C" int glqh_e8_fold_table(const uint32_t *table, int64_t n_entries, void *halves_out, int64_t capacity,
                                  uint32_t *map_out, int64_t *n_halves_out, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(table && halves_out && map_out && n_halves_out, "e8 fold table: null pointer");
    GLQH_REQUIRE(n_entries >= 1 && n_entries <= 65536 && capacity >= 1, "e8 fold table: %lld entries (1..65536)",
                 (long long)n_entries);
    hipStream_t st = (hipStream_t)stream;
    std::vector<uint32_t> words((size_t)n_entries), map((size_t)n_entries);
    std::vector<uint16_t> halves;                                  // 4 fp16 bit patterns per entry
    if (glqh_check_hip(hipMemcpyAsync(words.data(), table, (size_t)n_entries * 4, hipMemcpyDeviceToHost, st),
                       "e8 fold table: copy to host") ||
        glqh_check_hip(hipStreamSynchronize(st), "e8 fold table: synchronize"))
        return 1;
    std::unordered_map<uint32_t, uint32_t> number;                 // four codes of a half -> its number
    for (int64_t k = 0; k < n_entries; ++k) {
        uint32_t ids[2];
        for (int h = 0; h < 2; ++h) {
            uint32_t key = 0;
            uint16_t bits[4];
            for (int c = 0; c < 4; ++c) {
                const int col = 4 * h + c;                         // nibble p = column 2p, nibble p + 4 = column 2p + 1
                const int code = (int)((words[(size_t)k] >> (4 * ((col >> 1) + 4 * (col & 1)))) & 15u);
                GLQH_REQUIRE(code <= 12, "e8 fold table: entry %lld holds a code above 12", (long long)k);
                key |= (uint32_t)code << (4 * c);
                // fp16 bits of (code - 6) / 2: sign, then magnitude m / 2 for m = 1..6
                static const uint16_t mag[7] = {0x0000, 0x3800, 0x3C00, 0x3E00, 0x4000, 0x4100, 0x4200};
                bits[c] = (uint16_t)(mag[code < 6 ? 6 - code : code - 6] | (code < 6 ? 0x8000 : 0));
            }
            auto it = number.find(key);
            if (it == number.end()) {
                it = number.emplace(key, (uint32_t)(halves.size() / 4)).first;
                halves.insert(halves.end(), bits, bits + 4);
            }
            ids[h] = it->second;
        }
        map[(size_t)k] = ids[0] | ids[1] << 16;
    }
    const size_t n = halves.size() / 4;
    *n_halves_out = (int64_t)n;
    GLQH_REQUIRE((int64_t)n <= capacity && n <= 2048, "e8 fold table: %zu half codewords, room for %lld (at most 2048)", n,
                 (long long)capacity);
    if (glqh_check_hip(hipMemcpyAsync(halves_out, halves.data(), n * 8, hipMemcpyHostToDevice, st),
                       "e8 fold table: half codewords to device") ||
        glqh_check_hip(hipMemcpyAsync(map_out, map.data(), (size_t)n_entries * 4, hipMemcpyHostToDevice, st),
                       "e8 fold table: map to device") ||
        glqh_check_hip(hipStreamSynchronize(st), "e8 fold table: synchronize"))
        return 1;
    return 0;
}

int glqh_e8_mma_ksplit(int64_t m_pad, int64_t n_pad, int64_t B, int64_t n1, int fold);

extern "C" int glqh_e8_fold_eligible(int64_t m_pad, int64_t n_pad, int64_t B) {
    if (glqh_init() != 0 || m_pad < 1 || n_pad < 8 || (n_pad & 7) || B < 1) return 0;
    if (B > GLQH_E8_SMALL_BATCH) return glqh_e8_tile_ksplit(m_pad, n_pad, B, 1, 1) > 0 ? 1 : 0;   // the many-token kernel
    return glqh_e8_mma_ksplit(m_pad, n_pad, B, 65536, 1) > 0 ? 1 : 0;
}

extern "C" int64_t glqh_e8_folded_count(int64_t rows, int64_t cols) {
    if (rows < 1 || cols < 1) return 0;
    return ((rows + 15) / 16) * ((cols + 31) / 32) * 512;
}

extern "C" int glqh_e8_fold_indices(const void *q, int64_t rows, int64_t cols, const uint32_t *map, int64_t n_entries,
                                    uint16_t *lo16_out, uint8_t *hi8_out, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(q && map && lo16_out && hi8_out, "e8 fold indices: null pointer");
    GLQH_REQUIRE(rows >= 1 && cols >= 1 && n_entries >= 1 && n_entries <= 65536,
                 "e8 fold indices: %lld x %lld indices, %lld entries", (long long)rows, (long long)cols,
                 (long long)n_entries);
    return glqh_launch_e8_fold_indices(q, rows, cols, map, n_entries, lo16_out, hi8_out, (hipStream_t)stream);
}

struct e8_stages {
    const void *q[4];
    float scale[4];
    int n;
};

static int e8_resolve_stages(const void *q1, const void *q2, const void *q3, const void *q4,
                             double wscale, double inv_rs, double inv_rs2, double inv_rs3,
                             const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                             e8_stages *out) {
    GLQH_REQUIRE(q1 && table1, "e8 matmul: null index or table pointer");
    out->q[0] = q1; out->q[1] = q1; out->q[2] = q1; out->q[3] = q1;
    out->scale[0] = (float)wscale;
    out->scale[1] = out->scale[2] = out->scale[3] = 0.0f;
    out->n = 1;
    if (q2 && inv_rs != 0.0) {
        GLQH_REQUIRE(table2 && n_entries2 >= 1 && n_entries2 <= 65536,
                     "e8 matmul: stage 2 needs its table (1..65536 entries)");
        out->q[1] = q2;
        out->scale[1] = (float)(wscale * inv_rs);
        out->n = 2;
        if (q3 && inv_rs2 != 0.0) {
            out->q[2] = q3;
            out->scale[2] = (float)(wscale * inv_rs2);
            out->n = 3;
            if (q4 && inv_rs3 != 0.0) {
                out->q[3] = q4;
                out->scale[3] = (float)(wscale * inv_rs3);
                out->n = 4;
            }
        }
    }
    return 0;
}

static int e8_check_dims(int64_t m_pad, int64_t n_pad, int64_t B) {
    GLQH_REQUIRE(m_pad >= 1 && n_pad >= 8 && n_pad % 8 == 0, "e8 matmul: n_pad %lld must be a multiple of 8",
                 (long long)n_pad);
    GLQH_REQUIRE(B >= 1 && B <= 65535 * 4, "e8 matmul: B=%lld out of range", (long long)B);
    GLQH_REQUIRE((m_pad + 31) / 32 <= 2147483647ll, "e8 matmul: m_pad too large");
    return 0;
}

static size_t e8_part_bytes(int64_t m_pad, int64_t n_pad, int64_t B) {
    // the many-token kernel: stages are combined before the product (one or two stages get the most K
    // slots); folded streams take every width the indices take and more, so they bound the size
    const int tks = e8_tile_ks(m_pad, n_pad, B, 1, true);
    size_t tile = 0;
    if (tks > 0)                                                 // + the repacked activations
        tile = align256((size_t)tks * B * m_pad * sizeof(float)) + align256(glqh_e8_tile_xb_bytes(n_pad, B));
    if (tks > 0 && e8_tile_ks(m_pad, n_pad, B, 1, false) > 0) return tile;
    int ks = glqh_e8_pick_ksplit(m_pad, n_pad, B, 0);
    const int ksf = glqh_e8_pick_ksplit(m_pad, n_pad, B, 1);       // on folded streams
    if (ksf > ks) ks = ksf;
    const size_t plain = align256((size_t)ks * 4 * B * m_pad * sizeof(float));
    return plain > tile ? plain : tile;
}

extern "C" size_t glqh_e8_matmul_workspace_bytes(int64_t m_pad, int64_t n_pad, int64_t B) {
    if (m_pad < 1 || n_pad < 8 || B < 1) return 0;
    glqh_init();
    return e8_part_bytes(m_pad, n_pad, B);
}

extern "C" int glqh_e8_dequant_matmul(const void *x_f16, int64_t B, const void *q1, const void *q2,
                                      const void *q3, const void *q4, const uint32_t *table1,
                                      const uint32_t *table2, int64_t n_entries2, double wscale,
                                      double inv_rs, double inv_rs2, double inv_rs3, int64_t m_pad,
                                      int64_t n_pad, float *out, void *ws, size_t ws_bytes,
                                      void *stream) {
    return glqh_e8_dequant_matmul_folded(x_f16, B, q1, q2, q3, q4, table1, table2, n_entries2, wscale, inv_rs, inv_rs2,
                                         inv_rs3, m_pad, n_pad, out, ws, ws_bytes, stream, nullptr);
}

extern "C" int glqh_e8_dequant_matmul_folded(const void *x_f16, int64_t B, const void *q1, const void *q2,
                                             const void *q3, const void *q4, const uint32_t *table1,
                                             const uint32_t *table2, int64_t n_entries2, double wscale,
                                             double inv_rs, double inv_rs2, double inv_rs3, int64_t m_pad,
                                             int64_t n_pad, float *out, void *ws, size_t ws_bytes, void *stream,
                                             const glqh_e8_folded *folded) {
    GLQH_INIT();
    GLQH_REQUIRE(x_f16 && out, "e8 matmul: null pointer");
    e8_stages sg;
    if (e8_check_dims(m_pad, n_pad, B) ||
        e8_resolve_stages(q1, q2, q3, q4, wscale, inv_rs, inv_rs2, inv_rs3, table1, table2, n_entries2, &sg))
        return 1;
    hipStream_t st = (hipStream_t)stream;
    float *part = (float *)ws;
    const int tks = e8_tile_ks(m_pad, n_pad, B, sg.n, folded != nullptr);
    if (tks > 0) {
        const size_t pbytes = align256((size_t)tks * B * m_pad * sizeof(float));
        const size_t need = pbytes + glqh_e8_tile_xb_bytes(n_pad, B);
        GLQH_REQUIRE(ws && ws_bytes >= need, "e8 matmul: workspace of %zu bytes needed, got %zu", need, ws_bytes);
        const float rel[3] = {(float)inv_rs, (float)inv_rs2, (float)inv_rs3};
        if (glqh_launch_e8_tile(x_f16, (char *)ws + pbytes, B, sg.q, sg.n, table1, table2 ? table2 : table1, table2 ? n_entries2 : 65536,
                                rel, m_pad, n_pad, part, st, folded))
            return 1;
        return glqh_launch_reduce_splits(part, tks, B * m_pad, B, m_pad, (float)wscale, out, m_pad, 0, st);
    }
    // folded streams with K inside the workgroups: the kernel writes the finished sums itself
    if (folded && glqh_e8_mma_direct_ok(m_pad, n_pad, B, sg.n))
        return glqh_launch_e8_partial(x_f16, B, sg.q, sg.n, table1, table2 ? table2 : table1, table2 ? n_entries2 : 65536,
                                      m_pad, n_pad, 1, out, st, sg.scale, folded, 1);
    const int ks = glqh_e8_pick_ksplit(m_pad, n_pad, B, folded != nullptr);
    const size_t need = (size_t)ks * sg.n * B * m_pad * sizeof(float);
    GLQH_REQUIRE(ws && ws_bytes >= need, "e8 matmul: workspace of %zu bytes needed, got %zu", need, ws_bytes);
    // every stage's partial sums are written already multiplied by that stage's scale: one
    // reduction over ks * stages plain slots instead of one launch per stage
    if (glqh_launch_e8_partial(x_f16, B, sg.q, sg.n, table1, table2 ? table2 : table1,
                               table2 ? n_entries2 : 65536, m_pad, n_pad, ks, part, st, sg.scale, folded))
        return 1;
    return glqh_launch_reduce_splits(part, ks * sg.n, B * m_pad, B, m_pad, 1.0f, out, m_pad, 0, st);
}

extern "C" int glqh_e8_decompress(const void *q1, const void *q2, const void *q3, const void *q4,
                                  const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                                  double inv_rs, double inv_rs2, double inv_rs3, int64_t m_pad,
                                  int64_t n_pad, void *out_f16, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(out_f16, "e8 decompress: null pointer");
    e8_stages sg;
    if (e8_check_dims(m_pad, n_pad, 1) ||
        e8_resolve_stages(q1, q2, q3, q4, 1.0, inv_rs, inv_rs2, inv_rs3, table1, table2, n_entries2, &sg))
        return 1;
    return glqh_launch_e8_decompress(sg.q, sg.n, table1, table2 ? table2 : table1,
                                     table2 ? n_entries2 : 65536, sg.scale[1], sg.scale[2], sg.scale[3],
                                     m_pad, n_pad, out_f16, (hipStream_t)stream);
}

extern "C" int glqh_e8_decompress_f32(const void *q1, const void *q2, const void *q3, const void *q4,
                                      const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                                      double inv_rs, double inv_rs2, double inv_rs3, int64_t m_pad,
                                      int64_t n_pad, float *out_f32, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(out_f32, "e8 decompress: null pointer");
    e8_stages sg;
    if (e8_check_dims(m_pad, n_pad, 1) ||
        e8_resolve_stages(q1, q2, q3, q4, 1.0, inv_rs, inv_rs2, inv_rs3, table1, table2, n_entries2, &sg))
        return 1;
    return glqh_launch_e8_decompress_f32(sg.q, sg.n, table1, table2 ? table2 : table1,
                                         table2 ? n_entries2 : 65536, sg.scale[1], sg.scale[2], sg.scale[3],
                                         m_pad, n_pad, out_f32, (hipStream_t)stream);
}

extern "C" int glqh_e8_embedding_rows(const int64_t *ids, int64_t n_ids, const void *q1, const void *q2,
                                      const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                                      const float *wscale_rows, const float *inv_rs_rows, const void *sv_f16,
                                      int64_t n_pad, int64_t embedding_dim, int64_t num_embeddings,
                                      double embed_scale, void *out, int out_dtype, int64_t out_stride,
                                      void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(num_embeddings >= 1, "e8 embedding: empty table");
    GLQH_REQUIRE(!q2 || !table2 || (n_entries2 >= 1 && n_entries2 <= 65536), "e8 embedding: bad secondary table size");
    return glqh_launch_e8_embedding(ids, n_ids, q1, q2, table1, q2 ? (table2 ? table2 : table1) : nullptr,
                                    q2 ? (table2 ? n_entries2 : 65536) : 0, wscale_rows, inv_rs_rows, sv_f16,
                                    n_pad, embedding_dim, num_embeddings, (float)embed_scale, out, out_dtype,
                                    out_stride, (hipStream_t)stream);
}

extern "C" size_t glqh_fused_linear_e8_workspace_bytes(int64_t B, int64_t n_pad, int64_t m_pad) {
    if (m_pad < 1 || n_pad < 8 || B < 1) return 0;
    glqh_init();
    return align256((size_t)B * n_pad * sizeof(f16)) + e8_part_bytes(m_pad, n_pad, B);
}

extern "C" int glqh_fused_linear_e8(const void *x, int x_dtype, int64_t x_stride, int64_t B,
                                    const void *sv_f16, const void *su_f16, const void *q1,
                                    const void *q2, const void *q3, const void *q4,
                                    const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                                    double wscale, double inv_rs, double inv_rs2, double inv_rs3,
                                    const int64_t *blocks_n, int64_t n_blocks_n, const int64_t *blocks_m,
                                    int64_t n_blocks_m, const glqh_block_meta *bn_meta_dev,
                                    const glqh_block_meta *bm_meta_dev, int64_t in_features,
                                    int64_t out_features, int64_t n_pad, int64_t m_pad, void *y,
                                    int y_dtype, int64_t y_stride, void *ws, size_t ws_bytes,
                                    void *stream) {
    return glqh_fused_linear_e8_folded(x, x_dtype, x_stride, B, sv_f16, su_f16, q1, q2, q3, q4, table1, table2,
                                       n_entries2, wscale, inv_rs, inv_rs2, inv_rs3, blocks_n, n_blocks_n, blocks_m,
                                       n_blocks_m, bn_meta_dev, bm_meta_dev, in_features, out_features, n_pad, m_pad,
                                       y, y_dtype, y_stride, ws, ws_bytes, stream, nullptr);
}

extern "C" int glqh_fused_linear_e8_folded(const void *x, int x_dtype, int64_t x_stride, int64_t B,
                                           const void *sv_f16, const void *su_f16, const void *q1,
                                           const void *q2, const void *q3, const void *q4,
                                           const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                                           double wscale, double inv_rs, double inv_rs2, double inv_rs3,
                                           const int64_t *blocks_n, int64_t n_blocks_n, const int64_t *blocks_m,
                                           int64_t n_blocks_m, const glqh_block_meta *bn_meta_dev,
                                           const glqh_block_meta *bm_meta_dev, int64_t in_features,
                                           int64_t out_features, int64_t n_pad, int64_t m_pad, void *y,
                                           int y_dtype, int64_t y_stride, void *ws, size_t ws_bytes,
                                           void *stream, const glqh_e8_folded *folded) {
    GLQH_INIT();
    GLQH_REQUIRE(x && sv_f16 && su_f16 && y, "fused e8 linear: null pointer");
    e8_stages sg;
    if (e8_check_dims(m_pad, n_pad, B) ||
        e8_resolve_stages(q1, q2, q3, q4, wscale, inv_rs, inv_rs2, inv_rs3, table1, table2, n_entries2, &sg))
        return 1;
    GLQH_REQUIRE(B <= 65535, "fused e8 linear: B=%lld out of range", (long long)B);
    GLQH_REQUIRE(in_features <= n_pad && out_features <= m_pad, "fused e8 linear: features exceed padded dims");
    const size_t xb = align256((size_t)B * n_pad * sizeof(f16));
    const int tks = e8_tile_ks(m_pad, n_pad, B, sg.n, folded != nullptr);
    const int ks = tks > 0 ? tks : glqh_e8_pick_ksplit(m_pad, n_pad, B, folded != nullptr);
    const size_t tile_part = align256((size_t)ks * B * m_pad * sizeof(float));
    const size_t need = tks > 0 ? xb + tile_part + glqh_e8_tile_xb_bytes(n_pad, B)
                                : xb + (size_t)ks * sg.n * B * m_pad * sizeof(float);
    GLQH_REQUIRE(ws && ws_bytes >= need, "fused e8 linear: workspace of %zu bytes needed, got %zu", need,
                 ws_bytes);
    hipStream_t st = (hipStream_t)stream;
    f16 *x_rht = (f16 *)ws;
    float *part = (float *)((char *)ws + xb);
    // tile kernel: the transform writes the kernel's blocked operand layout itself where it can
    int blocked = -1;
    if (tks > 0)
        blocked = glqh_launch_input_rht_blocked(x, x_dtype, x_stride, sv_f16, (char *)ws + xb + tile_part, 1,
                                                glqh_e8_tile_padded_tokens(B, sg.n), B, in_features, n_pad,
                                                blocks_n, n_blocks_n, st);
    if (blocked > 0) return 1;
    if (blocked != 0 &&
        glqh_launch_input_rht(x, x_dtype, x_stride, sv_f16, x_rht, GLQH_F16, B, in_features, n_pad,
                              bn_meta_dev, blocks_n, n_blocks_n, 0.0f, st))
        return 1;
    if (tks > 0) {
        // many tokens: one combined product on the compressed indices, summed over its K slots and
        // scaled by the output transform.  From 257 tokens on folded streams the sums are rounded to fp16 on
        // the way out, times Wscale (half the bytes between the product and the output transform, as on the
        // trellis route; GLQ_E8_F16_SUMS=0 keeps them fp32).  The whole-block transform that reads them stores
        // 16 bytes at a time: rows of y that do not start on 16 bytes keep fp32 sums.
        static const bool f16_on = [] { const char *e = getenv("GLQ_E8_F16_SUMS"); return !(e && e[0] == '0'); }();
        const int64_t y_esz = y_dtype == GLQH_F32 ? 4 : 2;
        const int f16_sums = f16_on && tks <= tr_f16_sums_max_slots() && glqh_e8_tile_f16_sums_ok(B, folded != nullptr, m_pad) &&
                             glqh_output_rht_wide_eligible(B, blocks_m, n_blocks_m, m_pad) && ((uintptr_t)y & 15) == 0 &&
                             ((uintptr_t)su_f16 & 15) == 0 && (y_stride * y_esz) % 16 == 0;
        const float rel[3] = {(float)inv_rs, (float)inv_rs2, (float)inv_rs3};
        if (glqh_launch_e8_tile(blocked == 0 ? nullptr : x_rht, (char *)ws + xb + tile_part, B, sg.q, sg.n, table1,
                                table2 ? table2 : table1, table2 ? n_entries2 : 65536, rel, m_pad, n_pad, part, st, folded,
                                f16_sums, (float)wscale))
            return 1;
        glqh_ysrc src = {};
        src.nparts = 1;
        src.scale[0] = f16_sums ? 1.0f : (float)wscale;        // fp16 sums carry the scale already
        src.part = part;
        src.part_kstride = B * m_pad;
        src.ksplit = tks;
        src.part_f16 = f16_sums;
        return glqh_launch_output_rht(src, su_f16, y, y_dtype, y_stride, B, out_features, m_pad, bm_meta_dev,
                                      blocks_m, n_blocks_m, 0, 0.0f, st);
    }
    // Canonical output blocks at up to 16 tokens: every stage's partial sums are written already
    // multiplied by that stage's scale, which makes them ks * stages plain slots for the slice
    // kernels of the grouped launcher (faster than the generic multi-part transform).
    glqh_meta_args canon_m;
    const bool canon_out = B <= 16 && glqh_fill_meta_args(&canon_m, n_blocks_m > 1 ? blocks_m : nullptr,
                                                          n_blocks_m > 1 ? n_blocks_m : 1, m_pad) &&
                           canon_m.canon == m_pad;
    if (glqh_launch_e8_partial(x_rht, B, sg.q, sg.n, table1, table2 ? table2 : table1,
                               table2 ? n_entries2 : 65536, m_pad, n_pad, ks, part, st, canon_out ? sg.scale : nullptr,
                               folded))
        return 1;
    if (canon_out) {
        const float *pt[1] = {part};
        const void *sus[1] = {su_f16};
        void *ys[1] = {y};
        const float sc[1] = {1.0f};
        return glqh_launch_output_rht_group(pt, sus, ys, sc, &m_pad, &out_features, 1, y_dtype, y_stride, B,
                                            ks * sg.n, st);
    }
    glqh_ysrc src = {};
    src.nparts = sg.n;
    for (int s = 0; s < sg.n; ++s) src.scale[s] = sg.scale[s];
    src.part = part;
    src.part_sstride = B * m_pad;
    src.part_kstride = (int64_t)sg.n * B * m_pad;
    src.ksplit = ks;
    return glqh_launch_output_rht(src, su_f16, y, y_dtype, y_stride, B, out_features, m_pad, bm_meta_dev,
                                  blocks_m, n_blocks_m, 0, 0.0f, st);
}

// ---- encode side -------------------------------------------------------------------
int glqh_launch_e8_quantize(const float *x, const float *table, const float *norms, int64_t N, int K,
                            int64_t *idx_out, float *dec_out, hipStream_t stream);

extern "C" int glqh_e8_quantize(const float *x, const float *table_f32, const float *norms_f32, int64_t N,
                                int64_t n_entries, int64_t *idx_out, float *decoded_out, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(x && table_f32 && norms_f32 && idx_out, "e8 quantize: null pointer");
    GLQH_REQUIRE(N >= 1, "e8 quantize: N=%lld", (long long)N);
    GLQH_REQUIRE(n_entries >= 1 && n_entries <= 65536, "e8 quantize: %lld table rows (1..65536)",
                 (long long)n_entries);
    return glqh_launch_e8_quantize(x, table_f32, norms_f32, N, (int)n_entries, idx_out, decoded_out,
                                   (hipStream_t)stream);
}

int glqh_viterbi_init(void);
size_t glqh_viterbi_scratch_bytes(int K, int64_t n_tiles);
int glqh_launch_viterbi(const float *tiles, int64_t n_tiles, int K, uint8_t *scratch, int32_t *states,
                        float *hat, hipStream_t stream);

extern "C" size_t glqh_trellis_quantize_workspace_bytes(int K, int64_t n_tiles) {
    if (K < 1 || K > 4 || n_tiles < 1) return 0;
    glqh_init();
    return glqh_viterbi_scratch_bytes(K, n_tiles);
}

extern "C" int glqh_trellis_quantize_tiles(const float *tiles, int64_t n_tiles, int K, int32_t *states_out,
                                           float *hat_out, void *ws, size_t ws_bytes, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(tiles && states_out && hat_out, "trellis quantize: null pointer");
    GLQH_REQUIRE(K >= 1 && K <= 4, "trellis encoder supports K (bits/weight) 1-4, got %d", K);
    GLQH_REQUIRE(n_tiles >= 1, "trellis quantize: n_tiles=%lld", (long long)n_tiles);
    const size_t need = glqh_viterbi_scratch_bytes(K, n_tiles);
    GLQH_REQUIRE(ws && ws_bytes >= need, "trellis quantize: workspace of %zu bytes needed, got %zu", need, ws_bytes);
    return glqh_launch_viterbi(tiles, n_tiles, K, (uint8_t *)ws, states_out, hat_out, (hipStream_t)stream);
}

int glqh_launch_pack_states(const int32_t *states, int64_t m, int64_t n, int K, void *packed, hipStream_t stream);

extern "C" int glqh_trellis_pack_states(const int32_t *states, int64_t m, int64_t n, int K, void *packed_out,
                                        void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(states && packed_out, "trellis pack: null pointer");
    GLQH_REQUIRE(K >= 1 && K <= 4, "trellis kernel supports R (bits/weight) 1-4, got %d", K);
    GLQH_REQUIRE(glqh_trellis_kernel_supported(m, n), "trellis pack: m %% 32 and n %% 64 must be 0 (m=%lld, n=%lld)",
                 (long long)m, (long long)n);
    return glqh_launch_pack_states(states, m, n, K, packed_out, (hipStream_t)stream);
}

int glqh_launch_viterbi_acs_step(const float *cost, const void *x_f16, const float *lut, float *cost_out,
                                 int32_t *prev, int64_t B, int K, hipStream_t stream);

extern "C" int glqh_viterbi_acs_step(const float *cost, const void *x_f16, const float *lut_f32, float *cost_out,
                                     int32_t *prev_out, int64_t B, int K, void *stream) {
    GLQH_INIT();
    GLQH_REQUIRE(cost && x_f16 && lut_f32 && cost_out && prev_out, "viterbi step: null pointer");
    GLQH_REQUIRE(cost != cost_out, "viterbi step: cost_out must not alias cost");
    GLQH_REQUIRE(K >= 1 && K <= 4, "viterbi step supports K (bits/weight) 1-4, got %d", K);
    GLQH_REQUIRE(B >= 0 && B <= 65535, "viterbi step: %lld sequences (0..65535 per call)", (long long)B);
    if (B == 0) return 0;
    return glqh_launch_viterbi_acs_step(cost, x_f16, lut_f32, cost_out, prev_out, B, K, (hipStream_t)stream);
}
