// Error reporting, ABI version, topology tables and the initial span nodes.
#include "hsa_common.h"

#include <stdarg.h>
#include <stdio.h>

namespace hsa {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

static thread_local LaunchEvents g_launch_events;
void set_launch_events(hipEvent_t start, hipEvent_t stop) {
    g_launch_events.start = start;
    g_launch_events.stop = stop;
}
LaunchEvents take_launch_events() {
    LaunchEvents e = g_launch_events;
    g_launch_events = LaunchEvents();
    return e;
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return HSA_OK;
}

// ---- topology ---------------------------------------------------------------
// Closed forms of the "climb via the neighbour" construction:
//   idx[n,l]  = off_l + ((n >> l) ^ 1)
//   mask[n,l] = causal and bit l of n is 0 (the neighbour lies to the right)
//   gather[i] for node i = off_lv + j: the leaf range [(j^1) << lv, ((j^1)+1) << lv)
//   of its sibling and its own level lv; -1 for the root and, when causal, for
//   nodes whose sibling lies to the left (j odd).
__host__ __device__ inline void topo_forward_entry(int N, int causal, int n, int l, int32_t *idx,
                                                   uint8_t *mask, int L) {
    if (idx) idx[(size_t)n * L + l] = level_offset(N, l) + ((n >> l) ^ 1);
    if (mask) mask[(size_t)n * L + l] = (causal && ((n >> l) & 1) == 0) ? 1 : 0;
}

__host__ __device__ inline void topo_gather_entry(int N, int causal, int i, int32_t *gather) {
    // locate the level of node i: level lv spans [off_lv, off_lv + (N >> lv))
    int lv = 0, start = 0, count = N;
    while (i >= start + count) { start += count; count >>= 1; ++lv; }
    int j = i - start;
    int32_t *g = gather + (size_t)i * 3;
    bool root = (i == 2 * N - 2);
    if (root || (causal && (j & 1))) {
        g[0] = g[1] = g[2] = -1;
    } else {
        int s = j ^ 1;
        g[0] = s << lv;
        g[1] = (s + 1) << lv;
        g[2] = lv;
    }
}

__global__ void topology_kernel(int N, int L, int causal, int32_t *idx, uint8_t *mask,
                                int32_t *gather) {
    long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long n_fwd = (long)N * L;
    if (t < n_fwd) topo_forward_entry(N, causal, (int)(t / L), (int)(t % L), idx, mask, L);
    if (gather && t < 2L * N - 1) topo_gather_entry(N, causal, (int)t, gather);
}

// ---- initial span nodes -------------------------------------------------------
// One thread per (batch, channel-vector, leaf pair chain): a thread owns 2^T
// consecutive leaves of one channel and reduces them level by level in
// registers, rounding to the element type at each level like the reference's
// per-level `0.5*a + 0.5*b`.  Levels above T are finished by a second pass that
// reads the level-T nodes back (tiny).
template <typename T>
__global__ void span_y_kernel(const typename T::storage *__restrict__ x, size_t x_bs, int src_rows,
                              typename T::storage *__restrict__ y, size_t y_bs, int N, int C,
                              int lvl0, int nlev, int B) {
    // src: rows of level lvl0 (lvl0 == 0: x itself; else inside y).  Each thread
    // takes 2^nlev consecutive source rows of one channel; the last group of a level
    // whose row count is not a multiple of that is partly filled.
    const int span = 1 << nlev;
    const int groups = (src_rows + span - 1) >> nlev;
    size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t total = (size_t)B * groups * C;
    if (t >= total) return;
    int c = (int)(t % C);
    int g = (int)((t / C) % groups);
    int b = (int)(t / ((size_t)C * groups));
    const typename T::storage *src =
        (lvl0 == 0) ? x + (size_t)b * x_bs : y + (size_t)b * y_bs + (size_t)span_level_start(N, lvl0) * C;
    float v[32];
#pragma unroll
    for (int i = 0; i < 32; ++i)
        if (i < span) {
            const int row = g * span + i;
            v[i] = row < src_rows ? to_float<T>(src[(size_t)row * C + c]) : 0.f;
        }
    int cnt = span;
#pragma unroll
    for (int s = 1; s <= 5; ++s) {
        if (s <= nlev) {
            cnt >>= 1;
            int lvl = lvl0 + s;
            const int lvl_rows = src_rows >> s;
            typename T::storage *dst = y + (size_t)b * y_bs + (size_t)span_level_start(N, lvl) * C;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                if (i < cnt) {
                    // each half is rounded to the element type first (only matters for
                    // fp16 values that become subnormal), then the sum rounds once
                    float ha = to_float<T>(from_float<T>(0.5f * v[2 * i]));
                    float hb = to_float<T>(from_float<T>(0.5f * v[2 * i + 1]));
                    float m = ha + hb;
                    typename T::storage r = from_float<T>(m);
                    const int row = g * cnt + i;
                    if (row < lvl_rows) dst[(size_t)row * C + c] = r;
                    v[i] = to_float<T>(r);
                }
            }
        }
    }
}

template <typename T>
static int span_y_launch(const void *x, void *y, int B, int N, int C, hipStream_t st) {
    const int L = span_levels(N);
    const size_t y_rows = (size_t)span_rows(N);
    int lvl = 0, rows = N;
    while (lvl < L) {
        int nlev = L - lvl < 5 ? L - lvl : 5;
        size_t total = (size_t)B * ((rows + (1 << nlev) - 1) >> nlev) * C;
        int threads = 256;
        unsigned blocks = (unsigned)((total + threads - 1) / threads);
        span_y_kernel<T><<<blocks, threads, 0, st>>>((const typename T::storage *)x, (size_t)N * C, rows,
                                                     (typename T::storage *)y, y_rows * C, N,
                                                     C, lvl, nlev, B);
        lvl += nlev;
        rows >>= nlev;
    }
    return check_launch("span_y_kernel");
}

}  // namespace hsa

extern "C" {

int hsa_abi_version(void) { return 1; }

const char *hsa_last_error(void) { return hsa::g_err; }

int hsa_topology_host(int N, int causal, int32_t *idx, uint8_t *mask, int32_t *gather) {
    HSA_REQUIRE(N >= 1 && hsa::ilog2_exact(N) >= 0, "seq_len must be power of 2 (got %d)", N);
    const int L = hsa::ilog2_exact(N);
    if (idx || mask)
        for (int n = 0; n < N; ++n)
            for (int l = 0; l < L; ++l) hsa::topo_forward_entry(N, causal, n, l, idx, mask, L);
    if (gather)
        for (int i = 0; i < 2 * N - 1; ++i) hsa::topo_gather_entry(N, causal, i, gather);
    return HSA_OK;
}

int hsa_topology_device(int N, int causal, int32_t *idx, uint8_t *mask, int32_t *gather,
                        void *stream) {
    HSA_REQUIRE(N >= 1 && hsa::ilog2_exact(N) >= 0, "seq_len must be power of 2 (got %d)", N);
    HSA_REQUIRE(N <= (1 << 26), "seq_len %d too large", N);
    const int L = hsa::ilog2_exact(N);
    long work = (long)N * L;
    if (gather && work < 2L * N - 1) work = 2L * N - 1;
    if (!idx && !mask) work = gather ? 2L * N - 1 : 0;
    if (work == 0) return HSA_OK;
    // the forward part of the kernel writes both idx and mask entries under t < N*L
    int threads = 256;
    unsigned blocks = (unsigned)((work + threads - 1) / threads);
    hsa::topology_kernel<<<blocks, threads, 0, (hipStream_t)stream>>>(N, L, causal, idx, mask, gather);
    return hsa::check_launch("topology_kernel");
}

int hsa_span_input_y(const void *x, void *y, int B, int N, int C, int dtype, void *stream) {
    HSA_REQUIRE(x && y, "null pointer");
    HSA_REQUIRE(B >= 1 && C >= 1, "bad shape B=%d C=%d", B, C);
    HSA_REQUIRE(N >= 2 && N <= (1 << 26), "N must lie in [2, 2^26] (got %d)", N);
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case HSA_F32: return hsa::span_y_launch<hsa::F32>(x, y, B, N, C, st);
        case HSA_F16: return hsa::span_y_launch<hsa::F16>(x, y, B, N, C, st);
        case HSA_BF16: return hsa::span_y_launch<hsa::BF16>(x, y, B, N, C, st);
    }
    return hsa::fail(HSA_ERR_INVALID, "unknown dtype %d", dtype);
}

}  // extern "C"
