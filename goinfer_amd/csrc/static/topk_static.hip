// topk_static.hip — the top-K of logits rows for callers that cannot allocate: code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc. Same kernels as rd_topk_rows (../kernels/topk.h, compiled into this file's own code
// object), same results; the scratch between the launches (per-chunk histograms and maxima, candidate lists and counts, the
// chunks' shares of Z) lives in one file-scope device array instead of call-scoped allocations. Inputs and outputs are device
// pointers the caller owns. This file is built by hipcc into librocmdecode_static.so, which librocmdecode.so opens when a device
// is opened (rd_device_open looks the scratch address up for that device then, outside any capture) or, failing that, on the
// first call of rd_topk_rows_static; nothing here calls hipMalloc, hipFree or any allocating routine.
//
// Every call on a GPU shares that GPU's array and finds the previous call's contents in it: the candidate counts, which must
// start at zero, are cleared by a fill kernel at the head of every call (a kernel, not hipMemsetAsync: memset nodes captured
// into a graph have replayed wrongly), everything else is written before it is read. Calls that overlap on one GPU race.
#include <hip/hip_runtime.h>
#include <mutex>
#include <stdarg.h>
#include <stdio.h>
#include "../kernels/topk.h"

#define RD_STATIC_MAX_ROWS 32
#define RD_STATIC_MAX_V 262144
#define RD_STATIC_MAX_CHUNKS (RD_STATIC_MAX_V / RD_TOPK_CHUNK) // 16
#define RD_STATIC_MAX_DEVICES 16

// The scratch, carved by offsets (all multiples of 256 bytes). 5.3 MB per GPU, held until the process ends.
constexpr size_t OFF_GHIST = 0;
constexpr size_t OFF_CAND_I = OFF_GHIST + sizeof(int) * RD_STATIC_MAX_ROWS * RD_STATIC_MAX_CHUNKS * RD_TOPK_BINS;
constexpr size_t OFF_CAND_V = OFF_CAND_I + sizeof(int) * RD_STATIC_MAX_ROWS * RD_TOPK_CAP;
constexpr size_t OFF_ZPART = OFF_CAND_V + sizeof(float) * RD_STATIC_MAX_ROWS * RD_TOPK_CAP;
constexpr size_t OFF_GMAX = OFF_ZPART + sizeof(double) * RD_STATIC_MAX_ROWS * RD_STATIC_MAX_CHUNKS;
constexpr size_t OFF_CCOUNT = OFF_GMAX + sizeof(uint32_t) * RD_STATIC_MAX_ROWS * RD_STATIC_MAX_CHUNKS;
constexpr size_t SCRATCH_BYTES = OFF_CCOUNT + 256;
static_assert(OFF_CAND_I % 256 == 0 && OFF_CAND_V % 256 == 0 && OFF_ZPART % 256 == 0 && OFF_GMAX % 256 == 0 && OFF_CCOUNT % 256 == 0, "256-byte aligned parts");

static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

// In host code `scratch` is only a handle for the runtime's symbol table, never an address: the device address of each GPU's own
// copy is asked for once per device, with that device current, and kept here.
static unsigned char *g_scratch_ptr[RD_STATIC_MAX_DEVICES];
static std::mutex g_mu;

static int fail(char *err, size_t err_len, int rc, const char *fmt, ...) {
    if (err && err_len) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(err, err_len, fmt, ap);
        va_end(ap);
    }
    return rc;
}

__global__ void rd_k_static_zero_counts(int *__restrict__ ccount, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) ccount[i] = 0;
}

// The device address of `device`'s copy of the scratch, looked up once (with that device current; the caller's current device is
// put back). The lookup may load this file's code object onto the device, so it belongs outside stream capture: rd_device_open does it.
static int scratch_base(int device, unsigned char **base, char *err, size_t err_len) {
    std::lock_guard<std::mutex> lock(g_mu);
    if (!g_scratch_ptr[device]) {
        int prev = -1;
        hipError_t e = hipGetDevice(&prev);
        if (e != hipSuccess) return fail(err, err_len, -2, "hipGetDevice: %s", hipGetErrorString(e));
        if (prev != device && (e = hipSetDevice(device)) != hipSuccess) return fail(err, err_len, -2, "hipSetDevice(%d): %s", device, hipGetErrorString(e));
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (prev != device) (void)hipSetDevice(prev);
        if (e != hipSuccess || !p) return fail(err, err_len, -2, "hipGetSymbolAddress(scratch) on device %d: %s", device, hipGetErrorString(e));
        g_scratch_ptr[device] = (unsigned char *)p;
    }
    *base = g_scratch_ptr[device];
    return 0;
}

// Called by rd_device_open for the device it opens: the one-time lookup, done before anybody captures.
extern "C" int rd_topk_static_prepare(int device, char *err, size_t err_len) {
    if (device < 0 || device >= RD_STATIC_MAX_DEVICES) return fail(err, err_len, -1, "rd_topk_rows_static: device %d outside 0..%d", device, RD_STATIC_MAX_DEVICES - 1);
    unsigned char *base;
    return scratch_base(device, &base, err, err_len);
}

// Return codes are rocmdecode.h's: 0 ok, -1 bad argument, -2 HIP error. The caller's current device is the same on return.
extern "C" int rd_topk_rows_static_impl(int device, void *stream_v, const float *logits, int rows, int V, int k, double temperature, int want_z, int *ids,
                                        float *vals, double *z, char *err, size_t err_len) {
    if (!logits || !ids || !vals || (want_z && !z)) return fail(err, err_len, -1, "rd_topk_rows_static: null pointer");
    if (device < 0 || device >= RD_STATIC_MAX_DEVICES) return fail(err, err_len, -1, "rd_topk_rows_static: device %d outside 0..%d", device, RD_STATIC_MAX_DEVICES - 1);
    if (rows < 1 || rows > RD_STATIC_MAX_ROWS || V < 1 || V > RD_STATIC_MAX_V)
        return fail(err, err_len, -1, "rd_topk_rows_static: %d rows of %d entries exceed the static scratch (at most %d rows of %d)", rows, V,
                    RD_STATIC_MAX_ROWS, RD_STATIC_MAX_V);
    if (k < 1 || k > RD_TOPK_MAX) return fail(err, err_len, -1, "rd_topk_rows_static: k=%d outside [1,%d]", k, RD_TOPK_MAX);
    if (k > V) k = V;
    unsigned char *base;
    int rc = scratch_base(device, &base, err, err_len);
    if (rc) return rc;
    int prev = -1;
    hipError_t e = hipGetDevice(&prev);
    if (e != hipSuccess) return fail(err, err_len, -2, "hipGetDevice: %s", hipGetErrorString(e));
    if (prev != device && (e = hipSetDevice(device)) != hipSuccess) return fail(err, err_len, -2, "hipSetDevice(%d): %s", device, hipGetErrorString(e));
    (void)hipGetLastError(); // an error an earlier, unrelated call left behind is not this call's
    hipStream_t stream = (hipStream_t)stream_v;
    const float invT = temperature > 0 ? (float)(1.0 / temperature) : 1.f; // backend/cuda/topk.go:74-77
    double *zo = want_z ? z : nullptr;
    if (V < 2 * RD_TOPK_CHUNK) { // a narrow row: one block reads it a few times, no scratch between launches
        hipLaunchKernelGGL(rd_k_topk_rows, dim3(rows), dim3(RD_TOPK_THREADS), 0, stream, logits, V, k, invT, (const float *)nullptr, ids, vals, zo);
    } else {
        int *ghist = (int *)(base + OFF_GHIST), *cand_i = (int *)(base + OFF_CAND_I), *ccount = (int *)(base + OFF_CCOUNT);
        float *cand_v = (float *)(base + OFF_CAND_V);
        double *zpart = (double *)(base + OFF_ZPART);
        uint32_t *gmax = (uint32_t *)(base + OFF_GMAX);
        const unsigned chunks = (unsigned)((V + RD_TOPK_CHUNK - 1) / RD_TOPK_CHUNK);
        hipLaunchKernelGGL(rd_k_static_zero_counts, dim3(1), dim3(64), 0, stream, ccount, RD_STATIC_MAX_ROWS);
        hipLaunchKernelGGL(rd_k_topk_hist, dim3(chunks, rows), dim3(1024), 0, stream, logits, V, ghist, gmax);
        hipLaunchKernelGGL(rd_k_topk_pick, dim3(chunks, rows), dim3(1024), 0, stream, logits, V, k, invT, (const float *)nullptr, (const int *)ghist,
                           (const uint32_t *)gmax, cand_v, cand_i, ccount, want_z ? zpart : (double *)nullptr);
        hipLaunchKernelGGL(rd_k_topk_finish, dim3(rows), dim3(RD_TOPK_THREADS), 0, stream, logits, V, k, (int)chunks, (const float *)cand_v,
                           (const int *)cand_i, ccount, (const double *)zpart, ids, vals, zo);
    }
    e = hipGetLastError();
    if (prev != device) (void)hipSetDevice(prev);
    if (e != hipSuccess) return fail(err, err_len, -2, "rd_topk_rows_static: launch failed: %s", hipGetErrorString(e));
    return 0;
}
