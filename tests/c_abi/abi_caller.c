/* A caller of the library that knows nothing but its C header and the HIP runtime: plain C,
 * hipMalloc'd buffers, the null stream.  Test infrastructure: tests/test_c_caller_gpu.py writes
 * the operands as raw little-endian files, runs this program and checks what it writes back
 * against the oracle and against the Python wrappers (same library, so the same bits).
 *
 *   abi_caller lm2exp DIR R I J K            a.bin b.bin          -> c.bin
 *   abi_caller lt2exp DIR R S I J K MODE     w.bin a.bin b.bin    -> c.bin
 *   abi_caller vmax   DIR N                  x.bin                -> val.bin idx.bin
 *   abi_caller matmax DIR M N AXIS           x.bin                -> y.bin
 */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "triturus_hip.h"

#define CHECK_HIP(call)                                                                  \
    do {                                                                                 \
        hipError_t e_ = (call);                                                          \
        if (e_ != hipSuccess) {                                                          \
            fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));                   \
            exit(2);                                                                     \
        }                                                                                \
    } while (0)

#define CHECK_TRT(call)                                                                  \
    do {                                                                                 \
        int s_ = (call);                                                                 \
        if (s_ != 0) {                                                                   \
            fprintf(stderr, "%s: status %d (%s)\n", #call, s_, trt_error_string(s_));    \
            exit(3);                                                                     \
        }                                                                                \
    } while (0)

static void path_of(char *buf, size_t cap, const char *dir, const char *name) {
    snprintf(buf, cap, "%s/%s", dir, name);
}

/* file -> device buffer of `bytes` bytes */
static void *upload(const char *dir, const char *name, size_t bytes) {
    char path[4096];
    path_of(path, sizeof path, dir, name);
    FILE *f = fopen(path, "rb");
    if (!f) { perror(path); exit(4); }
    void *host = malloc(bytes ? bytes : 1);
    if (fread(host, 1, bytes, f) != bytes) { fprintf(stderr, "%s: short read\n", path); exit(4); }
    fclose(f);
    void *dev = NULL;
    CHECK_HIP(hipMalloc(&dev, bytes ? bytes : 1));
    CHECK_HIP(hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice));
    free(host);
    return dev;
}

/* device buffer -> file */
static void download(const char *dir, const char *name, const void *dev, size_t bytes) {
    char path[4096];
    path_of(path, sizeof path, dir, name);
    void *host = malloc(bytes ? bytes : 1);
    CHECK_HIP(hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost));
    FILE *f = fopen(path, "wb");
    if (!f) { perror(path); exit(4); }
    if (fwrite(host, 1, bytes, f) != bytes) { fprintf(stderr, "%s: short write\n", path); exit(4); }
    fclose(f);
    free(host);
}

static void *device_buffer(size_t bytes) {
    void *dev = NULL;
    CHECK_HIP(hipMalloc(&dev, bytes ? bytes : 1));
    return dev;
}

int main(int argc, char **argv) {
    if (argc < 4) { fprintf(stderr, "usage: abi_caller OP DIR SIZES...\n"); return 1; }
    const char *op = argv[1], *dir = argv[2];
    int64_t d[6] = {0, 0, 0, 0, 0, 0};
    for (int i = 3; i < argc && i < 9; ++i) d[i - 3] = strtoll(argv[i], NULL, 10);
    if (trt_version() != TRT_ABI_VERSION) { fprintf(stderr, "library / header version mismatch\n"); return 1; }
    CHECK_HIP(hipSetDevice(0));

    if (strcmp(op, "lm2exp") == 0) {
        const int64_t R = d[0], I = d[1], J = d[2], K = d[3];
        float *a = upload(dir, "a.bin", (size_t)(R * I * J) * 4), *b = upload(dir, "b.bin", (size_t)(R * J * K) * 4);
        float *c = device_buffer((size_t)(R * I * K) * 4);
        const int64_t sa[3] = {I * J, J, 1}, sb[3] = {J * K, K, 1}, sc[3] = {I * K, K, 1};
        const size_t ws_bytes = trt_lm2exp_workspace_bytes(R, I, J, K, 0, 0);
        void *ws = ws_bytes ? device_buffer(ws_bytes) : NULL;
        CHECK_TRT(trt_lm2exp_f32(a, b, c, R, I, J, K, sa, sb, sc, 0, 0, ws, ws_bytes, NULL));
        CHECK_HIP(hipDeviceSynchronize());
        download(dir, "c.bin", c, (size_t)(R * I * K) * 4);
    } else if (strcmp(op, "lt2exp") == 0) {
        const int64_t R = d[0], S = d[1], I = d[2], J = d[3], K = d[4];
        const int mode = (int)d[5];
        float *w = upload(dir, "w.bin", (size_t)(R * S * I * J) * 4);
        float *a = upload(dir, "a.bin", (size_t)(R * I * K) * 4), *b = upload(dir, "b.bin", (size_t)(R * J * K) * 4);
        float *c = device_buffer((size_t)(R * S * K) * 4);
        const int64_t sw[3] = {S * I * J, I * J, 1}, sa[3] = {I * K, K, 1}, sb[3] = {J * K, K, 1}, sc[3] = {S * K, K, 1};
        const size_t ws_bytes = trt_lt2exp_workspace_bytes(R, S, I, J, K, mode);
        void *ws = ws_bytes ? device_buffer(ws_bytes) : NULL;
        CHECK_TRT(trt_lt2exp_f32(w, a, b, c, R, S, I, J, K, sw, sa, sb, sc, mode, 0, ws, ws_bytes, NULL));
        CHECK_HIP(hipDeviceSynchronize());
        download(dir, "c.bin", c, (size_t)(R * S * K) * 4);
    } else if (strcmp(op, "vmax") == 0) {
        const int64_t n = d[0];
        float *x = upload(dir, "x.bin", (size_t)n * 4);
        float *val = device_buffer(4);
        int64_t *idx = device_buffer(8);
        size_t ws_bytes = trt_vmax_workspace_bytes(n, TRT_F32);
        void *ws = NULL;
        if (ws_bytes) {
            if (ws_bytes < TRT_MAX_TICKET_BYTES) ws_bytes = TRT_MAX_TICKET_BYTES;
            ws = device_buffer(ws_bytes);
            CHECK_TRT(trt_max_workspace_init(ws, ws_bytes, NULL));
        }
        /* twice: every call leaves the arrival counters idle for the next */
        CHECK_TRT(trt_vmax(x, n, TRT_F32, val, idx, ws, ws_bytes, NULL));
        CHECK_TRT(trt_vmax(x, n, TRT_F32, val, idx, ws, ws_bytes, NULL));
        CHECK_HIP(hipDeviceSynchronize());
        download(dir, "val.bin", val, 4);
        download(dir, "idx.bin", idx, 8);
    } else if (strcmp(op, "matmax") == 0) {
        const int64_t m = d[0], n = d[1];
        const int axis = (int)d[2];
        float *x = upload(dir, "x.bin", (size_t)(m * n) * 4);
        const int64_t len = axis == 0 ? n : m;
        float *y = device_buffer((size_t)len * 4);
        size_t ws_bytes = trt_matmax_workspace_bytes(m, n, axis, TRT_F32);
        void *ws = NULL;
        if (ws_bytes) {
            if (ws_bytes < TRT_MAX_TICKET_BYTES) ws_bytes = TRT_MAX_TICKET_BYTES;
            ws = device_buffer(ws_bytes);
            CHECK_TRT(trt_max_workspace_init(ws, ws_bytes, NULL));
        }
        CHECK_TRT(trt_matmax(x, y, m, n, axis, TRT_F32, ws, ws_bytes, NULL));
        CHECK_HIP(hipDeviceSynchronize());
        download(dir, "y.bin", y, (size_t)len * 4);
    } else {
        fprintf(stderr, "unknown op %s\n", op);
        return 1;
    }
    return 0;
}
